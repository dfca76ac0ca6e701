// Implicit-GEMM convolution on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16),
// 2-D, 3x3, stride 1, dilation 1, channels-first tensors in and out.
//
// Forward / dgrad kernel (one kernel, two weight preparations):
//   GEMM view   Y[co][pixel] = sum_{tap, ci} Wt[tap][co][ci] * X[ci][pixel + tap]
//   MFMA roles  A = weights (M = 32 output channels, K = 16 input channels),
//               B = input pixels (K = 16 channels, N = 32 consecutive pixels of a row),
//               so an accumulator lane owns one pixel and 16 output channels and the
//               stores run along W of the channels-first output.
//   Workgroup   512 threads = 8 wavefronts; output tile 16 rows x 64 columns x MT
//               output channels; wavefront w owns rows 4*(w/2).., columns 32*(w%2)..
//   LDS         the whole prepared weight block of the workgroup's output-channel
//               tile stays resident (<= 72 KiB); the input tile is streamed in
//               stages of 16 input channels, double buffered (2 x 40.5 KiB).
//               Input pixels are stored "8 channels per 16-byte slot" so that a B
//               fragment is one ds_read_b128 per lane; the channels-first global
//               rows are transposed in registers on the way in.
//   Schedule    persistent workgroups (one per CU) walk a contiguous, XCD-local
//               range of tiles; the global loads of stage s+1 are issued before the
//               MFMAs of stage s and written to LDS after them (one barrier/stage).
//   dgrad       the same kernel on the output gradient with virtual zero padding
//               k-1-p and the weights flipped and transposed by the preparation.
#include "conv_common.h"

namespace {

using jg::ConvGeom;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));

constexpr int KH = 3, KW = 3, TAPS = KH * KW;
constexpr int TH = 16, TW = 64;            // output tile of a workgroup
constexpr int WAVES = 8, THREADS = WAVES * 64;
constexpr int WROWS = 4;                   // output rows per wavefront
constexpr int IN_ROWS = TH + KH - 1;       // 18
constexpr int QUADS = (TW + KW - 1 + 3) / 4;  // 17 quads of 4 pixels cover 66 columns
constexpr int QP = 18;                     // quad slots per pixel-phase group (bank spread)
constexpr int ROW_SLOTS = 4 * QP;          // 16-byte slots per LDS row
constexpr int CK = 16;                     // input channels per stage
constexpr int STAGE_SLOTS = 2 * IN_ROWS * ROW_SLOTS;  // [kg][row][slot]
constexpr int STAGE_BYTES = STAGE_SLOTS * 16;         // 41472
constexpr int TASKS = 2 * IN_ROWS * QUADS;            // 612 (8 channels x 4 pixels each)
constexpr int TASK_ROUNDS = (TASKS + THREADS - 1) / THREADS;  // 2

__device__ __forceinline__ int in_slot(int row, int col) {
  return row * ROW_SLOTS + (col & 3) * QP + (col >> 2);
}

struct FwdParams {
  const uint16_t* x;    // (N, K, Hin, Win) bf16: the tensor that is convolved
  const u32x4* wprep;   // prepared weights, [m_tile][tap][c16][kg][MT][8]
  const uint16_t* bias; // (M,) or NULL
  uint16_t* y;          // (N, M, Hout, Wout)
  int N, K, M;          // batch, contraction channels, produced channels
  int Hin, Win, Hout, Wout;
  int pad_h, pad_w;     // virtual zero padding of x
  int tiles_h, tiles_w;
  int total_tiles;      // N * tiles_h * tiles_w
  int nc16;             // K / 16
};

// ---------------------------------------------------------------- weight prep
// dst[((mt*TAPS + tap)*nc16 + c16)*2 + kg][m_local][8 k] (bf16), MT produced
// channels per m-tile. transposed = 0: A[m][k] = w[m][k][kh][kw] (forward);
// transposed = 1: A[m][k] = w[k][m][KH-1-kh][KW-1-kw] (input gradient).
__global__ __launch_bounds__(256) void prep_weights_kernel(uint16_t* __restrict__ dst,
                                                           const uint16_t* __restrict__ w,
                                                           int M, int K, int MT, int transposed) {
  const int total = M * K * TAPS;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
    int e = i & 7;
    int r = i >> 3;
    int ml = r % MT; r /= MT;
    int kg = r & 1; r >>= 1;
    const int nc16 = K / CK;
    int c16 = r % nc16; r /= nc16;
    int tap = r % TAPS;
    int mt = r / TAPS;
    const int m = mt * MT + ml;
    const int k = c16 * CK + kg * 8 + e;
    const int kh = tap / KW, kw = tap % KW;
    uint16_t v;
    if (!transposed)
      v = w[((m * K + k) * KH + kh) * KW + kw];
    else
      v = w[((k * M + m) * KH + (KH - 1 - kh)) * KW + (KW - 1 - kw)];
    dst[i] = v;
  }
}

// ------------------------------------------------------------ forward kernel
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// EVEN: Win, pad_w and the plane size are even and x is 4-byte aligned, so every
// pixel pair of a task is one aligned dword that is either wholly inside or wholly
// outside the tensor. Otherwise the prefetch falls back to 2-byte loads.
template <int MT, bool EVEN>  // MT = produced channels per workgroup: 32 or 64
__global__ __launch_bounds__(THREADS) void conv3x3_mfma_kernel(FwdParams p) {
  constexpr int CB = MT / 32;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int w_slots = TAPS * p.nc16 * 2 * MT;  // 16-byte slots of the weight block
  u32x4* lds_w = reinterpret_cast<u32x4*>(smem);
  u32x4* lds_in = lds_w + w_slots;  // two stages
  float* lds_bias = reinterpret_cast<float*>(lds_in + 2 * STAGE_SLOTS);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int wrow0 = (wave >> 1) * WROWS, wcol0 = (wave & 1) * 32;
  const int mt = blockIdx.y;

  // ---- tile schedule: XCD x (= blockIdx.x % 8) owns a contiguous range
  const int G = gridDim.x;
  const int xcd = blockIdx.x & 7, slot_in_xcd = blockIdx.x >> 3;
  const int wg_per_xcd = (G + 7) >> 3;
  const int per_xcd = (p.total_tiles + 7) >> 3;
  const int t_begin = xcd * per_xcd;
  int t_end = t_begin + per_xcd;
  if (t_end > p.total_tiles) t_end = p.total_tiles;
  const int t_first = t_begin + slot_in_xcd;
  if (t_first >= t_end) return;

  // ---- resident weights and bias
  {
    const u32x4* src = p.wprep + (size_t)mt * w_slots;
    for (int i = tid; i < w_slots; i += THREADS) lds_w[i] = src[i];
    if (tid < MT) lds_bias[tid] = p.bias != nullptr ? jg::bf16_to_f32(p.bias[mt * MT + tid]) : 0.0f;
  }

  // ---- prefetch bookkeeping. A task = 8 channels x 4 pixels of one input row.
  const size_t plane = (size_t)p.Hin * p.Win;
  const uint32_t plane_b = (uint32_t)(plane * 2);
  int t_row[TASK_ROUNDS], t_col[TASK_ROUNDS];
  uint32_t t_off[TASK_ROUNDS];  // byte offset of the task inside the stage window
  int t_lds[TASK_ROUNDS];       // slot of pixel 0 of the task inside a stage buffer
#pragma unroll
  for (int rd = 0; rd < TASK_ROUNDS; ++rd) {
    const int q = tid + rd * THREADS;
    const int quad = q % QUADS;
    const int rr = q / QUADS;  // = g8 * IN_ROWS + row
    t_row[rd] = rr % IN_ROWS;
    t_col[rd] = quad * 4;
    const int g8 = rr / IN_ROWS;
    t_off[rd] = (uint32_t)(((size_t)g8 * 8 * plane + (size_t)t_row[rd] * p.Win + t_col[rd]) * 2);
    t_lds[rd] = rr * ROW_SLOTS + quad;
  }
  uint32_t stg[TASK_ROUNDS][8][2];

  auto issue_loads = [&](int tile, int c16) {
    const int tw = tile % p.tiles_w;
    const int tq = tile / p.tiles_w;
    const int th = tq % p.tiles_h;
    const int n = tq / p.tiles_h;
    const int ih0 = th * TH - p.pad_h, iw0 = tw * TW - p.pad_w;
    // wave-uniform origin of the stage window (lies before the tensor where padded)
    const char* origin = reinterpret_cast<const char*>(p.x) +
                         2 * ((ptrdiff_t)(((size_t)n * p.K + (size_t)c16 * CK) * plane) +
                              (ptrdiff_t)ih0 * p.Win + iw0);
    const bool interior =
        ih0 >= 0 && ih0 + IN_ROWS <= p.Hin && iw0 >= 0 && iw0 + QUADS * 4 <= p.Win;
#pragma unroll
    for (int rd = 0; rd < TASK_ROUNDS; ++rd) {
      if (tid + rd * THREADS < TASKS) {
        const char* a = origin + t_off[rd];
        if (EVEN && interior) {
#pragma unroll
          for (int c = 0; c < 8; ++c) {
            const u32x2_a4 v = *reinterpret_cast<const u32x2_a4*>(a + (size_t)c * plane_b);
            stg[rd][c][0] = v.x;
            stg[rd][c][1] = v.y;
          }
        } else if (EVEN) {
          const int ih = ih0 + t_row[rd], iw = iw0 + t_col[rd];
          const bool row_ok = (ih >= 0) && (ih < p.Hin);
          const bool lo_ok = row_ok && iw >= 0 && iw + 2 <= p.Win;
          const bool hi_ok = row_ok && iw + 2 >= 0 && iw + 4 <= p.Win;
#pragma unroll
          for (int c = 0; c < 8; ++c) {
            stg[rd][c][0] = lo_ok ? *reinterpret_cast<const uint32_t*>(a + (size_t)c * plane_b) : 0u;
            stg[rd][c][1] = hi_ok ? *reinterpret_cast<const uint32_t*>(a + (size_t)c * plane_b + 4) : 0u;
          }
        } else {
          const int ih = ih0 + t_row[rd], iw = iw0 + t_col[rd];
          const bool row_ok = (ih >= 0) && (ih < p.Hin);
#pragma unroll
          for (int c = 0; c < 8; ++c) {
            const uint16_t* e = reinterpret_cast<const uint16_t*>(a + (size_t)c * plane_b);
            uint32_t v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
              v[k] = (row_ok && iw + k >= 0 && iw + k < p.Win) ? (uint32_t)e[k] : 0u;
            stg[rd][c][0] = v[0] | (v[1] << 16);
            stg[rd][c][1] = v[2] | (v[3] << 16);
          }
        }
      }
    }
  };

  auto store_stage = [&](int buf) {
    u32x4* dst = lds_in + buf * STAGE_SLOTS;
#pragma unroll
    for (int rd = 0; rd < TASK_ROUNDS; ++rd) {
      if (tid + rd * THREADS < TASKS) {
        u32x4* row_base = dst + t_lds[rd];
#pragma unroll
        for (int px = 0; px < 4; ++px) {
          // pixel px of the quad: low (px even) or high (px odd) half of dword px/2
          const uint32_t sel = (px & 1) ? 0x07060302u : 0x05040100u;
          u32x4 v;
          v.x = __builtin_amdgcn_perm(stg[rd][1][px >> 1], stg[rd][0][px >> 1], sel);
          v.y = __builtin_amdgcn_perm(stg[rd][3][px >> 1], stg[rd][2][px >> 1], sel);
          v.z = __builtin_amdgcn_perm(stg[rd][5][px >> 1], stg[rd][4][px >> 1], sel);
          v.w = __builtin_amdgcn_perm(stg[rd][7][px >> 1], stg[rd][6][px >> 1], sel);
          row_base[px * QP] = v;
        }
      }
    }
  };

  f32x16 acc[CB][WROWS];

  auto compute_stage = [&](int buf, int c16) {
    const u32x4* in = lds_in + buf * STAGE_SLOTS + kg * (IN_ROWS * ROW_SLOTS);
    const u32x4* wt = lds_w + ((size_t)c16 * 2 + kg) * MT + ln;
#pragma unroll 1
    for (int kw = 0; kw < KW; ++kw) {
      bf16x8 a[KH][CB];
#pragma unroll
      for (int kh = 0; kh < KH; ++kh)
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
          u32x4 t = wt[(size_t)(kh * KW + kw) * p.nc16 * 2 * MT + cb * 32];
          a[kh][cb] = __builtin_bit_cast(bf16x8, t);
        }
      const int col = wcol0 + ln + kw;
      const u32x4* inb = in + wrow0 * ROW_SLOTS + (col & 3) * QP + (col >> 2);
#pragma unroll
      for (int rho = 0; rho < WROWS + KH - 1; ++rho) {
        u32x4 t = inb[rho * ROW_SLOTS];
        const bf16x8 b = __builtin_bit_cast(bf16x8, t);
#pragma unroll
        for (int kh = 0; kh < KH; ++kh) {
          const int r = rho - kh;
          if (r >= 0 && r < WROWS) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
              acc[cb][r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kh][cb], b, acc[cb][r], 0, 0, 0);
          }
        }
      }
    }
  };

  // Accumulator lane (ln, kg), register i of block cb: produced channel
  // cb*32 + 8*(i/4) + 4*kg + i%4, pixel column wcol0 + ln.
  auto init_acc = [&]() {
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 bv = *reinterpret_cast<const f32x4*>(lds_bias + cb * 32 + 8 * j + 4 * kg);
#pragma unroll
        for (int r = 0; r < WROWS; ++r) {
          acc[cb][r][4 * j + 0] = bv.x;
          acc[cb][r][4 * j + 1] = bv.y;
          acc[cb][r][4 * j + 2] = bv.z;
          acc[cb][r][4 * j + 3] = bv.w;
        }
      }
  };

  const size_t plane_o = (size_t)p.Hout * p.Wout;
  auto epilogue = [&](int tile) {
    const int tw = tile % p.tiles_w;
    const int tq = tile / p.tiles_w;
    const int th = tq % p.tiles_h;
    const int n = tq / p.tiles_h;
    const int ow = tw * TW + wcol0 + ln;
    char* ybase = reinterpret_cast<char*>(p.y) + 2 * (((size_t)n * p.M + (size_t)mt * MT) * plane_o);
#pragma unroll
    for (int r = 0; r < WROWS; ++r) {
      const int oh = th * TH + wrow0 + r;
      if (oh < p.Hout && ow < p.Wout) {
        const uint32_t voff = (uint32_t)(2 * ((size_t)(4 * kg) * plane_o + (size_t)oh * p.Wout + ow));
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
          for (int i = 0; i < 16; i += 2) {
            f32x2 v2 = {acc[cb][r][i], acc[cb][r][i + 1]};
            const bf16x2 h2 = __builtin_convertvector(v2, bf16x2);
            const int m0 = cb * 32 + 8 * (i >> 2) + (i & 3);
            *reinterpret_cast<__bf16*>(ybase + (size_t)m0 * plane_o * 2 + voff) = h2.x;
            *reinterpret_cast<__bf16*>(ybase + (size_t)(m0 + 1) * plane_o * 2 + voff) = h2.y;
          }
      }
    }
  };

  // ---- main loop
  int buf = 0;
  issue_loads(t_first, 0);
  store_stage(0);
  __syncthreads();
  for (int tile = t_first; tile < t_end; tile += wg_per_xcd) {
    init_acc();
    for (int c16 = 0; c16 < p.nc16; ++c16) {
      int nt = tile, nc = c16 + 1;
      if (nc == p.nc16) {
        nc = 0;
        nt = tile + wg_per_xcd;
      }
      const bool has_next = nt < t_end;
      if (has_next) issue_loads(nt, nc);
      compute_stage(buf, c16);
      if (has_next) store_stage(buf ^ 1);
      __syncthreads();
      buf ^= 1;
    }
    epilogue(tile);
  }
}

// ----------------------------------------------------------------- host side
int cu_count() {
  static int cached = 0;
  if (cached) return cached;
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
    n = 256;
  cached = n;
  return n;
}

bool shape_ok(int K, int M, const ConvGeom& g) {
  if (g.in[0] != 1 || g.k[0] != 1) return false;  // 2-D only
  if (g.k[1] != KH || g.k[2] != KW) return false;
  if (g.s[1] != 1 || g.s[2] != 1 || g.d[1] != 1 || g.d[2] != 1) return false;
  if (K % CK != 0 || M % 32 != 0) return false;
  const int MT = (M % 64 == 0) ? 64 : 32;
  const size_t lds = (size_t)TAPS * (K / CK) * 2 * MT * 16 + 2 * (size_t)STAGE_BYTES + MT * 4;
  if (lds > 160 * 1024) return false;
  // per-lane byte offsets inside one (batch entry, channel tile) are 32-bit
  const size_t in_plane = (size_t)g.in[1] * g.in[2], out_plane = (size_t)g.out[1] * g.out[2];
  const size_t big = in_plane > out_plane ? in_plane : out_plane;
  return big * 2 * 72 < (1ull << 31);
}

size_t prep_bytes(int K, int M) { return (size_t)K * M * TAPS * sizeof(uint16_t); }

int launch_conv(const uint16_t* x, const uint16_t* w, const uint16_t* bias, uint16_t* y, int N,
                int K, int M, int Hin, int Win, int Hout, int Wout, int pad_h, int pad_w,
                int transposed, void* ws, size_t ws_bytes, hipStream_t s, const char* who) {
  if (ws == nullptr || ws_bytes < prep_bytes(K, M))
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes, prep_bytes(K, M));
  JG_REQUIRE((reinterpret_cast<uintptr_t>(ws) & 15) == 0, "%s: workspace must be 16-byte aligned",
             who);
  const int MT = (M % 64 == 0) ? 64 : 32;
  uint16_t* wprep = static_cast<uint16_t*>(ws);
  const int total_w = M * K * TAPS;
  prep_weights_kernel<<<(total_w + 255) / 256, 256, 0, s>>>(wprep, w, M, K, MT, transposed);
  JG_CHECK_LAUNCH(who);

  FwdParams p;
  p.x = x; p.wprep = reinterpret_cast<const u32x4*>(wprep); p.bias = bias; p.y = y;
  p.N = N; p.K = K; p.M = M;
  p.Hin = Hin; p.Win = Win; p.Hout = Hout; p.Wout = Wout;
  p.pad_h = pad_h; p.pad_w = pad_w;
  p.tiles_h = (Hout + TH - 1) / TH;
  p.tiles_w = (Wout + TW - 1) / TW;
  const long long tiles = (long long)N * p.tiles_h * p.tiles_w;
  JG_REQUIRE(tiles < (1ll << 30), "%s: too many tiles", who);
  p.total_tiles = (int)tiles;
  p.nc16 = K / CK;
  if (tiles == 0) return JG_OK;
  const size_t lds = (size_t)TAPS * p.nc16 * 2 * MT * 16 + 2 * (size_t)STAGE_BYTES + MT * 4;
  int wgs = cu_count();
  if (wgs > tiles) wgs = (int)tiles;
  wgs = (wgs + 7) & ~7;  // whole XCD rounds
  dim3 grid((unsigned)wgs, (unsigned)(M / MT), 1);
  const bool even = (Win % 2 == 0) && (pad_w % 2 == 0) && ((reinterpret_cast<uintptr_t>(x) & 3) == 0);
  void (*kern)(FwdParams) = nullptr;
  if (MT == 64) kern = even ? &conv3x3_mfma_kernel<64, true> : &conv3x3_mfma_kernel<64, false>;
  else kern = even ? &conv3x3_mfma_kernel<32, true> : &conv3x3_mfma_kernel<32, false>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", who, lds);
  kern<<<grid, THREADS, lds, s>>>(p);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

}  // namespace

namespace jg {

bool mfma_fwd_supported(const ConvGeom& g, int dtype) {
  return dtype == JG_BF16 && shape_ok(g.cin, g.cout, g) && g.batch > 0;
}
bool mfma_dgrad_supported(const ConvGeom& g, int dtype) {
  if (dtype != JG_BF16 || g.batch <= 0) return false;
  if (g.p[1] > KH - 1 || g.p[2] > KW - 1) return false;
  return shape_ok(g.cout, g.cin, g);
}

size_t mfma_fwd_workspace(const ConvGeom& g) { return prep_bytes(g.cin, g.cout); }
size_t mfma_dgrad_workspace(const ConvGeom& g) { return prep_bytes(g.cout, g.cin); }

int mfma_fwd(void* y, const void* x, const void* w, const void* bias, const ConvGeom& g, void* ws,
             size_t ws_bytes, hipStream_t s) {
  return launch_conv(static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(w),
                     static_cast<const uint16_t*>(bias), static_cast<uint16_t*>(y), (int)g.batch,
                     g.cin, g.cout, g.in[1], g.in[2], g.out[1], g.out[2], g.p[1], g.p[2], 0, ws,
                     ws_bytes, s, "jg_conv_fwd(mfma)");
}

int mfma_dgrad(void* gx, const void* w, const void* go, const ConvGeom& g, void* ws,
               size_t ws_bytes, hipStream_t s) {
  // gx = conv(go zero-padded by k-1-p, flipped / transposed weights)
  return launch_conv(static_cast<const uint16_t*>(go), static_cast<const uint16_t*>(w), nullptr,
                     static_cast<uint16_t*>(gx), (int)g.batch, g.cout, g.cin, g.out[1], g.out[2],
                     g.in[1], g.in[2], KH - 1 - g.p[1], KW - 1 - g.p[2], 1, ws, ws_bytes, s,
                     "jg_conv_dgrad(mfma)");
}

}  // namespace jg
