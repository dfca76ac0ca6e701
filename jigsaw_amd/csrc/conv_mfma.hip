// Implicit-GEMM convolution on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16):
// 3x3 (2-D) and 3x3x3 (3-D), stride 1, dilation 1, channels-first tensors in and
// out. One kernel serves the forward pass and the input gradient.
//
//   GEMM view   Y[m][pixel] = sum_{tap, k} Wt[tap][m][k] * X[k][pixel + tap]
//               A 3-D problem is the 2-D one with the depth taps folded into the
//               contraction channels: channel kd*C + c of a tile at output depth d
//               is the plane X[c][d + kd - pad_d].
//   MFMA roles  A = weights (M = 32 produced channels, K = 16 contraction channels),
//               B = input pixels (K = 16 channels, N = 32 consecutive pixels of a
//               row), so an accumulator lane owns one pixel and 16 produced channels
//               and the stores run along W of the channels-first output.
//   Workgroup   512 threads = 8 wavefronts; output tile 16 rows x 64 columns x MT
//               produced channels; wavefront w owns rows 4*((w + 2*(w/4))%4).., columns 32*(w/4)..
//   LDS         the whole prepared weight block of the workgroup's produced-channel
//               tile stays resident; the input tile is streamed in stages of 16
//               contraction channels, double buffered (2 x 40.5 KiB). Input pixels
//               are stored "8 channels per 16-byte slot" so that a B fragment is one
//               ds_read_b128 per lane; the channels-first global rows (8 channels x
//               8 pixels per lane, 16-byte loads) are transposed in registers on the
//               way in. Slots of a row are interleaved by pixel phase (col % 8) so
//               that both the transposing writes and the fragment reads spread over
//               the banks.
//   Schedule    persistent workgroups (one per CU) walk a contiguous, XCD-local
//               range of tiles; the global loads of stage s+1 are issued before the
//               MFMAs of stage s and written to LDS between its MFMA groups (one
//               barrier per stage). A cursor decodes a tile's coordinates once and steps
//               through its stages by additions; the weight fragments of a group of 24
//               MFMAs are fetched under the group before, into the registers it frees.
//   Tile grid   tile column tw covers produced columns [org_w + 64 tw, + 64). The host picks
//               org_w <= 0 so that the staged row segments (144 bytes from input column
//               org_w + 64 tw - pad_w) start on cache lines where that costs no extra
//               tile column, and stages a window from one pixel earlier (lead) when it
//               would otherwise start on an odd column (4-byte aligned loads throughout).
//   Epilogue    16-bit results with rows of whole 16-byte pieces pass through LDS and leave as
//               16-byte stores; everything else as 2- or 4-byte stores along W.
//   dgrad       the same kernel on the output gradient with virtual zero padding
//               k-1-p and the weights flipped and transposed by the preparation.
//   Channels    any counts: the contraction is padded to 16-channel steps per depth tap
//               (zero weights; the registers of channels that do not exist are zeroed on
//               their way to LDS), the weights stay in LDS in groups of steps when they
//               do not fit at once, produced channels are padded to 32 and a ragged last
//               tile predicates its stores.
//   fp16        the same kernel on v_mfma_f32_32x32x16_f16 (a template flag; the staging moves
//               16-bit values without looking at them).
//   fp32        "split mode": an operand is the exact sum of three bf16 parts, kept as extra
//               channel groups; the contraction runs over the six part products that matter
//               and the result is stored as fp32. (A two-part form of it for fp16 operands
//               remains in the split kernels and is not dispatched.)
#include <type_traits>

#include "conv_common.h"

namespace {

using jg::ConvGeom;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

constexpr int KH = 3, KW = 3, TAPS = KH * KW;  // taps inside a plane
constexpr int TH = 16, TW = 64;                // output tile of a workgroup
constexpr int WAVES = 8, THREADS = WAVES * 64;
constexpr int WROWS = 4;                       // output rows per wavefront
constexpr int IN_ROWS = TH + KH - 1;           // 18
constexpr int OCTS = 9;                        // 9 octets of 8 pixels cover 66 (+6) columns
constexpr int ROW_SLOTS = 8 * OCTS;            // 16-byte slots per LDS row
constexpr int CK = 16;                         // contraction channels per stage
constexpr int STAGE_SLOTS = 2 * IN_ROWS * ROW_SLOTS;  // [kg][row][slot]
constexpr int STAGE_BYTES = STAGE_SLOTS * 16;         // 41472
constexpr int TASKS = 2 * IN_ROWS * OCTS;             // 324 tasks of 8 channels x 8 pixels

__device__ __forceinline__ int in_slot(int col) { return (col & 7) * OCTS + (col >> 3); }

struct FwdParams {
  const uint16_t* x;    // (N, C, Din, Hin, Win) bf16: the tensor that is convolved
  const char* x_end;    // one past the last byte of x
  const u32x4* wprep;   // prepared weights, [m_tile][group][tap9][wc16][kg][MT][8]
  const uint16_t* bias; // (M,) or NULL
  uint16_t* y;          // (N, M, Dout, Hout, Wout)
  int N, C, M;          // batch, channels of x, produced channels
  int Cp;               // C rounded up to a multiple of 16: contraction channels per depth tap
  // Split mode (fp32 / fp16 operands as sums of 3 / 2 bf16 parts): x holds Cx = parts * C channels per
  // batch entry (one channel group per part), the contraction runs over nblk = 6 / 3 blocks of KD * Cp
  // channels, block b reads part (xmap >> 2 b) & 3 of x against the weight part the
  // preparation put there. Plain mode: nblk = 1, xmap = 0, Cx = C.
  int nblk, Cx;
  uint32_t xmap;
  int out_kind;         // dtype of y and bias: 0 bf16, 1 fp32, 2 fp16
  int KD;               // depth taps (1 for 2-D); contraction channels K = KD * C
  int Din, Hin, Win, Dout, Hout, Wout;
  int pad_d, pad_h, pad_w;  // virtual zero padding of x
  int tiles_h, tiles_w;
  // Tile column tw covers produced columns [org_w + tw * TW, + TW), org_w <= 0: the host shifts the
  // grid to put the staged row segments on cache-line boundaries where that is free.
  // The staged window starts `lead` (0 / 1) pixels before the first one a tile needs, so that its
  // rows stay 4-byte aligned whatever the parity of pad_w - org_w.
  int org_w, lead;
  int sw;               // tile order inside a plane: row-major inside bands of sw tile columns, band after band
  int total_tiles;      // N * Dout * tiles_h * tiles_w
  int nc16;             // KD * Cp / 16
  int wc16;             // 16-channel steps whose weights sit in LDS at a time (a group)
  int ngroups;          // ceil(nc16 / wc16); > 1: the weights are reloaded group by group
  // Fold mode (input gradient written to its owners): y is the unpadded tile
  // (N, M, nD, nH, nW); produced cells outside [lo, lo + n) go to the strip of the
  // neighbour that owns them. fold = 0: y is the whole produced tensor.
  int fold;
  int lo_d, lo_h, lo_w, nD, nH, nW;
  // Framed input: xt (N, C, tn_d, tn_h, tn_w) is the own tile, which sits at [tlo, tlo + tn)
  // inside x. A stage whose window lies inside the tile reads xt, so that only a frame of
  // x near the edges has to hold data. NULL: everything comes from x.
  const uint16_t* xt;
  int tlo_d, tlo_h, tlo_w, tn_d, tn_h, tn_w;
};

// Strips of the 26 neighbours, slot (dd+1)*9 + (dh+1)*3 + (dw+1); first kernel
// parameter, so that a lane can index it in the kernel-argument segment.
struct StripTable {
  void* p[27];
};

__device__ __forceinline__ void* strip_entry(int idx) {
#if defined(__HIP_DEVICE_COMPILE__)
  void* const* kt = (void* const*)__builtin_amdgcn_kernarg_segment_ptr();
  return kt[idx];
#else
  (void)idx;
  return nullptr;
#endif
}

// ---------------------------------------------------------------- weight prep
// dst[(((mt*ngroups + group)*9 + tap9)*wc16 + c16 in group)*2 + kg][m_local][8 k] (bf16), contraction channel
// k = kd*Cp + c (channels C..Cp-1 are zero padding). transposed = 0: A[m][k] = w[m][c][kd][kh][kw] (forward, w is
// (M, C, KD, 3, 3)); transposed = 1: A[m][k] = w[c][m][KD-1-kd][2-kh][2-kw] (input
// gradient, w is (C, M, KD, 3, 3)).
__global__ __launch_bounds__(256) void prep_weights_kernel(uint16_t* __restrict__ dst,
                                                           const uint16_t* __restrict__ w,
                                                           int M, int C, int Cp, int KD, int MT, int mtiles,
                                                           int wc16, int ngroups, int transposed) {
  const int K = KD * Cp;
  const int total = mtiles * ngroups * TAPS * wc16 * 2 * MT * 8;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
    int e = i & 7;
    int r = i >> 3;
    int ml = r % MT; r /= MT;
    int kg = r & 1; r >>= 1;
    int c16l = r % wc16; r /= wc16;
    int tap = r % TAPS; r /= TAPS;
    int grp = r % ngroups;
    int mt = r / ngroups;
    const int m = mt * MT + ml;
    const int k = (grp * wc16 + c16l) * CK + kg * 8 + e;
    uint16_t v = 0;  // rows past M and steps past K are padding
    const int kd = k / Cp, c = k - kd * Cp;
    if (m < M && k < K && c < C) {
      const int kh = tap / KW, kw = tap % KW;
      if (!transposed)
        v = w[((((size_t)m * C + c) * KD + kd) * KH + kh) * KW + kw];
      else
        v = w[((((size_t)c * M + m) * KD + (KD - 1 - kd)) * KH + (KH - 1 - kh)) * KW + (KW - 1 - kw)];
    }
    dst[i] = v;
  }
}

// ---------------------------------------------------------------- split mode
// An fp32 value is the sum of three bf16 parts (8 + 8 + 8 significand bits): high = bf16(v),
// middle = bf16(v - high), low = bf16(v - high - middle); the subtractions are exact. A
// product of two fp32 values is then, to 2^-24 relative, the sum of the six part products
// whose indices add up to at most 2, each of which the bf16 matrix cores form exactly and
// add in fp32. An fp16 value (11 significand bits) is the sum of two parts, and the three
// products (0,0), (0,1), (1,0) carry it to 2^-16 relative, far below fp16's own rounding.
__device__ __forceinline__ uint16_t split_part(float v, int part) {
  const uint16_t hi = jg::f32_to_bf16(v);
  if (part == 0) return hi;
  const float hf = jg::bf16_to_f32(hi);
  const float r1 = (hf - hf == 0.0f) ? v - hf : 0.0f;  // an infinite (or NaN) high part carries everything
  const uint16_t mid = jg::f32_to_bf16(r1);
  if (part == 1) return mid;
  return jg::f32_to_bf16(r1 - jg::bf16_to_f32(mid));
}
// Contraction blocks of a split mode: block b multiplies input part x[b] with weight part w[b]
// (two bits each, block 0 in the lowest bits).
struct SplitSpec {
  int parts, nblk;
  uint32_t xparts, wparts;
};
constexpr uint32_t pack_parts(int a, int b, int c, int d, int e, int f) {
  return (uint32_t)a | ((uint32_t)b << 2) | ((uint32_t)c << 4) | ((uint32_t)d << 6) | ((uint32_t)e << 8) | ((uint32_t)f << 10);
}
inline SplitSpec split_spec(int mode) {
  if (mode == 1) return SplitSpec{3, 6, pack_parts(0, 0, 1, 0, 1, 2), pack_parts(0, 1, 0, 2, 1, 0)};  // fp32
  if (mode == 2) return SplitSpec{2, 3, pack_parts(0, 0, 1, 0, 0, 0), pack_parts(0, 1, 0, 0, 0, 0)};  // fp16
  return SplitSpec{1, 1, 0u, 0u};
}
template <typename SRC>
__device__ __forceinline__ float to_float(SRC v) { return (float)v; }

// dst (batch, parts, per_batch) bf16 = the parts of src (batch, per_batch), fp32 or fp16
template <typename SRC>
__global__ __launch_bounds__(256) void split_kernel(uint16_t* __restrict__ dst, const SRC* __restrict__ src,
                                                    size_t per_batch, size_t total, int parts) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
    const size_t n = i / per_batch, r = i - n * per_batch;
    const float v = to_float(src[i]);
    const uint16_t hi = jg::f32_to_bf16(v);
    const float hf = jg::bf16_to_f32(hi);
    const float r1 = (hf - hf == 0.0f) ? v - hf : 0.0f;
    const uint16_t mid = jg::f32_to_bf16(r1);
    uint16_t* d = dst + n * parts * per_batch + r;
    d[0] = hi;
    d[per_batch] = mid;
    if (parts == 3) d[2 * per_batch] = jg::f32_to_bf16(r1 - jg::bf16_to_f32(mid));
  }
}

// prep_weights_kernel for a split mode: w is fp32 or fp16, the contraction has nblk blocks of
// KD * Cp channels, block b holds part (wparts >> 2 b) & 3 of the weights.
template <typename SRC>
__global__ __launch_bounds__(256) void prep_weights_split_kernel(uint16_t* __restrict__ dst,
                                                                 const SRC* __restrict__ w, int M, int C, int Cp,
                                                                 int KD, int MT, int mtiles, int wc16, int ngroups,
                                                                 int transposed, int nblk, uint32_t wparts) {
  const int KB = KD * Cp, K = nblk * KB;
  const int total = mtiles * ngroups * TAPS * wc16 * 2 * MT * 8;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
    int e = i & 7;
    int r = i >> 3;
    int ml = r % MT; r /= MT;
    int kg = r & 1; r >>= 1;
    int c16l = r % wc16; r /= wc16;
    int tap = r % TAPS; r /= TAPS;
    int grp = r % ngroups;
    int mt = r / ngroups;
    const int m = mt * MT + ml;
    const int k = (grp * wc16 + c16l) * CK + kg * 8 + e;
    const int blk = k / KB, kin = k - blk * KB;
    const int kd = kin / Cp, c = kin - kd * Cp;
    uint16_t v = 0;
    if (m < M && k < K && c < C) {
      const int kh = tap / KW, kw = tap % KW;
      const float f = to_float(!transposed ? w[((((size_t)m * C + c) * KD + kd) * KH + kh) * KW + kw]
                                           : w[((((size_t)c * M + m) * KD + (KD - 1 - kd)) * KH + (KH - 1 - kh)) * KW + (KW - 1 - kw)]);
      v = split_part(f, (int)((wparts >> (2 * blk)) & 3u));
    }
    dst[i] = v;
  }
}

// ------------------------------------------------------------ forward kernel
// EVEN: Win, pad_w and the plane size are even and x is 4-byte aligned, so every
// pixel pair of a task is one aligned dword that is either wholly inside or wholly
// outside the tensor. Otherwise the prefetch falls back to 2-byte loads.
// 2-byte stores with a scalar base and a 32-bit lane offset. The epilogue issues 128 of
// them per lane and tile; with the 64-bit lane addresses the compiler builds for plain
// pointer code each one moves 512 bytes of addresses to the memory pipeline, which is what
// the epilogue then waits on. `base` must be wave-uniform.
__device__ inline void store_bf16_lo(const void* base, uint32_t lane_off, uint32_t pair) {
  asm volatile("global_store_short %0, %1, %2" : : "v"(lane_off), "v"(pair), "s"(base) : "memory");
}
__device__ inline void store_bf16_hi(const void* base, uint32_t lane_off, uint32_t pair) {
  asm volatile("global_store_short_d16_hi %0, %1, %2" : : "v"(lane_off), "v"(pair), "s"(base) : "memory");
}
__device__ inline void store_16_bytes(const void* base, uint32_t lane_off, u32x4 v) {
  // The store reads its 16 bytes of data from the registers a little after it issues; a vector
  // instruction that overwrites them within two wait states would be stored instead. The
  // compiler pads that for its own stores but does not look inside an asm statement.
  asm volatile("global_store_dwordx4 %0, %1, %2\n\ts_nop 1" : : "v"(lane_off), "v"(v), "s"(base) : "memory");
}
__device__ inline void store_f32(const void* base, uint32_t lane_off, float v) {
  asm volatile("global_store_dword %0, %1, %2" : : "v"(lane_off), "v"(v), "s"(base) : "memory");
}

// F16: the 16-bit tensors hold fp16 instead of bf16 (v_mfma_f32_32x32x16_f16; everything else moves
// 16-bit values without looking at them, the epilogue converts by out_kind).
// PX: the MFMA operands are exchanged, D[pixel][channel] instead of D[channel][pixel]: an accumulator lane
// then owns ONE produced channel and 16 pixels, 8 consecutive ones per lane half and register octet, so that
// a lane's results are whole 16-byte pieces of an output row and leave straight from the registers. The rows
// of the pixel operand are dealt to the pixels with bits 2 and 3 of the row number exchanged (row 8j + 4h + t
// of the result lies in lane half h, register 4j + t; pixel 16 (j / 2) + 8 h + 4 (j % 2) + t goes there).
// Used where every row segment of the result is made of whole, aligned 16-byte pieces.
__device__ __forceinline__ int px_of_row(int m) { return (m & 0x13) | ((m & 4) << 1) | ((m & 8) >> 1); }

template <int MT, bool EVEN, bool FOLD, bool FRAMED, bool F16 = false, bool PX = false>  // MT = produced channels per workgroup: 32 or 64
__global__ __launch_bounds__(THREADS) void conv3x3_mfma_kernel(StripTable strips, FwdParams p) {
  constexpr int CB = MT / 32;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int w_slots = TAPS * p.wc16 * 2 * MT;  // 16-byte slots of one group of weights
  u32x4* lds_w = reinterpret_cast<u32x4*>(smem);
  u32x4* lds_in = lds_w + w_slots;  // two stages
  float* lds_bias = reinterpret_cast<float*>(lds_in + 2 * STAGE_SLOTS);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  // Wavefronts w and w + 4 share a SIMD. They hold different column halves, so when a tile's second
  // half lies past the row end every SIMD drops half of that tile's MFMAs, and row groups two apart,
  // so a tile with few valid rows keeps two SIMDs busy instead of one.
  const int wrow0 = ((wave + 2 * (wave >> 2)) & 3) * WROWS, wcol0 = (wave >> 2) * 32;
  const int mt = blockIdx.y;

  // ---- tile schedule: XCD x (= blockIdx.x % 8) owns a contiguous range of tiles and
  // walks it cyclically from a start that differs per XCD. Without the stagger, ranges
  // that coincide with whole images make the 8 XCDs stream addresses that differ by a
  // multiple of the image size in lockstep, which piles them onto the same memory channels.
  const int G = gridDim.x;
  const int xcd = blockIdx.x & 7, slot_in_xcd = blockIdx.x >> 3;
  const int wg_per_xcd = (G + 7) >> 3;
  const int per_xcd = (p.total_tiles + 7) >> 3;
  const int t_begin = xcd * per_xcd;
  int t_end = t_begin + per_xcd;
  if (t_end > p.total_tiles) t_end = p.total_tiles;
  const int t_len = t_end - t_begin;
  if (slot_in_xcd >= t_len) return;
  const int t_rot = (int)(((long long)xcd * t_len) >> 3);
  const int my_tiles = (t_len - slot_in_xcd + wg_per_xcd - 1) / wg_per_xcd;
  auto tile_of = [&](int ti) {  // ti-th tile of this workgroup
    int i = slot_in_xcd + ti * wg_per_xcd + t_rot;
    if (i >= t_len) i -= t_len;
    return t_begin + i;
  };

  // ---- weights and bias. With one group the weights stay in LDS for the life of the
  // workgroup; with more (many input channels) group g is loaded before the stages that
  // contract its channels.
  auto load_weights = [&](int grp) {
    const u32x4* src = p.wprep + ((size_t)mt * p.ngroups + grp) * w_slots;
    for (int i = tid; i < w_slots; i += THREADS) lds_w[i] = src[i];
  };
  if (p.ngroups == 1) load_weights(0);
  if (tid < MT)
    lds_bias[tid] = (p.bias == nullptr || mt * MT + tid >= p.M) ? 0.0f
                    : p.out_kind == 1 ? reinterpret_cast<const float*>(p.bias)[mt * MT + tid]
                    : p.out_kind == 2 ? (float)reinterpret_cast<const _Float16*>(p.bias)[mt * MT + tid]
                                      : jg::bf16_to_f32(p.bias[mt * MT + tid]);

  // ---- prefetch bookkeeping. A task = 8 channels x 8 pixels of one input row.
  const size_t plane = (size_t)p.Hin * p.Win;
  const size_t chan_stride = plane * p.Din;            // elements between channels
  const uint32_t chan_b = (uint32_t)(chan_stride * 2);  // bytes
  const bool has_task = tid < TASKS;
  const int oct = tid % OCTS;
  const int rr = tid / OCTS;         // = g8 * IN_ROWS + row
  const int t_row = rr % IN_ROWS;
  const int t_col = oct * 8;
  const int g8 = rr / IN_ROWS;
  const uint32_t t_off = (uint32_t)(((size_t)g8 * 8 * chan_stride + (size_t)t_row * p.Win + t_col) * 2);
  const int t_lds = rr * ROW_SLOTS + oct;
  const size_t plane_t = (size_t)p.tn_h * p.tn_w;
  const size_t chan_stride_t = plane_t * p.tn_d;
  const uint32_t chan_bt = (uint32_t)(chan_stride_t * 2);
  const uint32_t t_off_t = (uint32_t)(((size_t)g8 * 8 * chan_stride_t + (size_t)t_row * p.tn_w + t_col) * 2);
  uint32_t stg[8][4];

  struct TileCoord {
    int n, od, th, tw;
  };
  auto coord = [&](int tile) {
    TileCoord c;
    const int per_plane = p.tiles_h * p.tiles_w;
    int tq = tile / per_plane;
    int j = tile - tq * per_plane;
    const int band = p.tiles_h * p.sw;          // tiles in a full band
    const int b = j / band;                     // band number; the last one may be narrower
    j -= b * band;
    const int width = min(p.sw, p.tiles_w - b * p.sw);
    c.th = j / width;
    c.tw = b * p.sw + (j - c.th * width);
    c.od = tq % p.Dout;
    c.n = tq / p.Dout;
    return c;
  };

  // ---- load cursor: the (tile, 16-channel step) whose loads are issued next; it runs two stages
  // ahead of the MFMAs. Everything that takes a division (the tile's coordinates) is done when
  // the cursor enters a tile; inside a tile the step moves by additions.
  struct Cursor {
    int ti;          // index into this workgroup's tiles
    int blk, inner;  // contraction block, channel offset inside it (= kd * Cp + c0)
    int kd, c0;      // depth tap and first channel of the step
    int od;          // produced depth plane of the tile
    int ih0, iw0;    // window origin in the input plane
    bool window_in;  // rows and columns of the window lie inside the plane
    bool window_in_t;  // ... inside the rank's own tile (framed input)
    const char* base;    // window origin in channel 0 of the batch entry, depth plane 0
    const char* base_t;  // the same in the rank's own tile (framed input)
  } cur;
  const int per_blk_ch = (p.nc16 / p.nblk) * CK;  // contraction channels (x depth taps) of one block
  auto cursor_enter = [&](int ti) __attribute__((always_inline)) {
    cur.ti = ti;
    cur.blk = 0; cur.inner = 0; cur.kd = 0; cur.c0 = 0;
    if (ti >= my_tiles) return;
    const TileCoord tc = coord(tile_of(ti));
    cur.od = tc.od;
    cur.ih0 = tc.th * TH - p.pad_h;
    cur.iw0 = tc.tw * TW + p.org_w - p.pad_w - p.lead;
    cur.window_in = cur.ih0 >= 0 && cur.ih0 + IN_ROWS <= p.Hin && cur.iw0 >= 0 && cur.iw0 + p.lead + TW + KW - 1 <= p.Win;
    cur.base = reinterpret_cast<const char*>(p.x) +
               2 * ((ptrdiff_t)((size_t)tc.n * p.Cx * chan_stride) + (ptrdiff_t)cur.ih0 * p.Win + cur.iw0);
    if (FRAMED) {
      const int ht = cur.ih0 - p.tlo_h, wt = cur.iw0 - p.tlo_w;
      cur.window_in_t = ht >= 0 && ht + IN_ROWS <= p.tn_h && wt >= 0 && wt + p.lead + TW + KW - 1 <= p.tn_w;
      cur.base_t = reinterpret_cast<const char*>(p.xt) +
                   2 * ((ptrdiff_t)((size_t)tc.n * p.Cx * chan_stride_t) + (ptrdiff_t)ht * p.tn_w + wt);
    }
  };
  auto cursor_advance = [&]() __attribute__((always_inline)) {
    cur.inner += CK;
    cur.c0 += CK;
    if (cur.c0 >= p.Cp) {
      cur.c0 = 0;
      ++cur.kd;
    }
    if (cur.inner == per_blk_ch) {
      cur.inner = 0; cur.kd = 0; cur.c0 = 0;
      if (++cur.blk == p.nblk) cursor_enter(cur.ti + 1);
    }
  };

  // Loads of the stage under the cursor.
  auto issue_loads = [&]() __attribute__((always_inline)) {
    const int kd = cur.kd, c0 = cur.c0;
    const int cx0 = (int)((p.xmap >> (2 * cur.blk)) & 3u) * p.C + c0;  // first channel of the step in x
    // Channels of this task that exist (all 8 unless C is not a multiple of 16). The vector
    // path below reads the others anyway (they lie inside the tensor: the interior test covers
    // all 16 channel planes) and store_stage zeroes them; the guarded paths skip them.
    const int cvalid = p.C - c0 - g8 * 8;
    const int id = cur.od + kd - p.pad_d;
    const int ih0 = cur.ih0, iw0 = cur.iw0;
    const bool depth_ok = id >= 0 && id < p.Din;
    // wave-uniform origin of the stage window (lies before the tensor where padded)
    const char* origin = cur.base + 2 * ((ptrdiff_t)((size_t)cx0 * chan_stride) + (ptrdiff_t)id * (ptrdiff_t)plane);
    // The last octet of a row holds 2 pixels that are used and 6 that no fragment
    // reads, so it may run past the row end as long as it stays inside the tensor.
    const char* last = origin + 2 * ((size_t)(CK - 1) * chan_stride + (size_t)(IN_ROWS - 1) * p.Win + OCTS * 8);
    const bool interior = depth_ok && cur.window_in && last <= p.x_end;
    if (FRAMED) {
      // window inside the own tile (wave-uniform): read the tile itself, at whatever
      // alignment its rows give the window
      const int dt = id - p.tlo_d;
      const char* origin_t = cur.base_t + 2 * ((ptrdiff_t)((size_t)cx0 * chan_stride_t) + (ptrdiff_t)dt * (ptrdiff_t)plane_t);
      if (dt >= 0 && dt < p.tn_d && cur.window_in_t) {
        if (!has_task) return;
        // 4-byte aligned accesses only (2-byte aligned vector loads run at a fraction of the
        // rate): a window that starts on an odd column is read one pixel early and shifted.
        const bool odd = ((reinterpret_cast<uintptr_t>(origin_t) + t_off_t) & 2) != 0;  // wave-uniform
        const char* at = origin_t + t_off_t;
        if (!odd) {
          if (oct == OCTS - 1) {
            // the last octet holds the window's last 2 pixels; the other 6 may lie past the row
            // (and the tensor), so only one dword is read
#pragma unroll
            for (int c = 0; c < 8; ++c) {
              stg[c][0] = *reinterpret_cast<const uint32_t*>(at + (size_t)c * chan_bt);
              stg[c][1] = 0u; stg[c][2] = 0u; stg[c][3] = 0u;
            }
          } else {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
              const u32x4_a4 v = *reinterpret_cast<const u32x4_a4*>(at + (size_t)c * chan_bt);
              stg[c][0] = v.x; stg[c][1] = v.y; stg[c][2] = v.z; stg[c][3] = v.w;
            }
          }
        } else {
          uint32_t d0[8];
#pragma unroll
          for (int c = 0; c < 8; ++c) d0[c] = *reinterpret_cast<const uint32_t*>(at - 2 + (size_t)c * chan_bt);
          if (oct == OCTS - 1) {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
              const uint32_t d1 = *reinterpret_cast<const uint32_t*>(at + 2 + (size_t)c * chan_bt);
              stg[c][0] = __builtin_amdgcn_alignbit(d1, d0[c], 16);
              stg[c][1] = 0u; stg[c][2] = 0u; stg[c][3] = 0u;
            }
          } else {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
              const u32x4_a4 v = *reinterpret_cast<const u32x4_a4*>(at + 2 + (size_t)c * chan_bt);
              stg[c][0] = __builtin_amdgcn_alignbit(v.x, d0[c], 16);
              stg[c][1] = __builtin_amdgcn_alignbit(v.y, v.x, 16);
              stg[c][2] = __builtin_amdgcn_alignbit(v.z, v.y, 16);
              stg[c][3] = __builtin_amdgcn_alignbit(v.w, v.z, 16);
            }
          }
        }
        return;
      }
    }
    if (!has_task) return;
    const char* a = origin + t_off;
    if (EVEN && interior) {
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const u32x4_a4 v = *reinterpret_cast<const u32x4_a4*>(a + (size_t)c * chan_b);
        stg[c][0] = v.x; stg[c][1] = v.y; stg[c][2] = v.z; stg[c][3] = v.w;
      }
    } else if (EVEN) {
      // A window that sticks out of the tensor (the border tiles of a padded problem: one tile in
      // seven of configuration 2's input gradient). Most of its tasks still lie wholly inside and
      // keep their 16-byte loads, the ones wholly outside load nothing; only the tasks that
      // straddle an edge go dword by dword.
      const int ih = ih0 + t_row, iw = iw0 + t_col;
      const bool row_ok = depth_ok && (ih >= 0) && (ih < p.Hin);
      if (row_ok && iw >= 0 && iw + 8 <= p.Win && cvalid >= 8) {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const u32x4_a4 v = *reinterpret_cast<const u32x4_a4*>(a + (size_t)c * chan_b);
          stg[c][0] = v.x; stg[c][1] = v.y; stg[c][2] = v.z; stg[c][3] = v.w;
        }
      } else if (!row_ok || iw + 8 <= 0 || iw >= p.Win) {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          stg[c][0] = 0u; stg[c][1] = 0u; stg[c][2] = 0u; stg[c][3] = 0u;
        }
      } else {
        bool ok[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) ok[j] = iw + 2 * j >= 0 && iw + 2 * j + 2 <= p.Win;
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            stg[c][j] = (ok[j] && c < cvalid) ? *reinterpret_cast<const uint32_t*>(a + (size_t)c * chan_b + 4 * j) : 0u;
      }
    } else {
      const int ih = ih0 + t_row, iw = iw0 + t_col;
      const bool rows_ok = depth_ok && (ih >= 0) && (ih < p.Hin);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const bool row_ok = rows_ok && c < cvalid;
        const uint16_t* e = reinterpret_cast<const uint16_t*>(a + (size_t)c * chan_b);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t lo = (row_ok && iw + 2 * j >= 0 && iw + 2 * j < p.Win) ? (uint32_t)e[2 * j] : 0u;
          const uint32_t hi = (row_ok && iw + 2 * j + 1 >= 0 && iw + 2 * j + 1 < p.Win) ? (uint32_t)e[2 * j + 1] : 0u;
          stg[c][j] = lo | (hi << 16);
        }
      }
    }
  };

  auto store_stage = [&](int buf, int stage) {  // stage: counted over this workgroup's tiles
    if (!has_task) return;
    if (p.Cp != p.C) {  // uniform: zero the channels of this step that do not exist
      const int cvalid = p.C - ((stage % p.nc16) * CK) % p.Cp - g8 * 8;
#pragma unroll
      for (int c = 0; c < 8; ++c)
        if (c >= cvalid) {
          stg[c][0] = 0u; stg[c][1] = 0u; stg[c][2] = 0u; stg[c][3] = 0u;
        }
    }
    u32x4* row_base = lds_in + buf * STAGE_SLOTS + t_lds;
#pragma unroll
    for (int px = 0; px < 8; ++px) {
      // pixel px of the octet: low (px even) or high (px odd) half of dword px/2
      const uint32_t sel = (px & 1) ? 0x07060302u : 0x05040100u;
      u32x4 v;
      v.x = __builtin_amdgcn_perm(stg[1][px >> 1], stg[0][px >> 1], sel);
      v.y = __builtin_amdgcn_perm(stg[3][px >> 1], stg[2][px >> 1], sel);
      v.z = __builtin_amdgcn_perm(stg[5][px >> 1], stg[4][px >> 1], sel);
      v.w = __builtin_amdgcn_perm(stg[7][px >> 1], stg[6][px >> 1], sel);
      row_base[px * OCTS] = v;
    }
  };

  f32x16 acc[CB][WROWS];

  // One third (one kw) of a stage's MFMAs. The fragments roll through the stage: the weight
  // fragments of tap row kh are last used by input row kh + WROWS - 1 of the group, and the
  // same registers are refilled right there with the next group's fragments (the next kw, or
  // after the last kw the first group of the next stage: the weights do not change at the
  // barrier), and the group's last step requests the first input fragment of the next kw. So
  // only the first input fragment of a stage is waited for with nothing else to issue.
  bf16x8 a[KH][CB];
  u32x4 bnext;
  int a_step = -1;  // the step inside the weight group whose kw = 0 fragments `a` holds
  auto weight_frag = [&](int wstep, int kh, int kw, int cb) {
    const u32x4* wt = lds_w + ((size_t)wstep * 2 + kg) * MT + ln;
    return __builtin_bit_cast(bf16x8, wt[(size_t)(kh * KW + kw) * p.wc16 * 2 * MT + cb * 32]);
  };
  auto compute_kw = [&](int buf, int wstep, int kw, int wstep_next) {  // wstep: the stage's step inside its weight group
    const u32x4* in = lds_in + buf * STAGE_SLOTS + kg * (IN_ROWS * ROW_SLOTS) + wrow0 * ROW_SLOTS;
    const int col0 = wcol0 + (PX ? px_of_row(ln) : ln) + p.lead;  // the tile's pixel 0 sits `lead` slots into the staged row
    const u32x4* inb = in + in_slot(col0 + kw);
    if (kw == 0) {
      if (a_step != wstep) {  // wave-uniform: the first stage, after a tile without work, after a weight reload
#pragma unroll
        for (int kh = 0; kh < KH; ++kh)
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) a[kh][cb] = weight_frag(wstep, kh, 0, cb);
      }
      bnext = inb[0];
    }
    // software pipeline over the input rows: the fragment of row rho+1 is requested
    // before the MFMAs of row rho are issued, so its LDS latency hides behind them
#pragma unroll
    for (int rho = 0; rho < WROWS + KH - 1; ++rho) {
      const bf16x8 b = __builtin_bit_cast(bf16x8, bnext);
      if (rho + 1 < WROWS + KH - 1) bnext = inb[(rho + 1) * ROW_SLOTS];
      else if (kw + 1 < KW) bnext = in[in_slot(col0 + kw + 1)];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kh = 0; kh < KH; ++kh) {
        const int r = rho - kh;
        if (r >= 0 && r < WROWS) {
#pragma unroll
          for (int cb = 0; cb < CB; ++cb)
            if (F16 && PX)
              acc[cb][r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, b),
                                                                  __builtin_bit_cast(f16x8, a[kh][cb]), acc[cb][r], 0, 0, 0);
            else if (F16)
              acc[cb][r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[kh][cb]),
                                                                  __builtin_bit_cast(f16x8, b), acc[cb][r], 0, 0, 0);
            else if (PX)
              acc[cb][r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a[kh][cb], acc[cb][r], 0, 0, 0);
            else
              acc[cb][r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kh][cb], b, acc[cb][r], 0, 0, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      const int kh_done = rho - (WROWS - 1);  // this tap row's weights are not read again in this group
      if (kh_done >= 0) {
        if (kw + 1 < KW) {
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) a[kh_done][cb] = weight_frag(wstep, kh_done, kw + 1, cb);
        } else if (p.ngroups == 1) {
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) a[kh_done][cb] = weight_frag(wstep_next, kh_done, 0, cb);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (kw == KW - 1) a_step = p.ngroups == 1 ? wstep_next : -1;
  };

  // Accumulator lane (ln, kg), register i of block cb: produced channel
  // cb*32 + 8*(i/4) + 4*kg + i%4, pixel column wcol0 + ln.
  auto init_acc = [&]() {
    if (PX) {  // a lane owns one channel per block
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        const float bv = lds_bias[cb * 32 + ln];
#pragma unroll
        for (int r = 0; r < WROWS; ++r)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[cb][r][i] = bv;
      }
      return;
    }
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
  const size_t ochan = plane_o * p.Dout;  // elements between produced channels
  // RAGGED: the last tile of produced channels when M is not a multiple of MT (its weight
  // rows past M are zero padding); a lane then stores only the channels that exist.
  // Rows of a wavefront through LDS: the accumulator holds one pixel and 32 channels per lane,
  // memory wants runs of pixels. A row of the wavefront (32 pixels x MT channels) is written to
  // LDS as 16-bit values, 64 bytes per channel, and read back as 16-byte pieces that go out as
  // 16-byte stores: 4 store instructions per row instead of 32 (MT = 64). The two channels a
  // lane pair (kg = 0, 1) writes at once, m and m + 4, sit in neighbouring 64-byte rows of the
  // scratch, so that the halves of the wavefront use different banks. `scratch`: 64 * MT bytes of
  // LDS of this wavefront. Needs 16-byte aligned row segments in y (checked by the caller).
  // `ytile` is wave-uniform (a scalar base), `row_off` the byte offset of the wavefront's row segment from it.
  // `pair(cb, i)`: the 16-bit values of accumulator registers i (low half) and i + 1 of block cb.
  auto row_through_lds = [&](unsigned char* scratch, auto pair, char* ytile, uint32_t row_off, size_t chan_bytes) {
    // lane's part of the write address: pixel ln of LDS row kg
    unsigned char* wr = scratch + kg * 64 + ln * 2;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const uint32_t h2 = pair(cb, i);
        // channel cb*32 + 8*(i/4) + i%4 (+ 4 kg): LDS row (that & ~7) + 2*(i%4) (+ kg); i + 1: two rows on
        const int row = cb * 32 + 8 * (i >> 2) + 2 * (i & 3);
        *reinterpret_cast<uint16_t*>(wr + row * 64) = (uint16_t)(h2 & 0xffffu);
        *reinterpret_cast<uint16_t*>(wr + (row + 2) * 64) = (uint16_t)(h2 >> 16);
      }
    // piece g = 64 q + lane: LDS row g / 4 = 16 q + lane / 4, pixels 8 (lane % 4) ..; its channel is
    // 16 q + (lane/4 & 8) + (lane/4 >> 1 & 3) + 4 (lane/4 & 1)
    const int l4 = lane >> 2;
    const int m_lane = (l4 & 8) + ((l4 >> 1) & 3) + ((l4 & 1) << 2);
    const uint32_t voff = (uint32_t)(m_lane * chan_bytes) + 16u * (lane & 3) + row_off;
    // all the row's pieces are requested before the first is stored: one LDS latency per row
    u32x4 piece[MT / 16];
#pragma unroll
    for (int q = 0; q < MT / 16; ++q) piece[q] = *reinterpret_cast<const u32x4*>(scratch + (q * 64 + lane) * 16);
#pragma unroll
    for (int q = 0; q < MT / 16; ++q) store_16_bytes(ytile + (size_t)q * 16 * chan_bytes, voff, piece[q]);
  };

  // PX layout: lane (ln, kg) holds channel cb * 32 + ln; registers 8 J .. 8 J + 7 hold the pixels
  // wcol0 + 16 J + 8 kg + (0 .. 7) of the wavefront's row: one 16-byte piece of 16-bit results.
  auto piece_16bit = [&](int cb, int r, int J) {
    u32x4 v;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      f32x2 v2 = {acc[cb][r][8 * J + 2 * d], acc[cb][r][8 * J + 2 * d + 1]};
      v[d] = F16 ? __builtin_bit_cast(uint32_t, __builtin_convertvector(v2, f16x2))
                 : __builtin_bit_cast(uint32_t, __builtin_convertvector(v2, bf16x2));
    }
    return v;
  };
  // A row of the wavefront (32 pixels x MT channels of 16-bit results) goes through LDS once, as 16-byte
  // pieces both ways: lane (channel ln, half kg) writes its pieces 2 J + kg of channels cb * 32 + ln, then
  // lane l reads piece l % 4 of channel 16 q + l / 4, so that four neighbouring lanes store 64 contiguous
  // bytes of one channel row. A channel's four pieces sit in one 64-byte LDS row, at slot piece ^ (channel / 4 % 4):
  // the 16 lanes of a write (consecutive channels, one piece) and of a read (four channels, all pieces)
  // then each cover all 64 banks once. `scratch`: 64 * MT bytes of LDS of this wavefront.
  auto epilogue_px = [&](const TileCoord& tc, int free_buf) {
    const int tw0 = tc.tw * TW + p.org_w;
    const size_t chan_bytes = 2 * ochan;
    unsigned char* scratch = reinterpret_cast<unsigned char*>(lds_in + free_buf * STAGE_SLOTS) + wave * (STAGE_BYTES / WAVES);
    // wave-uniform base: the tile's first column in produced channel mt * MT, row 0 (it may lie before
    // the row where the tile grid starts left of the tensor; such pieces are not stored)
    char* ytile = reinterpret_cast<char*>(p.y) +
                  2 * ((ptrdiff_t)(((size_t)tc.n * p.M + (size_t)mt * MT) * ochan + (size_t)tc.od * plane_o) + (ptrdiff_t)tw0);
    const int m_left = p.M - mt * MT;
    const int l4 = lane >> 2, pc = lane & 3;  // reading side: channel 16 q + l4, piece pc
    const int px = tw0 + wcol0 + 8 * pc;
    const bool px_ok = px >= 0 && px + 8 <= p.Wout;
    const uint32_t lane_off = (uint32_t)(l4 * chan_bytes) + 2u * (uint32_t)(wcol0 + 8 * pc);
    unsigned char* wr = scratch + ln * 64;
    const unsigned char* rd = scratch + l4 * 64 + ((pc ^ ((l4 >> 2) & 3)) << 4);
    const int wsw = (ln >> 2) & 3;
#pragma unroll
    for (int r = 0; r < WROWS; ++r) {
      const int oh = tc.th * TH + wrow0 + r;
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int J = 0; J < 2; ++J)
          *reinterpret_cast<u32x4*>(wr + cb * 32 * 64 + (((2 * J + kg) ^ wsw) << 4)) = piece_16bit(cb, r, J);
      u32x4 piece[MT / 16];
#pragma unroll
      for (int q = 0; q < MT / 16; ++q) piece[q] = *reinterpret_cast<const u32x4*>(rd + q * 16 * 64);
      if (oh < p.Hout) {
        const uint32_t row_off = lane_off + 2u * (uint32_t)oh * (uint32_t)p.Wout;
#pragma unroll
        for (int q = 0; q < MT / 16; ++q)
          if (px_ok && q * 16 + l4 < m_left) store_16_bytes(ytile + (size_t)q * 16 * chan_bytes, row_off, piece[q]);
      }
    }
  };

  auto epilogue_rows = [&](const TileCoord& tc, auto ragged, int free_buf) {
    constexpr bool RAGGED = decltype(ragged)::value;
    const int tw0 = tc.tw * TW + p.org_w;  // first produced column of the tile
    const int ow = tw0 + wcol0 + ln;
    if (!RAGGED && p.out_kind != 1 && (p.Wout & 7) == 0 && (tw0 & 7) == 0 && (reinterpret_cast<uintptr_t>(p.y) & 15) == 0 &&
        tw0 + wcol0 >= 0 && tw0 + wcol0 + 32 <= p.Wout) {  // wave-uniform
      unsigned char* scratch = reinterpret_cast<unsigned char*>(lds_in + free_buf * STAGE_SLOTS) + wave * (STAGE_BYTES / WAVES);
      char* ytile = reinterpret_cast<char*>(p.y) +
                    2 * (((size_t)tc.n * p.M + (size_t)mt * MT) * (plane_o * p.Dout) + (size_t)tc.od * plane_o +
                         (size_t)tw0);
#pragma unroll
      for (int r = 0; r < WROWS; ++r) {
        const int oh = tc.th * TH + wrow0 + r;
        auto pair = [&](int cb, int i) {
          f32x2 v2 = {acc[cb][r][i], acc[cb][r][i + 1]};
          return F16 ? __builtin_bit_cast(uint32_t, __builtin_convertvector(v2, f16x2))
                                 : __builtin_bit_cast(uint32_t, __builtin_convertvector(v2, bf16x2));
        };
        if (oh < p.Hout)
          row_through_lds(scratch, pair, ytile, (uint32_t)(2 * ((size_t)oh * p.Wout + wcol0)), 2 * plane_o * p.Dout);
      }
      return;
    }
    char* ybase = reinterpret_cast<char*>(p.y) +
                  2 * (((size_t)tc.n * p.M + (size_t)mt * MT) * ochan + (size_t)tc.od * plane_o);
    const int m_left = p.M - mt * MT - 4 * kg;  // channels from this lane's first one to the end
    if (p.out_kind == 1) {  // uniform: the same walk with 4-byte stores
      char* ybase32 = reinterpret_cast<char*>(p.y) +
                      4 * (((size_t)tc.n * p.M + (size_t)mt * MT) * ochan + (size_t)tc.od * plane_o);
#pragma unroll
      for (int r = 0; r < WROWS; ++r) {
        const int oh = tc.th * TH + wrow0 + r;
        if (oh < p.Hout && ow >= 0 && ow < p.Wout) {
          const uint32_t voff = (uint32_t)(4 * ((size_t)(4 * kg) * ochan + (size_t)oh * p.Wout + ow));
          // the channel's base walks by additions (a product per store costs a scalar multiply, a 64-bit add
          // and, with the scalar registers this kernel has left, a spill reload)
          const char* yc = ybase32;
          const size_t cs = ochan * 4;
#pragma unroll
          for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int m0 = cb * 32 + 8 * (i >> 2) + (i & 3);
              if (!RAGGED || m0 < m_left) store_f32(yc, voff, acc[cb][r][i]);
              yc += (i & 3) == 3 ? 5 * cs : cs;
            }
        }
      }
      return;
    }
#pragma unroll
    for (int r = 0; r < WROWS; ++r) {
      const int oh = tc.th * TH + wrow0 + r;
      if (oh < p.Hout && ow >= 0 && ow < p.Wout) {
        const uint32_t voff = (uint32_t)(2 * ((size_t)(4 * kg) * ochan + (size_t)oh * p.Wout + ow));
        const char* yc = ybase;  // walks by additions, as above
        const size_t cs = ochan * 2;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
          for (int i = 0; i < 16; i += 2) {
            f32x2 v2 = {acc[cb][r][i], acc[cb][r][i + 1]};
            const uint32_t h2 = F16 ? __builtin_bit_cast(uint32_t, __builtin_convertvector(v2, f16x2))
                                                : __builtin_bit_cast(uint32_t, __builtin_convertvector(v2, bf16x2));
            const int m0 = cb * 32 + 8 * (i >> 2) + (i & 3);
            if (!RAGGED || m0 < m_left) store_bf16_lo(yc, voff, h2);
            yc += cs;
            if (!RAGGED || m0 + 1 < m_left) store_bf16_hi(yc, voff, h2);
            yc += (i & 2) ? 5 * cs : cs;
          }
      }
    }
  };
  auto epilogue = [&](const TileCoord& tc, int free_buf) {
    if (PX) epilogue_px(tc, free_buf);
    else if ((mt + 1) * MT <= p.M) epilogue_rows(tc, std::false_type{}, free_buf);
    else epilogue_rows(tc, std::true_type{}, free_buf);
  };

  // Fold-mode epilogue: a produced cell goes to the unpadded tile when it lies inside
  // [lo, lo + n) on every axis, else to the strip of the neighbour that owns it (dropped
  // when that neighbour does not exist). Values pass through `0 + v`: the sign of a
  // zero is cleared, as the reference's scatter-add does for every cell.
  auto epilogue_fold = [&](const TileCoord& tc, int free_buf) {
    // bf16 pairs of the whole accumulator first (the fp32 registers are dead after this).
    // The sign of a zero only matters where a value is zero or rounds to zero, which is
    // rare: one min3 per two values finds out, and only then the bits are patched.
    uint32_t pk[CB][WROWS][8];
    float small = 3.0e38f;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
      for (int r = 0; r < WROWS; ++r)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          small = __builtin_fminf(small, __builtin_fminf(__builtin_fabsf(acc[cb][r][i]), __builtin_fabsf(acc[cb][r][i + 1])));
          f32x2 v2 = {acc[cb][r][i], acc[cb][r][i + 1]};
          pk[cb][r][i >> 1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2, bf16x2));
        }
    if (__builtin_amdgcn_ballot_w64(!(small >= 1.0e-39f)) != 0) {  // bf16 rounds |v| <= 2^-134 to zero
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int r = 0; r < WROWS; ++r)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            uint32_t bits = pk[cb][r][j];
            if ((bits & 0x00007fffu) == 0) bits &= 0xffff0000u;
            if ((bits & 0x7fff0000u) == 0) bits &= 0x0000ffffu;
            pk[cb][r][j] = bits;
          }
    }
    const int ow = tc.tw * TW + p.org_w + wcol0 + ln;
    const int hi_d = p.Dout - p.lo_d - p.nD, hi_h = p.Hout - p.lo_h - p.nH, hi_w = p.Wout - p.lo_w - p.nW;
    const int od = tc.od;
    const int rd = od < p.lo_d ? 0 : (od < p.lo_d + p.nD ? 1 : 2);
    const int cd = od - (rd == 0 ? 0 : (rd == 1 ? p.lo_d : p.lo_d + p.nD));
    const int ed = rd == 0 ? p.lo_d : (rd == 1 ? p.nD : hi_d);
    const size_t plane0 = (size_t)tc.n * p.M + (size_t)mt * MT;
    const int th0 = tc.th * TH, tw0 = tc.tw * TW + p.org_w;
    // A tile that lies wholly inside the own extent (wave-uniform test): plain rows of
    // the unpadded tile, no per-cell routing.
    if (rd == 1 && th0 >= p.lo_h && th0 + TH <= p.lo_h + p.nH && tw0 >= p.lo_w && tw0 + TW <= p.lo_w + p.nW) {
      const size_t ps = (size_t)p.nD * p.nH * p.nW;
      char* ybase = reinterpret_cast<char*>(p.y) + 2 * (plane0 * ps + (size_t)cd * p.nH * p.nW);
      if (((tw0 - p.lo_w) & 7) == 0 && (p.nW & 7) == 0 && (reinterpret_cast<uintptr_t>(p.y) & 15) == 0) {  // uniform
        // the tile's rows start on the 16-byte grid of the unpadded tile (the host shifts the tile
        // grid to make it so): 16-byte stores through this wavefront's slice of the free stage buffer
        unsigned char* scratch =
            reinterpret_cast<unsigned char*>(lds_in + free_buf * STAGE_SLOTS) + wave * (STAGE_BYTES / WAVES);
        char* ytile = ybase + 2 * (ptrdiff_t)(tw0 - p.lo_w);
#pragma unroll
        for (int r = 0; r < WROWS; ++r) {
          const int oh = th0 + wrow0 + r - p.lo_h;
          auto pair = [&](int cb, int i) { return pk[cb][r][i >> 1]; };
          row_through_lds(scratch, pair, ytile, (uint32_t)(2 * ((size_t)oh * p.nW + wcol0)), 2 * ps);
        }
        return;
      }
      // One scalar base for the tile; the channel walks in the 32-bit lane offset (the host checks that MT
      // planes fit it): one vector add per store. A scalar base per channel cost a multiply, a 64-bit add and
      // the reload of a spilled scalar per store, three to four instructions for each 2-byte store.
      const uint32_t st = (uint32_t)(2 * ps), st5 = 5u * st;
#pragma unroll
      for (int r = 0; r < WROWS; ++r) {
        const int oh = th0 + wrow0 + r - p.lo_h;
        uint32_t vo = (uint32_t)(2 * ((size_t)(4 * kg) * ps + (size_t)oh * p.nW + (ow - p.lo_w)));
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
          for (int j = 0; j < 8; ++j) {  // channels cb * 32 + 8 * (j / 2) + 2 * (j % 2) and the one after (+ 4 kg, in vo)
            const uint32_t bits = pk[cb][r][j];
            store_bf16_lo(ybase, vo, bits);
            vo += st;
            store_bf16_hi(ybase, vo, bits);
            vo += (j & 1) ? st5 : st;
          }
      }
      return;
    }
    // Otherwise a cell goes to the unpadded tile when it lies inside [lo, lo + n) on every
    // axis, else to the strip of the neighbour that owns it (dropped when that neighbour
    // does not exist).
    const int rw = ow < p.lo_w ? 0 : (ow < p.lo_w + p.nW ? 1 : 2);
    const int cw = ow - (rw == 0 ? 0 : (rw == 1 ? p.lo_w : p.lo_w + p.nW));
    const int ew = rw == 0 ? p.lo_w : (rw == 1 ? p.nW : hi_w);
#pragma unroll
    for (int r = 0; r < WROWS; ++r) {
      const int oh = th0 + wrow0 + r;
      if (oh >= p.Hout || ow >= p.Wout || ow < 0) continue;
      const int rh = oh < p.lo_h ? 0 : (oh < p.lo_h + p.nH ? 1 : 2);
      const int ch = oh - (rh == 0 ? 0 : (rh == 1 ? p.lo_h : p.lo_h + p.nH));
      const int eh = rh == 0 ? p.lo_h : (rh == 1 ? p.nH : hi_h);
      // The row's three possible destinations (one per region across W) are read with wave-uniform indices,
      // i.e. through the scalar cache, and chosen per lane: a per-lane index into the table is a vector load,
      // and waiting for it also waits for every store the row before has just issued.
      const int slot0 = __builtin_amdgcn_readfirstlane(rd * 9 + rh * 3);
      char* const b_lo = static_cast<char*>(strip_entry(slot0));
      char* const b_mid = slot0 + 1 == 13 ? reinterpret_cast<char*>(p.y) : static_cast<char*>(strip_entry(slot0 + 1));
      char* const b_hi = static_cast<char*>(strip_entry(slot0 + 2));
      char* base = rw == 0 ? b_lo : (rw == 1 ? b_mid : b_hi);
      if (base == nullptr) continue;
      const uint32_t ps = (uint32_t)ed * (uint32_t)eh * (uint32_t)ew;  // elements per plane of that destination
      char* dst = base + 2 * ((plane0 + 4 * kg) * (size_t)ps + ((size_t)cd * eh + ch) * ew + cw);
      // bytes between produced channels (checked on the host to fit); the destination's plane size differs
      // from lane to lane, so the pointer walks by additions: a product per store is a quarter-rate
      // vector multiply
      const uint32_t step = 2u * ps, step5 = 5u * step;
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int j = 0; j < 8; ++j) {  // channels cb * 32 + 8 * (j / 2) + 2 * (j % 2) and the one after (+ 4 kg, in dst)
          const uint32_t bits = pk[cb][r][j];
          *reinterpret_cast<uint16_t*>(dst) = (uint16_t)(bits & 0xffffu);
          dst += step;
          *reinterpret_cast<uint16_t*>(dst) = (uint16_t)(bits >> 16);
          dst += (j & 1) ? step5 : step;
        }
    }
  };

  // ---- main loop over the stages (tile, 16-channel step) of this workgroup. The
  // global loads of a stage are issued a whole stage ahead: right after the previous
  // stage's registers were written to LDS, in the middle of the stage before.
  const int stages = my_tiles * p.nc16;
  auto issue_stage = [&]() __attribute__((always_inline)) {
    issue_loads();
    cursor_advance();
  };
  // Which two stage at the head of a stage (see the stage loop) was tried all ways round, in engine cycles of
  // configuration 2: forward 4 and 5: 1.18 M, 0 and 1: 1.12 M, 2 and 3: 1.14 M, 0 to 3: 1.15 M, 2 to 5: 1.17 M;
  // dgrad with the fold epilogue 4 and 5: 1.455 M, 0 and 1: 1.47 M, 0 to 3: 1.48 M, nobody or 2 to 5: 1.49 M,
  // all six: 1.59 M. (In the fold's epilogue the older wavefronts of a SIMD get their stores out first and are
  // back in the stage loop while 4 to 7 still store.)
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const bool stage_early = FOLD ? (wave_u == 4 || wave_u == 5) : (wave_u == 0 || wave_u == 1);
  // Does the epilogue put anything into the free stage buffer? Every epilogue but the fold's does (rows go
  // through LDS to leave as 16-byte pieces), and the fold's does where the tile grid lies on the 16-byte grid
  // of the unpadded gradient (the same test as in epilogue_fold; it is the same for every tile of a launch).
  const bool epilogue_uses_lds =
      !FOLD || ((((p.org_w - p.lo_w) & 7) == 0) && (p.nW & 7) == 0 && (reinterpret_cast<uintptr_t>(p.y) & 15) == 0);
  int buf = 0;
  cursor_enter(0);
  issue_stage();
  store_stage(0, 0);
  if (stages > 1) issue_stage();
  __syncthreads();
  int q = 0;
  for (int ti = 0; ti < my_tiles; ++ti) {
    init_acc();
    // a wavefront whose 4 x 32 pixels all lie outside the produced tensor (ragged last tiles) only
    // takes part in the staging and the barriers
    const TileCoord tcur = coord(tile_of(ti));
    const int wave_col = tcur.tw * TW + p.org_w + wcol0;
    const bool live = wave_col < p.Wout && wave_col + 32 > 0 && tcur.th * TH + wrow0 < p.Hout;
    int wstep = 0, wgroup = 0;
    for (int c16 = 0; c16 < p.nc16; ++c16, ++q) {
      if (p.ngroups > 1 && wstep == 0) {
        // every wavefront is past the barrier that closed the last stage of the group before
        load_weights(wgroup);
        __syncthreads();
      }
      const int wstep_next = wstep + 1 == p.wc16 ? 0 : wstep + 1;
      // Wavefronts 4 and 5 hold staging tasks like wavefronts 0..3 and share SIMD 0 and 1 with 0 and 1.
      // One of each pair stages at the head of the stage, while its SIMD's other wavefront multiplies, and that
      // one stages later, while the first multiplies; done at the same point, the two leave the matrix core idle.
      // (Not in a tile's first stage where the buffer is the last epilogue's scratch until the barrier below.)
      const bool after_epilogue = epilogue_uses_lds && c16 == 0 && ti > 0;
      const bool stage_now = stage_early && !after_epilogue;
      if (stage_now) {
        if (q + 1 < stages) store_stage(buf ^ 1, q + 1);
        if (q + 2 < stages) issue_stage();
      }
      if (live) {
        compute_kw(buf, wstep, 0, wstep_next);
        compute_kw(buf, wstep, 1, wstep_next);
      }
      // the buffer written next was the last epilogue's scratch (the fold's 2-byte stores leave from the registers:
      // nothing to wait for, and the wavefronts that are through with their stores do not wait for the others here)
      if (after_epilogue) __syncthreads();
      if (!stage_now) {
        if (q + 1 < stages) store_stage(buf ^ 1, q + 1);  // other buffer: no hazard with this stage's reads
        if (q + 2 < stages) issue_stage();
      }
      if (live) compute_kw(buf, wstep, 2, wstep_next);
      __syncthreads();
      buf ^= 1;
      if (++wstep == p.wc16) {
        wstep = 0;
        ++wgroup;
      }
    }
    // The epilogue stages its rows in the stage buffer the last stage was computed from, which is
    // free until the next stage is stored into it. That store waits (barrier above, in the first
    // stage of the next tile) until every wavefront has left this epilogue; until then a
    // wavefront that is done early already runs the next tile's MFMAs.
    if (FOLD) epilogue_fold(tcur, buf ^ 1);
    else epilogue(tcur, buf ^ 1);
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

// How a problem maps onto the kernel: produced channels in tiles of MT (M padded up to a
// multiple of 32 with zero weight rows), contraction steps of 16 channels in groups of wc16
// steps whose weights fit LDS beside the two input stages.
struct Layout {
  int MT, mtiles, nc16, wc16, ngroups;
  size_t prep_bytes, lds_bytes;
};

int pad16(int c) { return (c + CK - 1) / CK * CK; }

// K: contraction length with the channels padded to a multiple of 16 per depth tap
Layout layout_of(int K, int M) {
  Layout L;
  const int mpad = (M + 31) / 32 * 32;
  L.MT = (mpad % 64 == 0) ? 64 : 32;
  L.mtiles = mpad / L.MT;
  L.nc16 = K / CK;
  const size_t budget = 160 * 1024 - 2 * (size_t)STAGE_BYTES - L.MT * 4;
  int cap = (int)(budget / ((size_t)TAPS * 2 * L.MT * 16));
  if (cap < 1) cap = 1;
  L.wc16 = L.nc16 < cap ? L.nc16 : cap;
  if (L.wc16 < 1) L.wc16 = 1;
  L.ngroups = (L.nc16 + L.wc16 - 1) / L.wc16;
  const size_t slots = (size_t)TAPS * L.wc16 * 2 * L.MT;
  L.prep_bytes = (size_t)L.mtiles * L.ngroups * slots * 16;
  L.lds_bytes = slots * 16 + 2 * (size_t)STAGE_BYTES + L.MT * 4;
  return L;
}

// C = channels of the convolved tensor, M = produced channels
bool shape_ok(int C, int M, const ConvGeom& g) {
  if (g.k[1] != KH || g.k[2] != KW) return false;
  if (g.k[0] != 1 && g.k[0] != 3) return false;
  if (g.k[0] == 1 && (g.in[0] != 1 || g.p[0] != 0)) return false;
  for (int a = 0; a < 3; ++a)
    if (g.s[a] != 1 || g.d[a] != 1) return false;
  if (C <= 0 || M <= 0) return false;
  // per-lane byte offsets inside one batch entry are 32-bit
  const size_t in_sz = (size_t)g.in[0] * g.in[1] * g.in[2], out_sz = (size_t)g.out[0] * g.out[1] * g.out[2];
  const size_t big = in_sz > out_sz ? in_sz : out_sz;
  return big * 2 * 72 < (1ull << 31);
}

size_t prep_bytes(int K, int M) { return layout_of(K, M).prep_bytes; }

struct Launch {
  const void* x;
  const void* w;
  const void* bias;
  void* y;
  int split;                // split mode: 0 16-bit tensors as they are, 1 fp32 (six bf16 products), 2 fp16 (three)
  int f16;                  // the 16-bit tensors are fp16 (split 0 only)
  int N, C, M, KD;
  int Din, Hin, Win, Dout, Hout, Wout;
  int pad_d, pad_h, pad_w;
  int transposed;
  int fold;                 // fold mode: y is the unpadded tile, strips receive the halo cells
  int lo[3], n[3];          // own extent inside the produced tensor (fold mode)
  void* const* strips;      // 27 slots (fold mode)
  const uint16_t* xt;       // own tile for the framed input, or NULL (bf16 only)
  int tlo[3], tn[3];
};

// Bytes of the split copy of an input (its bf16 parts), rounded to 256
size_t split_bytes(size_t elements, int parts) { return (elements * parts * 2 + 255) / 256 * 256; }
size_t conv_ws_bytes(int split, int KD, int C, int M, size_t x_elements) {
  const SplitSpec sp = split_spec(split);
  const size_t prep = prep_bytes(sp.nblk * KD * pad16(C), M);
  return split ? (prep + 255) / 256 * 256 + split_bytes(x_elements, sp.parts) : prep;
}

template <typename SRC>
int split_launch(uint16_t* dst, const SRC* src, size_t batch, size_t per_batch, int parts, hipStream_t s) {
  const size_t total = batch * per_batch;
  if (total == 0) return JG_OK;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  split_kernel<SRC><<<(unsigned)blocks, 256, 0, s>>>(dst, src, per_batch, total, parts);
  JG_CHECK_LAUNCH("split_parts_bf16");
  return JG_OK;
}

int launch_conv(const Launch& L, void* ws, size_t ws_bytes, hipStream_t s, const char* who) {
  const SplitSpec sp = split_spec(L.split);
  const int nblk = sp.nblk;
  const int K = nblk * L.KD * pad16(L.C);
  const size_t x_elements = (size_t)L.N * L.C * L.Din * L.Hin * L.Win;
  const size_t need = conv_ws_bytes(L.split, L.KD, L.C, L.M, x_elements);
  if (ws == nullptr || ws_bytes < need)
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes, need);
  JG_REQUIRE((reinterpret_cast<uintptr_t>(ws) & 15) == 0, "%s: workspace must be 16-byte aligned",
             who);
  const Layout lay = layout_of(K, L.M);
  const int MT = lay.MT;
  uint16_t* wprep = static_cast<uint16_t*>(ws);
  const size_t total_w = lay.prep_bytes / 2;
  JG_REQUIRE(total_w < (1ull << 31), "%s: weight tensor too large", who);
  const uint16_t* x16 = static_cast<const uint16_t*>(L.x);
  if (L.split) {
    const unsigned wblocks = (unsigned)((total_w + 255) / 256);
    uint16_t* xs = reinterpret_cast<uint16_t*>(static_cast<char*>(ws) + (lay.prep_bytes + 255) / 256 * 256);
    int rc;
    if (L.split == 1) {
      prep_weights_split_kernel<float><<<wblocks, 256, 0, s>>>(wprep, static_cast<const float*>(L.w), L.M, L.C,
                                                                pad16(L.C), L.KD, MT, lay.mtiles, lay.wc16, lay.ngroups,
                                                                L.transposed, nblk, sp.wparts);
      rc = split_launch(xs, static_cast<const float*>(L.x), (size_t)L.N, x_elements / L.N, sp.parts, s);
    } else {
      prep_weights_split_kernel<_Float16><<<wblocks, 256, 0, s>>>(wprep, static_cast<const _Float16*>(L.w), L.M, L.C,
                                                                   pad16(L.C), L.KD, MT, lay.mtiles, lay.wc16,
                                                                   lay.ngroups, L.transposed, nblk, sp.wparts);
      rc = split_launch(xs, static_cast<const _Float16*>(L.x), (size_t)L.N, x_elements / L.N, sp.parts, s);
    }
    JG_CHECK_LAUNCH(who);
    if (rc) return rc;
    x16 = xs;
  } else {
    prep_weights_kernel<<<(unsigned)((total_w + 255) / 256), 256, 0, s>>>(wprep, static_cast<const uint16_t*>(L.w), L.M,
                                                                           L.C, pad16(L.C), L.KD, MT, lay.mtiles,
                                                                           lay.wc16, lay.ngroups, L.transposed);
    JG_CHECK_LAUNCH(who);
  }

  FwdParams p;
  p.x_end = reinterpret_cast<const char*>(x16) + 2 * x_elements * sp.parts;
  p.x = x16; p.wprep = reinterpret_cast<const u32x4*>(wprep);
  p.bias = static_cast<const uint16_t*>(L.bias); p.y = static_cast<uint16_t*>(L.y);
  p.N = L.N; p.C = L.C; p.M = L.M; p.KD = L.KD;
  p.Cp = pad16(L.C);
  p.nblk = nblk; p.Cx = sp.parts * L.C; p.xmap = sp.xparts; p.out_kind = L.f16 ? 2 : L.split;
  p.Din = L.Din; p.Hin = L.Hin; p.Win = L.Win;
  p.Dout = L.Dout; p.Hout = L.Hout; p.Wout = L.Wout;
  p.pad_d = L.pad_d; p.pad_h = L.pad_h; p.pad_w = L.pad_w;
  p.tiles_h = (L.Hout + TH - 1) / TH;
  // Where to put the tile grid. A tile's staged rows start at input column org_w + TW * tw - pad_w.
  // When the rows of x are a multiple of 128 bytes apart, an origin that makes this a multiple of
  // TW puts every staged row segment on a cache-line boundary (144 bytes: two lines instead of
  // three); it is taken when it costs no extra tile column.
  p.org_w = 0;
  // (not where it would take the 16-byte store path away: a plain 16-bit result with rows of whole pieces)
  const bool wide_rows = !L.fold && L.split != 1 && L.Wout % 8 == 0;
  if (!wide_rows && L.pad_w % TW != 0 && L.Win % 64 == 0 && (reinterpret_cast<uintptr_t>(x16) & 127) == 0) {
    const int org = L.pad_w % TW - TW;
    if ((L.Wout - org + TW - 1) / TW <= (L.Wout + TW - 1) / TW) p.org_w = org;
  }
  p.lead = (L.pad_w - p.org_w) & 1;
  p.tiles_w = (L.Wout - p.org_w + TW - 1) / TW;
  p.sw = p.tiles_w;
  const long long tiles = (long long)L.N * L.Dout * p.tiles_h * p.tiles_w;
  JG_REQUIRE(tiles < (1ll << 30), "%s: too many tiles", who);
  p.total_tiles = (int)tiles;
  p.nc16 = lay.nc16;
  p.wc16 = lay.wc16;
  p.ngroups = lay.ngroups;
  p.fold = L.fold;
  p.lo_d = L.lo[0]; p.lo_h = L.lo[1]; p.lo_w = L.lo[2];
  p.nD = L.n[0]; p.nH = L.n[1]; p.nW = L.n[2];
  p.xt = L.xt;
  p.tlo_d = L.tlo[0]; p.tlo_h = L.tlo[1]; p.tlo_w = L.tlo[2];
  p.tn_d = L.tn[0]; p.tn_h = L.tn[1]; p.tn_w = L.tn[2];
  StripTable tab;
  for (int i = 0; i < 27; ++i) tab.p[i] = (L.fold && L.strips != nullptr) ? L.strips[i] : nullptr;
  if (tiles == 0) return JG_OK;
  const size_t lds = lay.lds_bytes;
  int wgs = cu_count();
  if (wgs > tiles) wgs = (int)tiles;
  wgs = (wgs + 7) & ~7;  // whole XCD rounds
  dim3 grid((unsigned)wgs, (unsigned)lay.mtiles, 1);
  // rows of the staged windows start at even columns (`lead` sees to that): 4-byte aligned loads
  const bool even = (L.Win % 2 == 0) && ((reinterpret_cast<uintptr_t>(x16) & 3) == 0);
  void (*kern)(StripTable, FwdParams) = nullptr;
  if (L.f16 && (L.fold || L.xt != nullptr))
    JG_FAIL(JG_ERR_UNSUPPORTED, "%s: the fold epilogue and the framed input are built for bf16 only", who);
  if (L.fold) {
    if (MT == 64) kern = even ? &conv3x3_mfma_kernel<64, true, true, false> : &conv3x3_mfma_kernel<64, false, true, false>;
    else kern = even ? &conv3x3_mfma_kernel<32, true, true, false> : &conv3x3_mfma_kernel<32, false, true, false>;
  } else if (L.xt != nullptr) {
    if (MT == 64) kern = even ? &conv3x3_mfma_kernel<64, true, false, true> : &conv3x3_mfma_kernel<64, false, false, true>;
    else kern = even ? &conv3x3_mfma_kernel<32, true, false, true> : &conv3x3_mfma_kernel<32, false, false, true>;
  } else if (wide_rows && (reinterpret_cast<uintptr_t>(L.y) & 15) == 0) {
    // every row segment of the result is whole, aligned 16-byte pieces: results leave from the registers
    if (L.f16) {
      if (MT == 64)
        kern = even ? &conv3x3_mfma_kernel<64, true, false, false, true, true> : &conv3x3_mfma_kernel<64, false, false, false, true, true>;
      else
        kern = even ? &conv3x3_mfma_kernel<32, true, false, false, true, true> : &conv3x3_mfma_kernel<32, false, false, false, true, true>;
    } else {
      if (MT == 64)
        kern = even ? &conv3x3_mfma_kernel<64, true, false, false, false, true> : &conv3x3_mfma_kernel<64, false, false, false, false, true>;
      else
        kern = even ? &conv3x3_mfma_kernel<32, true, false, false, false, true> : &conv3x3_mfma_kernel<32, false, false, false, false, true>;
    }
  } else if (L.f16) {
    if (MT == 64)
      kern = even ? &conv3x3_mfma_kernel<64, true, false, false, true> : &conv3x3_mfma_kernel<64, false, false, false, true>;
    else
      kern = even ? &conv3x3_mfma_kernel<32, true, false, false, true> : &conv3x3_mfma_kernel<32, false, false, false, true>;
  } else {
    if (MT == 64) kern = even ? &conv3x3_mfma_kernel<64, true, false, false> : &conv3x3_mfma_kernel<64, false, false, false>;
    else kern = even ? &conv3x3_mfma_kernel<32, true, false, false> : &conv3x3_mfma_kernel<32, false, false, false>;
  }
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", who, lds);
  kern<<<grid, THREADS, lds, s>>>(tab, p);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

}  // namespace

namespace jg {

// fp32 runs in split mode (three bf16 parts per operand, fp32 result); its 4-byte stores halve
// the extent the 32-bit lane offsets reach.
// fp32 runs in split mode; fp16 has its own MFMA instruction and runs like bf16
static int split_mode(int dtype) { return dtype == JG_F32 ? 1 : 0; }
static bool dtype_ok(const ConvGeom& g, int dtype) {
  if (g.groups != 1) return false;  // grouped layers run the direct kernels
  if (dtype == JG_BF16 || dtype == JG_F16) return true;
  if (dtype != JG_F32) return false;
  const size_t in_sz = (size_t)g.in[0] * g.in[1] * g.in[2], out_sz = (size_t)g.out[0] * g.out[1] * g.out[2];
  const size_t big = in_sz > out_sz ? in_sz : out_sz;
  return big * 4 * 72 < (1ull << 31);
}
int split_parts_bf16(uint16_t* dst, const void* src, int src_dtype, size_t batch, size_t per_batch, hipStream_t s) {
  if (src_dtype == JG_F32) return split_launch(dst, static_cast<const float*>(src), batch, per_batch, 3, s);
  return split_launch(dst, static_cast<const _Float16*>(src), batch, per_batch, 2, s);
}

bool mfma_fwd_supported(const ConvGeom& g, int dtype) {
  return dtype_ok(g, dtype) && shape_ok(g.cin, g.cout, g) && g.batch > 0;
}
bool mfma_dgrad_supported(const ConvGeom& g, int dtype) {
  if (!dtype_ok(g, dtype) || g.batch <= 0) return false;
  for (int a = 0; a < 3; ++a)
    if (g.p[a] > g.k[a] - 1) return false;
  return shape_ok(g.cout, g.cin, g);
}

size_t mfma_fwd_workspace(const ConvGeom& g, int dtype) {
  return conv_ws_bytes(split_mode(dtype), g.k[0], g.cin, g.cout, (size_t)g.batch * g.cin * g.in[0] * g.in[1] * g.in[2]);
}
size_t mfma_dgrad_workspace(const ConvGeom& g, int dtype) {
  return conv_ws_bytes(split_mode(dtype), g.k[0], g.cout, g.cin, (size_t)g.batch * g.cout * g.out[0] * g.out[1] * g.out[2]);
}

static int fwd_launch(void* y, const void* x, const void* xt, const int* tlo, const int* tn, const void* w,
                      const void* bias, const ConvGeom& g, void* ws, size_t ws_bytes, hipStream_t s,
                      const char* who, int dtype = JG_BF16) {
  Launch L;
  L.x = x; L.w = w; L.bias = bias; L.y = y;
  L.split = split_mode(dtype);
  L.f16 = dtype == JG_F16 ? 1 : 0;
  L.N = (int)g.batch; L.C = g.cin; L.M = g.cout; L.KD = g.k[0];
  L.Din = g.in[0]; L.Hin = g.in[1]; L.Win = g.in[2];
  L.Dout = g.out[0]; L.Hout = g.out[1]; L.Wout = g.out[2];
  L.pad_d = g.p[0]; L.pad_h = g.p[1]; L.pad_w = g.p[2];
  L.transposed = 0;
  L.fold = 0;
  L.strips = nullptr;
  L.xt = static_cast<const uint16_t*>(xt);
  for (int a = 0; a < 3; ++a) {
    L.lo[a] = L.n[a] = 0;
    L.tlo[a] = tlo ? tlo[a] : 0;
    L.tn[a] = tn ? tn[a] : 0;
  }
  return launch_conv(L, ws, ws_bytes, s, who);
}

int mfma_fwd(void* y, const void* x, const void* w, const void* bias, const ConvGeom& g, void* ws,
             size_t ws_bytes, hipStream_t s, int dtype) {
  return fwd_launch(y, x, nullptr, nullptr, nullptr, w, bias, g, ws, ws_bytes, s, "jg_conv_fwd(mfma)", dtype);
}

int mfma_fwd_framed(void* y, const void* x_frame, const void* xt, const int tlo[3], const int tn[3],
                    const void* w, const void* bias, const ConvGeom& g, void* ws, size_t ws_bytes,
                    hipStream_t s) {
  return fwd_launch(y, x_frame, xt, tlo, tn, w, bias, g, ws, ws_bytes, s, "jg_conv_fwd_framed(mfma)");
}

// Bands of the padded tile that the framed kernels read from x_frame: everything a
// 16 x 64 output tile window (18 x 72 cells) touches when it does not lie inside the tile.
void mfma_frame_bands(const ConvGeom& g, const int tlo[3], const int tn[3], int band_lo[3], int band_hi[3]) {
  // depth: a stage reads one plane; planes outside the tile are read whole
  band_lo[0] = tlo[0];
  band_hi[0] = g.in[0] - tlo[0] - tn[0];
  const int tile[3] = {1, TH, TW};
  const int reach[3] = {1, IN_ROWS, OCTS * 8};  // cells a window may touch (the last octet in full)
  const int need[3] = {1, IN_ROWS, TW + KW - 1};
  for (int a = 1; a < 3; ++a) {
    const int ntiles = (g.out[a] + tile[a] - 1) / tile[a];
    int first_in = -1, last_in = -1;  // tiles whose window lies inside [tlo, tlo + tn)
    for (int t = 0; t < ntiles; ++t) {
      const int w0 = t * tile[a] - g.p[a];
      if (w0 >= tlo[a] && w0 + need[a] <= tlo[a] + tn[a]) {
        if (first_in < 0) first_in = t;
        last_in = t;
      }
    }
    if (first_in < 0) {  // no tile reads the own tile along this axis: everything from the frame
      band_lo[a] = g.in[a];
      band_hi[a] = 0;
      continue;
    }
    int lo_end = (first_in - 1) * tile[a] - g.p[a] + reach[a];  // end of the last window before
    if (first_in == 0 || lo_end < 0) lo_end = 0;
    if (lo_end > g.in[a]) lo_end = g.in[a];
    int hi_begin = (last_in + 1) * tile[a] - g.p[a];             // start of the first window after
    if (last_in == ntiles - 1 || hi_begin > g.in[a]) hi_begin = g.in[a];
    if (hi_begin < 0) hi_begin = 0;
    band_lo[a] = lo_end;
    band_hi[a] = g.in[a] - hi_begin;
  }
}

// gx = conv(go zero-padded by k-1-p, flipped / transposed weights). With `own` given,
// the produced tensor is split between the unpadded tile gx and the neighbours' strips.
static int dgrad_launch(void* gx, void* const* strips, const int* lo, const int* n, const void* w,
                        const void* go, const ConvGeom& g, void* ws, size_t ws_bytes, hipStream_t s,
                        const char* who, int dtype = JG_BF16) {
  Launch L;
  L.x = go; L.w = w; L.bias = nullptr; L.y = gx;
  L.split = split_mode(dtype);
  L.f16 = dtype == JG_F16 ? 1 : 0;
  L.N = (int)g.batch; L.C = g.cout; L.M = g.cin; L.KD = g.k[0];
  L.Din = g.out[0]; L.Hin = g.out[1]; L.Win = g.out[2];
  L.Dout = g.in[0]; L.Hout = g.in[1]; L.Wout = g.in[2];
  L.pad_d = g.k[0] - 1 - g.p[0]; L.pad_h = KH - 1 - g.p[1]; L.pad_w = KW - 1 - g.p[2];
  L.transposed = 1;
  L.fold = lo != nullptr;
  L.strips = strips;
  L.xt = nullptr;
  for (int a = 0; a < 3; ++a) {
    L.lo[a] = lo ? lo[a] : 0;
    L.n[a] = n ? n[a] : 0;
    L.tlo[a] = L.tn[a] = 0;
  }
  return launch_conv(L, ws, ws_bytes, s, who);
}

int mfma_dgrad(void* gx, const void* w, const void* go, const ConvGeom& g, void* ws,
               size_t ws_bytes, hipStream_t s, int dtype) {
  return dgrad_launch(gx, nullptr, nullptr, nullptr, w, go, g, ws, ws_bytes, s, "jg_conv_dgrad(mfma)", dtype);
}

int mfma_dgrad_fold(void* gx, void* const strips[27], const int lo[3], const int n[3], const void* w,
                    const void* go, const ConvGeom& g, void* ws, size_t ws_bytes, hipStream_t s) {
  // the fold epilogue has no path for a ragged last tile of produced channels
  const Layout lay = layout_of(g.k[0] * pad16(g.cout), g.cin);
  if (lay.mtiles * lay.MT != g.cin)
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_conv_dgrad_fold(mfma): %d input channels are not a multiple of %d", g.cin, lay.MT);
  // the epilogue addresses the MT channel planes of a tile through a 32-bit byte offset
  if ((long long)n[0] * n[1] * n[2] * 2 * lay.MT >= (1ll << 32) || (long long)g.in[0] * g.in[1] * g.in[2] * 2 * lay.MT >= (1ll << 32))
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_conv_dgrad_fold(mfma): %d planes of the tile do not fit a 32-bit offset", lay.MT);
  return dgrad_launch(gx, strips, lo, n, w, go, g, ws, ws_bytes, s, "jg_conv_dgrad_fold(mfma)");
}

}  // namespace jg
