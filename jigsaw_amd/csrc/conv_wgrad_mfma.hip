// Weight gradient of the 2-D 3x3 convolution on the bf16 matrix cores, for
// 64 -> 64 channels, stride 1, dilation 1, channels-first tensors.
//
//   gw[co][ci][kh][kw] = sum_{n,h,w} g[n][co][h][w] * x[n][ci][h+kh-ph][w+kw-pw]
//
//   GEMM view   M = output channels, N = input channels, K = pixels. Both operands
//               are pixel-contiguous in the channels-first tensors, so the tiles go
//               to LDS untransposed.
//   MFMA roles  A = g (32 channels x 16 pixels of a row), B = x (16 pixels x 32
//               channels) shifted by the tap. The kw shift is not 16-byte aligned in
//               LDS, so a lane reads 10 consecutive pixels once (b128 + b32) and
//               builds the three kw fragments with funnel shifts.
//   Workgroup   512 threads = 8 wavefronts; wavefront = (co block, ci block) pair x
//               column half. It keeps its 9 taps x 32x32 fp32 accumulators in
//               registers for the whole kernel (144 VGPRs) and walks the pixels.
//   Stage       2 output rows x 64 columns: g tile 64 x 2 x 64, x tile 64 x 4 x 66;
//               prefetched to registers during the MFMAs of the previous stage,
//               double buffered in LDS (one barrier per stage). Channel strides in
//               LDS are odd multiples of 16 bytes so that the 32 channel-lanes of a
//               fragment read hit distinct banks.
//   Reduction   every workgroup writes its partial (2 halves) to the workspace; a
//               second kernel sums the partials in a fixed order (deterministic) and
//               writes gw in the weight layout.
#include "conv_common.h"

namespace {

using jg::ConvGeom;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

constexpr int C = 64;                 // channels on both sides
constexpr int THREADS = 512;
constexpr int SR = 2, SW = 64;        // output rows / columns per stage
constexpr int XR = SR + 2;            // x rows per stage
constexpr int G_CH = SR * SW * 2 + 16;        // 272 bytes per g channel
constexpr int X_ROW = 144;                    // 72 pixels
constexpr int X_CH = XR * X_ROW + 16;         // 592 bytes per x channel
constexpr int G_BYTES = C * G_CH;             // 17408
constexpr int X_BYTES = C * X_CH;             // 37888
constexpr int STAGE_BYTES = G_BYTES + X_BYTES;
constexpr int G_CHUNKS = C * SR * (SW / 8);   // 1024 chunks of 8 pixels
constexpr int X_CPR = 9;                      // chunks per x row (72 pixels)
constexpr int X_CHUNKS = C * XR * X_CPR;      // 2304
constexpr int CHUNKS = G_CHUNKS + X_CHUNKS;   // 3328
constexpr int ROUNDS = (CHUNKS + THREADS - 1) / THREADS;  // 7
constexpr int PART = C * C * 9;               // floats per partial

struct WgradParams {
  const uint16_t* x;  // (N, 64, Hin, Win)
  const uint16_t* g;  // (N, 64, Hout, Wout)
  float* part;        // [slots][tap][co][ci]
  int N, Hin, Win, Hout, Wout, pad_h, pad_w;
  int row_pairs, col_tiles;
  int total_stages;   // N * col_tiles * row_pairs
};

template <bool EVEN>
__global__ __launch_bounds__(THREADS) void wgrad3x3_mfma_kernel(WgradParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kgp = lane >> 5;
  const int pair = wave & 3, half = wave >> 2;
  const int cb = pair >> 1, ib = pair & 1;

  // contiguous range of stages for this workgroup; stage -> (n, column tile, row pair),
  // row pair fastest, so consecutive stages walk down one column of one image
  const long long per = ((long long)p.total_stages + gridDim.x - 1) / gridDim.x;
  const long long s_begin = per * blockIdx.x;
  long long s_end = s_begin + per;
  if (s_end > p.total_stages) s_end = p.total_stages;

  const size_t plane_x = (size_t)p.Hin * p.Win, plane_g = (size_t)p.Hout * p.Wout;

  // chunk bookkeeping (fixed per thread): which 8 pixels of which channel / row
  u32x4 stg[ROUNDS];
  auto issue_loads = [&](long long stage) {
    const int hp = (int)(stage % p.row_pairs);
    const long long t = stage / p.row_pairs;
    const int ct = (int)(t % p.col_tiles);
    const int n = (int)(t / p.col_tiles);
    const int oh0 = hp * SR, ow0 = ct * SW;
    const int ih0 = oh0 - p.pad_h, iw0 = ow0 - p.pad_w;
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int q = tid + rd * THREADS;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (q < G_CHUNKS) {
        const int c8 = q & 7, r = (q >> 3) & (SR - 1), ch = q >> 4;
        const int oh = oh0 + r, ow = ow0 + c8 * 8;
        const uint16_t* src = p.g + ((size_t)n * C + ch) * plane_g + (size_t)oh * p.Wout + ow;
        if (oh < p.Hout) {
          if (ow + 8 <= p.Wout && (reinterpret_cast<uintptr_t>(src) & 3) == 0) {
            v = *reinterpret_cast<const u32x4_a4*>(src);
          } else {
            uint32_t e[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) e[k] = (ow + k < p.Wout) ? (uint32_t)src[k] : 0u;
            v.x = e[0] | (e[1] << 16); v.y = e[2] | (e[3] << 16);
            v.z = e[4] | (e[5] << 16); v.w = e[6] | (e[7] << 16);
          }
        }
      } else if (q < CHUNKS) {
        const int qx = q - G_CHUNKS;
        const int c9 = qx % X_CPR;
        const int rr = qx / X_CPR;
        const int rho = rr & (XR - 1), ch = rr >> 2;
        const int ih = ih0 + rho, iw = iw0 + c9 * 8;
        const uint16_t* src = p.x + ((size_t)n * C + ch) * plane_x + (ptrdiff_t)ih * p.Win + iw;
        if (ih >= 0 && ih < p.Hin) {
          if (EVEN && iw >= 0 && iw + 8 <= p.Win) {
            v = *reinterpret_cast<const u32x4_a4*>(src);
          } else {
            uint32_t e[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) e[k] = (iw + k >= 0 && iw + k < p.Win) ? (uint32_t)src[k] : 0u;
            v.x = e[0] | (e[1] << 16); v.y = e[2] | (e[3] << 16);
            v.z = e[4] | (e[5] << 16); v.w = e[6] | (e[7] << 16);
          }
        }
      }
      stg[rd] = v;
    }
  };

  auto store_stage = [&](int buf) {
    unsigned char* base = smem + buf * STAGE_BYTES;
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int q = tid + rd * THREADS;
      if (q < G_CHUNKS) {
        const int c8 = q & 7, r = (q >> 3) & (SR - 1), ch = q >> 4;
        *reinterpret_cast<u32x4*>(base + ch * G_CH + r * (SW * 2) + c8 * 16) = stg[rd];
      } else if (q < CHUNKS) {
        const int qx = q - G_CHUNKS;
        const int c9 = qx % X_CPR;
        const int rr = qx / X_CPR;
        const int rho = rr & (XR - 1), ch = rr >> 2;
        *reinterpret_cast<u32x4*>(base + G_BYTES + ch * X_CH + rho * X_ROW + c9 * 16) = stg[rd];
      }
    }
  };

  f32x16 acc[3][3];
#pragma unroll
  for (int a = 0; a < 3; ++a)
#pragma unroll
    for (int b = 0; b < 3; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.0f;

  auto compute_stage = [&](int buf) {
    const unsigned char* gb = smem + buf * STAGE_BYTES + (cb * 32 + ln) * G_CH + kgp * 16;
    const unsigned char* xb = smem + buf * STAGE_BYTES + G_BYTES + (ib * 32 + ln) * X_CH + kgp * 16;
#pragma unroll
    for (int cgi = 0; cgi < 2; ++cgi) {
      const int cg = half * 2 + cgi;  // 16-pixel column group of this wavefront
      bf16x8 a[SR];
#pragma unroll
      for (int r = 0; r < SR; ++r)
        a[r] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(gb + r * (SW * 2) + cg * 32));
#pragma unroll
      for (int rho = 0; rho < XR; ++rho) {
        const u32x4 d = *reinterpret_cast<const u32x4*>(xb + rho * X_ROW + cg * 32);
        const uint32_t d4 = *reinterpret_cast<const uint32_t*>(xb + rho * X_ROW + cg * 32 + 16);
        u32x4 s1, s2;
        s1.x = __builtin_amdgcn_alignbit(d.y, d.x, 16);
        s1.y = __builtin_amdgcn_alignbit(d.z, d.y, 16);
        s1.z = __builtin_amdgcn_alignbit(d.w, d.z, 16);
        s1.w = __builtin_amdgcn_alignbit(d4, d.w, 16);
        s2.x = d.y; s2.y = d.z; s2.z = d.w; s2.w = d4;
        const bf16x8 b0 = __builtin_bit_cast(bf16x8, d);
        const bf16x8 b1 = __builtin_bit_cast(bf16x8, s1);
        const bf16x8 b2 = __builtin_bit_cast(bf16x8, s2);
#pragma unroll
        for (int r = 0; r < SR; ++r) {
          const int kh = rho - r;
          if (kh >= 0 && kh < 3) {
            acc[kh][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r], b0, acc[kh][0], 0, 0, 0);
            acc[kh][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r], b1, acc[kh][1], 0, 0, 0);
            acc[kh][2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r], b2, acc[kh][2], 0, 0, 0);
          }
        }
      }
    }
  };

  if (s_begin < s_end) {
    int buf = 0;
    issue_loads(s_begin);
    store_stage(0);
    __syncthreads();
    for (long long st = s_begin; st < s_end; ++st) {
      const bool has_next = st + 1 < s_end;
      if (has_next) issue_loads(st + 1);
      compute_stage(buf);
      if (has_next) store_stage(buf ^ 1);
      __syncthreads();
      buf ^= 1;
    }
  }

  // partial of this wavefront: slot = workgroup * 2 + half, layout [tap][co][ci]
  float* out = p.part + ((size_t)blockIdx.x * 2 + half) * PART;
#pragma unroll
  for (int kh = 0; kh < 3; ++kh)
#pragma unroll
    for (int kw = 0; kw < 3; ++kw)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int co = cb * 32 + 8 * (i >> 2) + 4 * kgp + (i & 3);
        out[((kh * 3 + kw) * C + co) * C + ib * 32 + ln] = acc[kh][kw][i];
      }
}

// out[co][ci][tap] (bf16) = sum over slots of part[slot][tap][co][ci], fixed order.
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(uint16_t* __restrict__ gw,
                                                           const float* __restrict__ part,
                                                           int slots) {
  const int i = blockIdx.x * 256 + threadIdx.x;  // index in [tap][co][ci]
  if (i >= PART) return;
  // four independent chains keep the loads in flight; the order stays fixed
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  int k = 0;
  for (; k + 4 <= slots; k += 4) {
    s0 += part[(size_t)(k + 0) * PART + i];
    s1 += part[(size_t)(k + 1) * PART + i];
    s2 += part[(size_t)(k + 2) * PART + i];
    s3 += part[(size_t)(k + 3) * PART + i];
  }
  for (; k < slots; ++k) s0 += part[(size_t)k * PART + i];
  const float s = (s0 + s1) + (s2 + s3);
  const int ci = i % C, co = (i / C) % C, tap = i / (C * C);
  gw[(co * C + ci) * 9 + tap] = jg::f32_to_bf16(s);
}

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

int wg_count(long long stages) {
  long long n = cu_count();
  if (n > stages) n = stages;
  if (n < 1) n = 1;
  return (int)n;
}

long long stage_count(const ConvGeom& g) {
  return g.batch * ((g.out[1] + SR - 1) / SR) * ((g.out[2] + SW - 1) / SW);
}

}  // namespace

namespace jg {

bool mfma_wgrad_supported(const ConvGeom& g, int dtype) {
  if (dtype != JG_BF16 || g.batch <= 0) return false;
  if (g.in[0] != 1 || g.k[0] != 1) return false;
  if (g.k[1] != 3 || g.k[2] != 3) return false;
  if (g.s[1] != 1 || g.s[2] != 1 || g.d[1] != 1 || g.d[2] != 1) return false;
  if (g.cin != C || g.cout != C) return false;
  return stage_count(g) < (1ll << 40);
}

size_t mfma_wgrad_workspace(const ConvGeom& g) {
  return (size_t)wg_count(stage_count(g)) * 2 * PART * sizeof(float);
}

int mfma_wgrad(void* gw, const void* x, const void* go, const ConvGeom& g, void* ws,
               size_t ws_bytes, hipStream_t s) {
  const char* who = "jg_conv_wgrad(mfma)";
  if (ws == nullptr || ws_bytes < mfma_wgrad_workspace(g))
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes,
            mfma_wgrad_workspace(g));
  JG_REQUIRE((reinterpret_cast<uintptr_t>(ws) & 15) == 0, "%s: workspace must be 16-byte aligned",
             who);
  WgradParams p;
  p.x = static_cast<const uint16_t*>(x);
  p.g = static_cast<const uint16_t*>(go);
  p.part = static_cast<float*>(ws);
  p.N = (int)g.batch;
  p.Hin = g.in[1]; p.Win = g.in[2]; p.Hout = g.out[1]; p.Wout = g.out[2];
  p.pad_h = g.p[1]; p.pad_w = g.p[2];
  p.row_pairs = (g.out[1] + SR - 1) / SR;
  p.col_tiles = (g.out[2] + SW - 1) / SW;
  const long long stages = stage_count(g);
  JG_REQUIRE(stages < (1ll << 31), "%s: too many stages", who);
  p.total_stages = (int)stages;
  const int wgs = wg_count(stages);
  const bool even = (p.Win % 2 == 0) && (p.pad_w % 2 == 0) &&
                    ((reinterpret_cast<uintptr_t>(x) & 3) == 0);
  const size_t lds = 2 * (size_t)STAGE_BYTES;
  void (*kern)(WgradParams) = even ? &wgrad3x3_mfma_kernel<true> : &wgrad3x3_mfma_kernel<false>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", who, lds);
  kern<<<wgs, THREADS, lds, s>>>(p);
  JG_CHECK_LAUNCH(who);
  wgrad_reduce_kernel<<<(PART + 255) / 256, 256, 0, s>>>(static_cast<uint16_t*>(gw), p.part,
                                                         wgs * 2);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

}  // namespace jg
