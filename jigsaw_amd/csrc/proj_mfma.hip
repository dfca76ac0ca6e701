// Token projections around the attention core, with the head split / head merge done
// by the addressing of the GEMM instead of by a copy.
//
// Reference behaviour restated here (jigsaw/modules/attention/_attention.py:881-918):
//   qkv = self.qkv(x)                                   (rows, C) x (3 h d, C)^T + bias
//   rearrange(qkv, "... n s (three h d) -> three ... n h s d")
//   out = attn_core(q, k, v)                            (..., h, s, d)
//   rearrange(out, "... n h s d -> ... n s (h d)").contiguous(); self.head_concat(out)
//
// A matrix operand or result with rows = tokens and columns = features is addressed
// through a Map: either row-major (row * ld + feature), or "heads": the tensor is
// (t, B, H, S, D), token = b * S + s, feature = (t * H + h) * D + d. In both cases
// the element offset is row_part(token) + feat_part(feature), and 8 consecutive
// features starting at a multiple of 8 are contiguous (D % 8 == 0).
//
//   proj_nt_kernel   out(r, n) = sum_k a(r, k) * w[n][k] + bias[n]      (forward, and the
//                    input gradients with the transposed weight)
//   proj_tn_kernel   part[split](n, c) = sum_{r in split} g(r, n) * x(r, c)   (weight gradient;
//                    bias gradient sum_r g(r, n) on the way), then proj_reduce_kernel
//
// bf16 on v_mfma_f32_32x32x16_bf16 with fp32 accumulation. Workgroup tile 128 x 128, four
// wavefronts of 64 x 64 (2 x 2 MFMA blocks); operands are staged through LDS in 16-byte
// slots of 8 contraction elements, fetched to registers one stage ahead of the MFMAs.
// proj_generic_kernel covers the other dtypes and unaligned shapes with plain FMAs.
#include "jg_common.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

struct Map {
  int heads;     // 0: row-major with leading dimension ld; 1: (t, B, H, S, D)
  long long ld;
  int B, H, S, D;
};

__device__ __forceinline__ long long row_part(const Map& m, long long r) {
  if (!m.heads) return r * m.ld;
  const long long b = r / m.S, s = r - b * m.S;
  return (b * m.H * m.S + s) * m.D;
}
__device__ __forceinline__ long long feat_part(const Map& m, int j) {
  if (!m.heads) return j;
  const int hd = j / m.D, d = j - hd * m.D;
  const int t = hd / m.H, h = hd - t * m.H;
  return ((long long)t * m.B * m.H + h) * m.S * m.D + d;
}

// Walks consecutive tokens without a division per token.
struct RowWalk {
  long long b, s;  // heads: batch entry and position; row-major: s = token
  __device__ __forceinline__ void start(const Map& m, long long r) {
    if (m.heads) {
      b = r / m.S;
      s = r - b * m.S;
    } else {
      b = 0;
      s = r;
    }
  }
  __device__ __forceinline__ void advance(const Map& m, int by) {
    s += by;
    if (m.heads)
      while (s >= m.S) {
        s -= m.S;
        ++b;
      }
  }
  __device__ __forceinline__ long long part(const Map& m) const {
    return m.heads ? (b * m.H * m.S + s) * m.D : s * m.ld;
  }
};


// ------------------------------------------------------------------------ NT
constexpr int BK = 64;  // contraction elements per stage

struct NtParams {
  const uint16_t* a;
  const uint16_t* w;     // (N, K) row-major
  const uint16_t* bias;  // (N,) or NULL
  uint16_t* out;
  Map am, om;
  long long rows;
  int N, K;
  int tiles_n;
  // What happens to a result on its way out (the values are the bf16-rounded acc + bias, as a
  // separate elementwise pass over the stored tensor would see them; arithmetic in fp32):
  //   EPI_NONE  out = y
  //   EPI_GELU  out = y, aux = gelu(y)                (aux is written)
  //   EPI_DGELU out = y * gelu'(aux)                  (aux is read: the saved pre-activation)
  //   EPI_ADD   out = y + aux                         (aux is read: the residual)
  // aux has the layout of out.
  int epi;
  uint16_t* aux;
};
constexpr int EPI_NONE = 0, EPI_GELU = 1, EPI_DGELU = 2, EPI_ADD = 3;

// GELU in its erf form (torch.nn.GELU's default) and its derivative. (1 + erf(z)) / 2 with z = h / sqrt 2 from
// the rational approximation 7.1.26 of Abramowitz & Stegun, erfc |z| = p(t) exp(-z^2), t = 1 / (1 + 0.3275911 |z|),
// absolute error below 1.5e-7 (the results are rounded to 16 bits): one reciprocal, one exponential and
// five multiply-adds where the library's erff took the epilogue of the MLP's two fused GEMMs most of
// their time. Negative z takes erfc |z| / 2 directly, so the small values there keep their relative accuracy;
// exp(-z^2) = exp(-h^2 / 2) is also what the derivative's density term needs.
__device__ __forceinline__ float half_one_plus_erf(float h, float* density_exp) {
  const float az = __builtin_fabsf(h) * 0.70710678118654752f;
  const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, az, 1.0f));
  float poly = __builtin_fmaf(1.061405429f, t, -1.453152027f);
  poly = __builtin_fmaf(poly, t, 1.421413741f);
  poly = __builtin_fmaf(poly, t, -0.284496736f);
  poly = __builtin_fmaf(poly, t, 0.254829592f);
  const float e = __expf(-az * az);
  const float half_erfc = 0.5f * poly * t * e;
  *density_exp = e;
  return h >= 0.0f ? 1.0f - half_erfc : half_erfc;
}
__device__ __forceinline__ float gelu_f(float h) {
  float e;
  return h * half_one_plus_erf(h, &e);
}
__device__ __forceinline__ float dgelu_f(float h) {
  float e;
  const float cdf = half_one_plus_erf(h, &e);
  return __builtin_fmaf(h * 0.3989422804014327f, e, cdf);
}
// op on 8 bf16 values packed in 16 bytes (second operand optional)
template <typename F>
__device__ __forceinline__ u32x4 map8(u32x4 y, u32x4 r, F f) {
  uint32_t yy[4] = {y.x, y.y, y.z, y.w}, rr[4] = {r.x, r.y, r.z, r.w}, oo[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const f32x2 v = {f(__uint_as_float(yy[i] << 16), __uint_as_float(rr[i] << 16)),
                     f(__uint_as_float(yy[i] & 0xffff0000u), __uint_as_float(rr[i] & 0xffff0000u))};
    oo[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  }
  return u32x4{oo[0], oo[1], oo[2], oo[3]};
}

// Shape of a workgroup: WM x WN wavefronts, each with IM x JN blocks of 32 tokens x 32 features.
template <int IM, int JN, int WM, int WN>
struct NtShape {
  static constexpr int TM = 32 * IM * WM, TNF = 32 * JN * WN;  // tokens, features of a tile
  static constexpr int THREADS = 64 * WM * WN;
  static constexpr int OP_A = 8 * TM, OP_W = 8 * TNF;          // 16-byte slots per stage: [chunk of 8 k][row ^ 2 chunk]
  static constexpr int STAGE = OP_A + OP_W;
  static constexpr int OUT_PITCH = TNF + 8;                    // elements per token row of the result tile in LDS
  static constexpr int MAIN = 2 * STAGE * 16 > TM * OUT_PITCH * 2 ? 2 * STAGE * 16 : TM * OUT_PITCH * 2;
  static constexpr int LDS = MAIN + TNF * 4;                   // then the bias of the tile as floats
  static constexpr int PASS_A = TM * 8 / THREADS, PASS_W = TNF * 8 / THREADS;
  static_assert(TM * 8 % THREADS == 0 && TNF * 8 % THREADS == 0, "whole load passes");
};

template <int IM, int JN, int WM, int WN>
__global__ __launch_bounds__(64 * WM * WN) void proj_nt_kernel(NtParams p) {
  typedef NtShape<IM, JN, WM, WN> SH;
  constexpr int TM = SH::TM, TNF = SH::TNF, THREADS = SH::THREADS;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  u32x4* lds = reinterpret_cast<u32x4*>(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int wm = wave % WM, wn = wave / WM;
  // Workgroups go to the 8 XCDs round-robin; give each XCD a contiguous range of tiles, so that the
  // tiles that share a panel of `a` (consecutive ids) meet in one L2.
  const unsigned per_xcd = gridDim.x / 8;
  const unsigned tile_id = blockIdx.x < per_xcd * 8 ? (blockIdx.x % 8) * per_xcd + blockIdx.x / 8 : blockIdx.x;
  const long long m0 = (long long)(tile_id / p.tiles_n) * TM;
  const int n0 = (tile_id % p.tiles_n) * TNF;
  if (tid < TNF)  // read after the barriers of the stage loop
    reinterpret_cast<float*>(smem + SH::MAIN)[tid] =
        (p.bias != nullptr && n0 + tid < p.N) ? jg::bf16_to_f32(p.bias[n0 + tid]) : 0.0f;

  // loads of a stage: chunk column c, rows tid / 8 + (THREADS / 8) i of both operands
  constexpr int RSTEP = THREADS / 8;
  const int c = tid & 7, lrow = tid >> 3;
  // byte offsets from the start of a / w: 32 bits (the host checks the tensor sizes), so that a
  // load takes the uniform base from scalar registers and one vector register per address
  uint32_t a_row[SH::PASS_A], w_row[SH::PASS_W];
#pragma unroll
  for (int i = 0; i < SH::PASS_A; ++i) {
    long long r = m0 + lrow + RSTEP * i;
    if (r > p.rows - 1) r = p.rows - 1;  // a row past the end repeats the last one and is dropped
    a_row[i] = (uint32_t)(row_part(p.am, r) * 2);
  }
#pragma unroll
  for (int i = 0; i < SH::PASS_W; ++i) {
    int n = n0 + lrow + RSTEP * i;
    if (n > p.N - 1) n = p.N - 1;
    w_row[i] = (uint32_t)((long long)n * p.K * 2);
  }
  const char* a_bytes = reinterpret_cast<const char*>(p.a);
  const char* w_bytes = reinterpret_cast<const char*>(p.w);
  u32x4 ra[SH::PASS_A], rw[SH::PASS_W];
  bool ld_ok = true;
  auto load = [&](int ks) {
    const int k = ks * BK + c * 8;
    ld_ok = k < p.K;  // a chunk past the contraction length is read at k = 0 and zeroed on the way to LDS
    const int kk = ld_ok ? k : 0;
    const uint32_t fa = (uint32_t)(feat_part(p.am, kk) * 2), fw = (uint32_t)kk * 2;
#pragma unroll
    for (int i = 0; i < SH::PASS_A; ++i) ra[i] = *reinterpret_cast<const u32x4*>(a_bytes + (size_t)(a_row[i] + fa));
#pragma unroll
    for (int i = 0; i < SH::PASS_W; ++i) rw[i] = *reinterpret_cast<const u32x4*>(w_bytes + (size_t)(w_row[i] + fw));
  };
  auto store = [&](int buf) {
    u32x4* sa = lds + buf * SH::STAGE;
    u32x4* sw = sa + SH::OP_A;
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < SH::PASS_A; ++i) sa[c * TM + ((lrow + RSTEP * i) ^ (2 * c))] = ld_ok ? ra[i] : zero;
#pragma unroll
    for (int i = 0; i < SH::PASS_W; ++i) sw[c * TNF + ((lrow + RSTEP * i) ^ (2 * c))] = ld_ok ? rw[i] : zero;
  };

  f32x16 acc[IM][JN];
#pragma unroll
  for (int i = 0; i < IM; ++i)
#pragma unroll
    for (int j = 0; j < JN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // acc[i][j] = w fragment (rows: features) x a fragment (columns: tokens). The fragments of
  // the next 16-wide step are requested before the MFMAs of this one are issued.
  auto compute = [&](int buf) {
    const u32x4* sa = lds + buf * SH::STAGE;
    const u32x4* sw = sa + SH::OP_A;
    u32x4 fr[2][IM + JN];
    auto fetch = [&](int kk, u32x4 (&f)[IM + JN]) {
      const int cc = kk * 2 + kg;
#pragma unroll
      for (int t = 0; t < IM; ++t) f[t] = sa[cc * TM + ((wm * 32 * IM + t * 32 + ln) ^ (2 * cc))];
#pragma unroll
      for (int t = 0; t < JN; ++t) f[IM + t] = sw[cc * TNF + ((wn * 32 * JN + t * 32 + ln) ^ (2 * cc))];
    };
    fetch(0, fr[0]);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      if (kk + 1 < BK / 16) fetch(kk + 1, fr[(kk + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int j = 0; j < JN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fr[kk & 1][IM + j]),
                                                              __builtin_bit_cast(bf16x8, fr[kk & 1][i]), acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  const int nk = (p.K + BK - 1) / BK;
  load(0);
  store(0);
  __syncthreads();
  for (int ks = 0; ks < nk; ++ks) {
    if (ks + 1 < nk) load(ks + 1);
    compute(ks & 1);
    if (ks + 1 < nk) store((ks + 1) & 1);
    __syncthreads();
  }

  // Accumulator lane (ln, kg), register e of block (i, j): feature (wn*JN + j)*32 + 8*(e/4) +
  // 4*kg + e%4, token (wm*IM + i)*32 + ln. The tile goes to LDS as bf16 [token][feature]
  // (the stages are done with), and leaves it in 16-byte pieces of 8 features.
  uint16_t* tile = reinterpret_cast<uint16_t*>(smem);
  const float* lds_bias = reinterpret_cast<const float*>(smem + SH::MAIN);
#pragma unroll
  for (int i = 0; i < IM; ++i)
#pragma unroll
    for (int j = 0; j < JN; ++j)
#pragma unroll
      for (int e4 = 0; e4 < 4; ++e4) {
        const int f = (wn * JN + j) * 32 + e4 * 8 + kg * 4;
        const int tok = (wm * IM + i) * 32 + ln;
        const f32x4 bq = *reinterpret_cast<const f32x4*>(lds_bias + f);
        const f32x2 lo = {acc[i][j][e4 * 4 + 0] + bq.x, acc[i][j][e4 * 4 + 1] + bq.y};
        const f32x2 hi = {acc[i][j][e4 * 4 + 2] + bq.z, acc[i][j][e4 * 4 + 3] + bq.w};
        u32x2 pk;
        pk.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2));
        pk.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2));
        *reinterpret_cast<u32x2*>(tile + tok * SH::OUT_PITCH + f) = pk;
      }
  __syncthreads();
  {
    constexpr int CPR = TNF / 8, RPP = THREADS / CPR;  // 16-byte pieces per token row, rows per pass
    const int fc = tid % CPR, trow = tid / CPR;
    const int n = n0 + fc * 8;
    const long long fo = feat_part(p.om, n < p.N ? n : 0);
    RowWalk rwk;
    rwk.start(p.om, m0 + trow);
#pragma unroll 4
    for (int q = 0; q < TM / RPP; ++q) {
      const long long r = m0 + trow + RPP * q;
      if (r < p.rows && n < p.N) {
        const long long at = rwk.part(p.om) + fo;
        u32x4 y = *reinterpret_cast<const u32x4*>(tile + (trow + RPP * q) * SH::OUT_PITCH + fc * 8);
        if (p.epi == EPI_GELU) {
          *reinterpret_cast<u32x4*>(p.aux + at) = map8(y, y, [](float h, float) { return gelu_f(h); });
        } else if (p.epi == EPI_DGELU) {
          y = map8(y, *reinterpret_cast<const u32x4*>(p.aux + at), [](float g, float h) { return g * dgelu_f(h); });
        } else if (p.epi == EPI_ADD) {
          y = map8(y, *reinterpret_cast<const u32x4*>(p.aux + at), [](float a, float b) { return a + b; });
        }
        *reinterpret_cast<u32x4*>(p.out + at) = y;
      }
      rwk.advance(p.om, RPP);
    }
  }
}

template <int IM, int JN, int WM, int WN>
int launch_nt(NtParams& p, hipStream_t s, const char* who) {
  typedef NtShape<IM, JN, WM, WN> SH;
  p.tiles_n = jg::cdiv(p.N, SH::TNF);
  const long long tiles = (long long)jg::cdiv(p.rows, SH::TM) * p.tiles_n;
  JG_REQUIRE(tiles < (1ll << 31), "%s: too many tiles", who);
  void (*kern)(NtParams) = &proj_nt_kernel<IM, JN, WM, WN>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     SH::LDS);
  if (e != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS", who, SH::LDS);
  kern<<<(unsigned)tiles, SH::THREADS, SH::LDS, s>>>(p);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

// ------------------------------------------------------------------------ TN
constexpr int BR = 64;  // tokens per stage

struct TnParams {
  const uint16_t* g;  // tokens x N
  const uint16_t* x;  // tokens x C
  float* part;        // [split][N][C]
  float* bias_part;   // [split][N] or NULL
  Map gm, xm;
  long long rows;
  int N, C;
  int tiles_c;        // column tiles; blockIdx.x = (tile_n * tiles_c + tile_c), blockIdx.y = split
  int stages_per_split;
};

// WM x WN wavefronts, each with IM x JN blocks of 32 features of g x 32 features of x; the tile is
// square (T x T) and the workgroup has 2 T threads: one 8 token x 8 feature block per thread and stage.
template <int IM, int JN, int WM, int WN>
struct TnShape {
  static constexpr int T = 32 * IM * WM;
  static_assert(T == 32 * JN * WN, "square tile");
  static constexpr int THREADS = 64 * WM * WN;
  static_assert(THREADS == 2 * T, "one block per thread");
  static constexpr int PITCH = T + T / 8;  // slots per chunk of 8 tokens: feature f at f + f / 8
  static constexpr int OP = 8 * PITCH;
  static constexpr int STAGE = 2 * OP;
  static constexpr int LDS = 2 * STAGE * 16;
};

// acc + the eight bf16 values of v. Plain shifts and adds: v_dot2c_f32_bf16 against a pair of ones is a
// quarter of the instructions and gave the right sums by itself, but wrong ones in this kernel (chains of
// dependent dot instructions), so it is not used.
__device__ __forceinline__ float add_bf16x8(float acc, const u32x4& v) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    acc += __builtin_bit_cast(float, v[j] << 16);
    acc += __builtin_bit_cast(float, v[j] & 0xffff0000u);
  }
  return acc;
}

template <int IM, int JN, int WM, int WN, int AHEAD>
__global__ __launch_bounds__(64 * WM * WN) void proj_tn_kernel(TnParams p) {
  typedef TnShape<IM, JN, WM, WN> SH;
  constexpr int T = SH::T;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  u32x4* lds = reinterpret_cast<u32x4*>(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int wn = wave % WM, wc = wave / WM;
  const int tile_c = blockIdx.x % p.tiles_c, tile_n = blockIdx.x / p.tiles_c;
  const int n0 = tile_n * T, c0 = tile_c * T;
  const int split = blockIdx.y;
  const long long r_first = (long long)split * p.stages_per_split * BR;
  long long r_last = r_first + (long long)p.stages_per_split * BR;
  if (r_last > p.rows) r_last = p.rows;
  const int nst = r_last > r_first ? (int)((r_last - r_first + BR - 1) / BR) : 0;

  // loads: the first half of the threads fetches g, the second x; a thread owns an 8 token x 8 feature block
  // `half` is the same for a whole wavefront (T is a multiple of 64). The operand's map is copied
  // field by field: a reference chosen per thread (`half ? p.xm : p.gm`) made the compiler keep a
  // pointer to the argument and re-read the fields from memory in every stage, each read followed by a
  // wait for ALL outstanding loads, the staged ones included, which undid the lookahead below.
  const int half = __builtin_amdgcn_readfirstlane(tid / T), tt = tid % T;
  const int jc = tt % (T / 8), ro = tt / (T / 8);
  Map mp;
  mp.heads = half ? p.xm.heads : p.gm.heads;
  mp.ld = half ? p.xm.ld : p.gm.ld;
  mp.B = half ? p.xm.B : p.gm.B;
  mp.H = half ? p.xm.H : p.gm.H;
  mp.S = half ? p.xm.S : p.gm.S;
  mp.D = half ? p.xm.D : p.gm.D;
  const uint16_t* src = half ? p.x : p.g;
  const int f_count = half ? p.C : p.N;
  int f = (half ? c0 : n0) + jc * 8;
  if (f > f_count - 8) f = f_count - 8;  // a block past the last feature repeats the last one and is dropped
  const long long fpart = feat_part(mp, f);
  RowWalk walk;
  walk.start(mp, r_first + ro * 8);
  const bool want_bias = (p.bias_part != nullptr) && half == 0 && tile_c == 0;
  float bsum[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) bsum[j] = 0.0f;

  // AHEAD register sets: the loads of stage st + AHEAD are issued at the head of stage st (into the set
  // stage st was stored from), so a load has AHEAD - 1 whole stages to arrive before its registers go to
  // LDS. With one set a workgroup moved 32 KB per memory latency: a stage's matrix instructions take a
  // quarter of one.
  u32x4 vs[AHEAD][8];
  long long rl[AHEAD];
  const uint32_t tok_stride32 = (uint32_t)(mp.heads ? mp.D : mp.ld);  // between consecutive tokens of one batch entry
  uint32_t tok_off[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) tok_off[i] = (uint32_t)i * tok_stride32;
  auto load = [&](int st, u32x4 (&v)[8], long long& r_loaded) {
    // tokens r_first + st*BR + ro*8 + i, all of one batch entry (S % 8 == 0); `walk` stands at i = 0.
    // A token past the end repeats the last one (or token 0) and is zeroed on the way to LDS.
    r_loaded = r_first + (long long)st * BR + ro * 8;
    const long long left = p.rows - r_loaded;
    const int last = left >= 8 ? 7 : (left > 0 ? (int)left - 1 : 0);
    const uint16_t* b0 = src + (left > 0 ? walk.part(mp) : 0) + fpart;
    // 32-bit element offsets inside the block of eight tokens (the host checks that 7 strides fit): the eight
    // products are made once; a block cut short by the end of the tensor repeats its last token
    const uint32_t last_off = (uint32_t)last * tok_stride32;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = *reinterpret_cast<const u32x4*>(b0 + (i < last ? tok_off[i] : last_off));
    walk.advance(mp, BR);
  };
  auto store = [&](int buf, u32x4 (&v)[8], long long r_loaded, bool counted) {  // counted: a stage of this split
    const bool add_bias = want_bias && counted;
    u32x4* dst = lds + buf * SH::STAGE + half * SH::OP + ro * SH::PITCH + jc * 9;
    if (r_loaded + 8 > p.rows) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (r_loaded + i >= p.rows) v[i] = u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int px = 0; px < 8; ++px) {
      const uint32_t sel = (px & 1) ? 0x07060302u : 0x05040100u;
      u32x4 t;
      t.x = __builtin_amdgcn_perm(v[1][px >> 1], v[0][px >> 1], sel);
      t.y = __builtin_amdgcn_perm(v[3][px >> 1], v[2][px >> 1], sel);
      t.z = __builtin_amdgcn_perm(v[5][px >> 1], v[4][px >> 1], sel);
      t.w = __builtin_amdgcn_perm(v[7][px >> 1], v[6][px >> 1], sel);
      dst[px] = t;
      if (add_bias) bsum[px] = add_bf16x8(bsum[px], t);
    }
  };

  f32x16 acc[IM][JN];
#pragma unroll
  for (int i = 0; i < IM; ++i)
#pragma unroll
    for (int j = 0; j < JN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  auto compute = [&](int buf) {
    const u32x4* sg = lds + buf * SH::STAGE;
    const u32x4* sx = sg + SH::OP;
    u32x4 fr[2][IM + JN];
    auto fetch = [&](int kk, u32x4 (&fq)[IM + JN]) {
      const int cc = kk * 2 + kg;
#pragma unroll
      for (int t = 0; t < IM; ++t) {
        const int fg = (wn * IM + t) * 32 + ln;
        fq[t] = sg[cc * SH::PITCH + fg + (fg >> 3)];
      }
#pragma unroll
      for (int t = 0; t < JN; ++t) {
        const int fx = (wc * JN + t) * 32 + ln;
        fq[IM + t] = sx[cc * SH::PITCH + fx + (fx >> 3)];
      }
    };
    fetch(0, fr[0]);
#pragma unroll
    for (int kk = 0; kk < BR / 16; ++kk) {
      if (kk + 1 < BR / 16) fetch(kk + 1, fr[(kk + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < IM; ++i)
#pragma unroll
        for (int j = 0; j < JN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fr[kk & 1][i]),
                                                              __builtin_bit_cast(bf16x8, fr[kk & 1][IM + j]), acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // stage st lives in register set st % AHEAD; the loop is unrolled AHEAD times so that the sets are named at
  // compile time. Nothing in the main loop is conditional: a load or an LDS store under a condition made the
  // compiler merge the set's old and new values through copies, and a copy waits for the load. Loads past the
  // split's last stage read tokens that exist (clamped in `load`) and are never multiplied.
#pragma unroll
  for (int a = 0; a < AHEAD; ++a) load(a, vs[a], rl[a]);
  store(0, vs[0], rl[0], nst > 0);
  __syncthreads();
  const int nst_main = nst - nst % AHEAD;
  int st = 0;
  for (; st < nst_main; st += AHEAD) {
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) {
      load(st + a + AHEAD, vs[a], rl[a]);
      compute((st + a) & 1);
      store((st + a + 1) & 1, vs[(a + 1) % AHEAD], rl[(a + 1) % AHEAD], st + a + 1 < nst);
      __syncthreads();
    }
  }
  // the last nst % AHEAD stages: their tokens are in the sets already, the first of them in LDS
#pragma unroll
  for (int a = 0; a < AHEAD - 1; ++a) {
    if (st + a < nst) {  // uniform
      compute((st + a) & 1);
      if (st + a + 1 < nst) store((st + a + 1) & 1, vs[a + 1], rl[a + 1], true);
      __syncthreads();
    }
  }

  // register e of block (i, j): row n0 + (wn*IM + i)*32 + 8*(e/4) + 4*kg + e%4, column c0 + (wc*JN + j)*32 + ln
  float* part = p.part + (size_t)split * p.N * p.C;
#pragma unroll
  for (int i = 0; i < IM; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int n = n0 + (wn * IM + i) * 32 + (e >> 2) * 8 + kg * 4 + (e & 3);
      if (n < p.N) {
#pragma unroll
        for (int j = 0; j < JN; ++j) {
          const int cidx = c0 + (wc * JN + j) * 32 + ln;
          if (cidx < p.C) part[(size_t)n * p.C + cidx] = acc[i][j][e];
        }
      }
    }

  if (p.bias_part != nullptr && tile_c == 0) {  // uniform over the workgroup
    float* red = reinterpret_cast<float*>(smem);  // [8 token octets][T features]; the stages are done with
    if (half == 0) {
#pragma unroll
      for (int px = 0; px < 8; ++px) red[ro * T + jc * 8 + px] = bsum[px];
    }
    __syncthreads();
    if (tid < T) {
      float sum = 0.0f;
#pragma unroll
      for (int o = 0; o < 8; ++o) sum += red[o * T + tid];
      // a clamped block would count the last features twice: only features of this tile are written
      if (n0 + tid < p.N && (n0 + (tid & ~7) <= p.N - 8)) p.bias_part[(size_t)split * p.N + n0 + tid] = sum;
    }
  }
}

// out[i] (bf16) = sum over the splits of part[split][i], for the weight gradient and (blocks behind
// it) the bias gradient in one launch. A block takes 256 consecutive outputs: 64 lanes x 4 values,
// and its W wavefronts (4, or 16 where there are many splits: a small weight matrix has few blocks,
// and each of their threads would walk the splits one load after the other) each add every W-th
// split; the W sums are then added in a fixed order, so the result does not depend on scheduling.
struct ReduceArgs {
  void* out_w;
  const float* part_w;
  size_t count_w;
  void* out_b;  // NULL: no bias gradient
  const float* part_b;
  size_t count_b;
  int splits;
  int out32;  // write fp32 instead of bf16
};

template <int W>
__global__ __launch_bounds__(64 * W) void proj_reduce_kernel(ReduceArgs a) {
  __shared__ f32x4 sm[W][64];
  const size_t blocks_w = (a.count_w + 255) / 256;
  const bool second = blockIdx.x >= blocks_w;
  void* out_any = second ? a.out_b : a.out_w;
  const float* part = second ? a.part_b : a.part_w;
  const size_t count = second ? a.count_b : a.count_w;
  const int q = threadIdx.x & 63, grp = threadIdx.x >> 6;
  const size_t i0 = (blockIdx.x - (second ? blocks_w : 0)) * 256 + (size_t)q * 4;
  // every split's slice starts 16-byte aligned when the count is a multiple of 4 and the base is aligned
  const bool vec = (count & 3) == 0 && (reinterpret_cast<uintptr_t>(part) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(out_any) & 15) == 0;
  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
  if (i0 < count) {
    if (vec) {
      for (int k = grp; k < a.splits; k += W) acc += *reinterpret_cast<const f32x4*>(part + (size_t)k * count + i0);
    } else {
      for (int k = grp; k < a.splits; k += W)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (i0 + e < count) acc[e] += part[(size_t)k * count + i0 + e];
    }
  }
  sm[grp][q] = acc;
  __syncthreads();
  if (grp != 0 || i0 >= count) return;
  f32x4 t = sm[0][q];
#pragma unroll
  for (int w = 1; w < W; ++w) t += sm[w][q];
  if (a.out32) {
    float* o32 = static_cast<float*>(out_any);
    if (vec) {
      *reinterpret_cast<f32x4*>(o32 + i0) = t;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i0 + e < count) o32[i0 + e] = t[e];
    }
    return;
  }
  uint16_t* out = static_cast<uint16_t*>(out_any);
  if (vec) {
    u32x2 o;
    o.x = (uint32_t)jg::f32_to_bf16(t[0]) | ((uint32_t)jg::f32_to_bf16(t[1]) << 16);
    o.y = (uint32_t)jg::f32_to_bf16(t[2]) | ((uint32_t)jg::f32_to_bf16(t[3]) << 16);
    *reinterpret_cast<u32x2*>(out + i0) = o;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (i0 + e < count) out[i0 + e] = jg::f32_to_bf16(t[e]);
  }
}

// ------------------------------------------------------------------- generic
template <int DT>
struct Elem;
template <>
struct Elem<JG_F32> {
  typedef float T;
  __device__ static __forceinline__ float up(float v) { return v; }
  __device__ static __forceinline__ float down(float v) { return v; }
};
template <>
struct Elem<JG_BF16> {
  typedef uint16_t T;
  __device__ static __forceinline__ float up(uint16_t v) { return jg::bf16_to_f32(v); }
  __device__ static __forceinline__ uint16_t down(float v) { return jg::f32_to_bf16(v); }
};
template <>
struct Elem<JG_F16> {
  typedef _Float16 T;
  __device__ static __forceinline__ float up(_Float16 v) { return (float)v; }
  __device__ static __forceinline__ _Float16 down(float v) { return (_Float16)v; }
};

struct GenParams {
  const void* p;   // NT: a (tokens x K);       TN: g (tokens x I)
  const void* q;   // NT: w (J, K) row-major;    TN: x (tokens x J)
  const void* bias;
  void* out;       // NT: tokens x J through om; TN: (I, J) row-major
  Map pm, qm, om;
  long long I;     // NT: tokens; TN: features of g
  int J;
  long long L;     // contraction length: NT: K; TN: tokens
  int out32;       // TN: write fp32 whatever the operands' dtype
};

// out(i, j) = sum_l P(i, l) * Q(j, l): 16 x 16 outputs per workgroup, the operands pass
// through LDS in tiles of 16 contraction steps. TRANS = 0: P(i, l) = a(i, l), Q(j, l) = w[j][l].
// TRANS = 1: P(i, l) = g(l, i), Q(j, l) = x(l, j).
template <int DT, bool TRANS>
__global__ __launch_bounds__(256) void proj_generic_kernel(GenParams p) {
  typedef typename Elem<DT>::T T;
  __shared__ float sp[16][17], sq[16][17];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const long long i0 = (long long)blockIdx.y * 16;
  const int j0 = blockIdx.x * 16;
  const T* P = static_cast<const T*>(p.p);
  const T* Q = static_cast<const T*>(p.q);
  float acc = 0.0f;
  for (long long l0 = 0; l0 < p.L; l0 += 16) {
    // thread (ty, tx) stages P(i0 + ty, l0 + tx) and Q(j0 + ty, l0 + tx)
    const long long l = l0 + tx;
    float pv = 0.0f, qv = 0.0f;
    if (l < p.L) {
      if (i0 + ty < p.I)
        pv = Elem<DT>::up(TRANS ? P[row_part(p.pm, l) + feat_part(p.pm, (int)(i0 + ty))]
                                : P[row_part(p.pm, i0 + ty) + feat_part(p.pm, (int)l)]);
      if (j0 + ty < p.J)
        qv = Elem<DT>::up(TRANS ? Q[row_part(p.qm, l) + feat_part(p.qm, j0 + ty)]
                                : Q[(long long)(j0 + ty) * p.L + l]);
    }
    sp[ty][tx] = pv;
    sq[ty][tx] = qv;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) acc += sp[ty][k] * sq[tx][k];
    __syncthreads();
  }
  const long long i = i0 + ty;
  const int j = j0 + tx;
  if (i >= p.I || j >= p.J) return;
  T* out = static_cast<T*>(p.out);
  if (TRANS) {
    if (p.out32) static_cast<float*>(p.out)[i * p.J + j] = acc;
    else out[i * p.J + j] = Elem<DT>::down(acc);
  } else {
    if (p.bias != nullptr) acc += Elem<DT>::up(static_cast<const T*>(p.bias)[j]);
    out[row_part(p.om, i) + feat_part(p.om, j)] = Elem<DT>::down(acc);
  }
}

// gb[n] = sum over the tokens of g(r, n): one workgroup per feature, fixed order
template <int DT>
__global__ __launch_bounds__(256) void proj_colsum_kernel(void* gb, const void* g, Map gm, long long rows, bool out32) {
  typedef typename Elem<DT>::T T;
  __shared__ float red[256];
  const int n = blockIdx.x;
  const long long fo = feat_part(gm, n);
  float s = 0.0f;
  for (long long r = threadIdx.x; r < rows; r += 256) s += Elem<DT>::up(static_cast<const T*>(g)[row_part(gm, r) + fo]);
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    if (out32) static_cast<float*>(gb)[n] = red[0];
    else static_cast<T*>(gb)[n] = Elem<DT>::down(red[0]);
  }
}

// --------------------------------------------------------------------- host
int make_map(Map* m, int heads, long long features, long long rows, int B, int H, int S, int D, const char* who,
             const char* what) {
  m->heads = heads ? 1 : 0;
  m->ld = features;
  m->B = B; m->H = H; m->S = S; m->D = D;
  if (!heads) return JG_OK;
  JG_REQUIRE(B > 0 && H > 0 && S > 0 && D > 0, "%s: %s: heads layout needs positive B, H, S, D", who, what);
  JG_REQUIRE((long long)B * S == rows, "%s: %s: B * S = %lld does not match %lld tokens", who, what,
             (long long)B * S, rows);
  JG_REQUIRE(features % ((long long)H * D) == 0, "%s: %s: %lld features are not a multiple of H * D = %lld", who, what,
             features, (long long)H * D);
  return JG_OK;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }
// 16-byte chunks of 8 features stay inside one head and start aligned
bool map_vec_ok(const Map& m, long long features) {
  if (features % 8 != 0) return false;
  return m.heads ? (m.D % 8 == 0) : (m.ld % 8 == 0);
}
// eight consecutive tokens starting at a multiple of 8 belong to one batch entry
bool map_octets_ok(const Map& m) { return !m.heads || m.S % 8 == 0; }

// Token ranges (splits) the contraction is cut into so that `tiles` tiles fill the chip; a
// split is worth its partial tile from about 8 stages on.
int splits_for(long long rows, int tiles, int target, bool small_tiles = false) {
  const long long stages = (rows + BR - 1) / BR;
  long long want = (target + tiles - 1) / tiles;
  // at most 64 splits, but with one to three 128-wide tiles as many as put a workgroup on every compute
  // unit: a compute unit streams its operands at some 20 GB/s, so 64 workgroups leave three quarters of
  // the memory system idle (128 x 128 over 65536 tokens: 23 -> 13 us, the reduction 5 -> 6 us)
  const long long cap = !small_tiles || tiles * 64 >= 256 ? 64 : 256 / tiles;
  if (want > stages / (cap > 64 ? 4 : 8)) want = stages / (cap > 64 ? 4 : 8);
  if (want < 1) want = 1;
  if (want > cap) want = cap;
  return (int)want;
}
// Tile edge of the weight-gradient kernel: 256 (half the operand traffic per MFMA, one workgroup
// per compute unit) when such tiles and their splits still fill most of the chip, else 128.
int tn_tile(long long rows, int n, int c) {
  if (n < 256 || c < 256) return 128;
  const int tiles = jg::cdiv(n, 256) * jg::cdiv(c, 256);
  return tiles * splits_for(rows, tiles, 256) >= 192 ? 256 : 128;
}
int tn_splits(long long rows, int n, int c) {
  const int t = tn_tile(rows, n, c);
  return splits_for(rows, jg::cdiv(n, t) * jg::cdiv(c, t), t == 256 ? 256 : 1024, t == 128);
}

template <int IM, int JN, int WM, int WN>
int launch_tn(TnParams& p, int splits, hipStream_t s, const char* who) {
  typedef TnShape<IM, JN, WM, WN> SH;
  p.tiles_c = jg::cdiv(p.C, SH::T);
  const int tiles = jg::cdiv(p.N, SH::T) * p.tiles_c;
  // the 128-wide tile has the registers for three sets of staged loads, the 256-wide one for one
  void (*kern)(TnParams) = &proj_tn_kernel<IM, JN, WM, WN, (IM * JN <= 4 ? 3 : 1)>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     SH::LDS);
  if (e != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS", who, SH::LDS);
  kern<<<dim3((unsigned)tiles, (unsigned)splits), SH::THREADS, SH::LDS, s>>>(p);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

template <bool TRANS>
int launch_generic(const GenParams& gp, int dtype, hipStream_t s, const char* who) {
  dim3 grid((unsigned)jg::cdiv(gp.J, 16), (unsigned)jg::cdiv(gp.I, 16));
  JG_REQUIRE(grid.y <= 65535u, "%s: too many rows for the generic kernel", who);
  switch (dtype) {
    case JG_F32: proj_generic_kernel<JG_F32, TRANS><<<grid, 256, 0, s>>>(gp); break;
    case JG_BF16: proj_generic_kernel<JG_BF16, TRANS><<<grid, 256, 0, s>>>(gp); break;
    case JG_F16: proj_generic_kernel<JG_F16, TRANS><<<grid, 256, 0, s>>>(gp); break;
    default: JG_FAIL(JG_ERR_BAD_ARG, "%s: unknown dtype %d", who, dtype);
  }
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

}  // namespace

extern "C" {

static int proj_nt_common(const char* who, void* out, void* aux, int epi, const void* a, const void* w, const void* bias,
                          int dtype, int64_t rows, int n_out, int k_in, int a_heads, int out_heads, int B, int H, int S,
                          int D, void* stream) {
  JG_REQUIRE(out && a && w, "%s: null pointer", who);
  JG_REQUIRE(jg::dtype_size(dtype) != 0, "%s: unknown dtype %d", who, dtype);
  JG_REQUIRE(rows >= 0 && n_out > 0 && k_in > 0, "%s: bad sizes rows=%lld n_out=%d k_in=%d", who, (long long)rows, n_out,
             k_in);
  if (rows == 0) return JG_OK;
  Map am, om;
  int rc = make_map(&am, a_heads, k_in, rows, B, H, S, D, who, "input");
  if (rc) return rc;
  rc = make_map(&om, out_heads, n_out, rows, B, H, S, D, who, "output");
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool fast = dtype == JG_BF16 && map_vec_ok(am, k_in) && map_vec_ok(om, n_out) && aligned16(a) &&
                    aligned16(w) && aligned16(out) && rows < (1ll << 31) - 256 &&
                    (unsigned long long)rows * k_in < (1ull << 31) && (unsigned long long)n_out * k_in < (1ull << 31);
  if (!fast) {
    if (epi != EPI_NONE)
      JG_FAIL(JG_ERR_UNSUPPORTED, "%s: the fused epilogues are built for bf16 operands on 16-byte aligned rows", who);
    GenParams gp;
    gp.p = a; gp.q = w; gp.bias = bias; gp.out = out;
    gp.pm = am; gp.qm = am; gp.om = om;
    gp.I = rows; gp.J = n_out; gp.L = k_in;
    gp.out32 = 0;
    return launch_generic<false>(gp, dtype, s, who);
  }
  NtParams p;
  p.epi = epi;
  p.aux = static_cast<uint16_t*>(aux);
  p.a = static_cast<const uint16_t*>(a);
  p.w = static_cast<const uint16_t*>(w);
  p.bias = static_cast<const uint16_t*>(bias);
  p.out = static_cast<uint16_t*>(out);
  p.am = am; p.om = om;
  p.rows = rows; p.N = n_out; p.K = k_in;
  // 256 x 256 tiles (half the operand traffic per MFMA) once they fill the chip, else 128 x 128
  const long long big_tiles = (long long)jg::cdiv(rows, 256) * jg::cdiv(n_out, 256);
  // the 256-wide tile only where its last column of tiles is more than half full
  const int waste = jg::cdiv(n_out, 256) * 256 - n_out;
  if (big_tiles >= 256 && waste < 128) return launch_nt<4, 2, 2, 4>(p, s, who);
  return launch_nt<2, 2, 2, 2>(p, s, who);
}

int jg_proj_nt(void* out, const void* a, const void* w, const void* bias, int dtype, int64_t rows, int n_out,
               int k_in, int a_heads, int out_heads, int B, int H, int S, int D, void* stream) {
  return proj_nt_common("jg_proj_nt", out, nullptr, EPI_NONE, a, w, bias, dtype, rows, n_out, k_in, a_heads, out_heads,
                        B, H, S, D, stream);
}

int jg_proj_nt_fused(void* out, void* aux, int epilogue, const void* a, const void* w, const void* bias, int dtype,
                     int64_t rows, int n_out, int k_in, void* stream) {
  const char* who = "jg_proj_nt_fused";
  JG_REQUIRE(epilogue == EPI_GELU || epilogue == EPI_DGELU || epilogue == EPI_ADD, "%s: unknown epilogue %d", who,
             epilogue);
  JG_REQUIRE(aux != nullptr && aligned16(aux), "%s: aux must be a 16-byte aligned tensor of the shape of out", who);
  return proj_nt_common(who, out, aux, epilogue, a, w, bias, dtype, rows, n_out, k_in, 0, 0, 1, 1, 1, 1, stream);
}

size_t jg_proj_tn_workspace(int64_t rows, int n, int c) {
  if (rows <= 0 || n <= 0 || c <= 0) return 0;
  const size_t splits = (size_t)tn_splits(rows, n, c);
  return splits * ((size_t)n * c + n) * sizeof(float);
}

int jg_proj_tn(void* gw, void* gb, const void* g, const void* x, int dtype, int grad_dtype, int64_t rows, int n, int c,
               int g_heads, int x_heads, int B, int H, int S, int D, void* workspace, size_t workspace_bytes,
               void* stream) {
  const char* who = "jg_proj_tn";
  JG_REQUIRE(gw && g && x, "%s: null pointer", who);
  JG_REQUIRE(jg::dtype_size(dtype) != 0, "%s: unknown dtype %d", who, dtype);
  JG_REQUIRE(grad_dtype == dtype || grad_dtype == JG_F32, "%s: gradient dtype %d with operand dtype %d", who, grad_dtype,
             dtype);
  const bool out32 = grad_dtype == JG_F32 && dtype != JG_F32;
  JG_REQUIRE(rows > 0 && n > 0 && c > 0, "%s: bad sizes rows=%lld n=%d c=%d", who, (long long)rows, n, c);
  JG_REQUIRE(n < (1 << 27) && c < (1 << 27), "%s: more than 2^27 features a row (n=%d c=%d)", who, n, c);
  Map gm, xm;
  int rc = make_map(&gm, g_heads, n, rows, B, H, S, D, who, "gradient");
  if (rc) return rc;
  rc = make_map(&xm, x_heads, c, rows, B, H, S, D, who, "input");
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool fast = dtype == JG_BF16 && map_vec_ok(gm, n) && map_vec_ok(xm, c) && map_octets_ok(gm) &&
                    map_octets_ok(xm) && aligned16(g) && aligned16(x);
  if (!fast) {
    GenParams gp;
    gp.p = g; gp.q = x; gp.bias = nullptr; gp.out = gw;
    gp.pm = gm; gp.qm = xm; gp.om = gm;
    gp.I = n; gp.J = c; gp.L = rows;
    gp.out32 = out32 ? 1 : 0;
    rc = launch_generic<true>(gp, dtype, s, who);
    if (rc) return rc;
    if (gb != nullptr) {
      switch (dtype) {
        case JG_F32: proj_colsum_kernel<JG_F32><<<n, 256, 0, s>>>(gb, g, gm, rows, out32); break;
        case JG_BF16: proj_colsum_kernel<JG_BF16><<<n, 256, 0, s>>>(gb, g, gm, rows, out32); break;
        default: proj_colsum_kernel<JG_F16><<<n, 256, 0, s>>>(gb, g, gm, rows, out32); break;
      }
      JG_CHECK_LAUNCH(who);
    }
    return JG_OK;
  }
  const size_t need = jg_proj_tn_workspace(rows, n, c);
  if (workspace == nullptr || workspace_bytes < need)
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, workspace_bytes, need);
  JG_REQUIRE(aligned16(workspace), "%s: workspace must be 16-byte aligned", who);
  TnParams p;
  p.g = static_cast<const uint16_t*>(g);
  p.x = static_cast<const uint16_t*>(x);
  p.gm = gm; p.xm = xm;
  p.rows = rows; p.N = n; p.C = c;
  const int splits = tn_splits(rows, n, c);
  const long long stages = (rows + BR - 1) / BR;
  p.stages_per_split = (int)((stages + splits - 1) / splits);
  p.part = static_cast<float*>(workspace);
  p.bias_part = gb != nullptr ? p.part + (size_t)splits * n * c : nullptr;
  rc = tn_tile(rows, n, c) == 256 ? launch_tn<4, 2, 2, 4>(p, splits, s, who) : launch_tn<2, 2, 2, 2>(p, splits, s, who);
  if (rc) return rc;
  ReduceArgs ra{};
  ra.out_w = gw;
  ra.part_w = p.part;
  ra.count_w = (size_t)n * c;
  ra.out_b = gb;
  ra.part_b = p.bias_part;
  ra.count_b = gb != nullptr ? (size_t)n : 0;
  ra.splits = splits;
  ra.out32 = out32 ? 1 : 0;
  const size_t blocks = (ra.count_w + 255) / 256 + (ra.count_b + 255) / 256;
  if (splits >= 32) proj_reduce_kernel<16><<<(unsigned)blocks, 1024, 0, s>>>(ra);
  else proj_reduce_kernel<4><<<(unsigned)blocks, 256, 0, s>>>(ra);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

}  // extern "C"
