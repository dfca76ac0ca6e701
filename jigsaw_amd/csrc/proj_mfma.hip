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

constexpr int THREADS = 256;
constexpr int TILE = 128;  // rows and columns of a workgroup tile

// ------------------------------------------------------------------------ NT
constexpr int BK = 64;                 // contraction elements per stage
constexpr int NT_OP = 8 * TILE;        // slots of one operand per stage: [chunk of 8 k][row ^ 2 chunk]
constexpr int NT_STAGE = 2 * NT_OP;
constexpr int NT_LDS = 2 * NT_STAGE * 16;

struct NtParams {
  const uint16_t* a;
  const uint16_t* w;     // (N, K) row-major
  const uint16_t* bias;  // (N,) or NULL
  uint16_t* out;
  Map am, om;
  long long rows;
  int N, K;
  int tiles_n;
};

__device__ __forceinline__ int nt_slot(int chunk, int row) { return chunk * TILE + (row ^ (2 * chunk)); }

__global__ __launch_bounds__(THREADS) void proj_nt_kernel(NtParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  u32x4* lds = reinterpret_cast<u32x4*>(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int wm = wave & 1, wn = wave >> 1;
  const long long m0 = (long long)(blockIdx.x / p.tiles_n) * TILE;
  const int n0 = (blockIdx.x % p.tiles_n) * TILE;

  // loads of a stage: chunk column c, rows tid / 8 + 32 i of both operands
  const int c = tid & 7, lrow = tid >> 3;
  long long a_row[4], w_row[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    long long r = m0 + lrow + 32 * i;
    if (r > p.rows - 1) r = p.rows - 1;  // a row past the end repeats the last one and is dropped
    a_row[i] = row_part(p.am, r);
    int n = n0 + lrow + 32 * i;
    if (n > p.N - 1) n = p.N - 1;
    w_row[i] = (long long)n * p.K;
  }
  u32x4 ra[4], rw[4];
  bool ld_ok = true;
  auto load = [&](int ks) {
    const int k = ks * BK + c * 8;
    ld_ok = k < p.K;  // a chunk past the contraction length is read at k = 0 and zeroed on the way to LDS
    const int kk = ld_ok ? k : 0;
    const long long fa = feat_part(p.am, kk);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ra[i] = *reinterpret_cast<const u32x4*>(p.a + a_row[i] + fa);
      rw[i] = *reinterpret_cast<const u32x4*>(p.w + w_row[i] + kk);
    }
  };
  auto store = [&](int buf) {
    u32x4* sa = lds + buf * NT_STAGE;
    u32x4* sw = sa + NT_OP;
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int slot = nt_slot(c, lrow + 32 * i);
      sa[slot] = ld_ok ? ra[i] : zero;
      sw[slot] = ld_ok ? rw[i] : zero;
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  auto compute = [&](int buf) {
    const u32x4* sa = lds + buf * NT_STAGE;
    const u32x4* sw = sa + NT_OP;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      const int cc = kk * 2 + kg;
      bf16x8 af[2], wf[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        af[t] = __builtin_bit_cast(bf16x8, sa[nt_slot(cc, wm * 64 + t * 32 + ln)]);
        wf[t] = __builtin_bit_cast(bf16x8, sw[nt_slot(cc, wn * 64 + t * 32 + ln)]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
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

  // accumulator lane (ln, kg), register e of block (i, j): token m0 + wm*64 + i*32 +
  // 8*(e/4) + 4*kg + e%4, feature n0 + wn*64 + j*32 + ln
  long long fo[2];
  float bv[2];
  bool n_ok[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn * 64 + j * 32 + ln;
    n_ok[j] = n < p.N;
    fo[j] = feat_part(p.om, n_ok[j] ? n : 0);
    bv[j] = (p.bias != nullptr && n_ok[j]) ? jg::bf16_to_f32(p.bias[n]) : 0.0f;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const long long rbase = m0 + wm * 64 + i * 32 + kg * 4;
    RowWalk rwk;
    rwk.start(p.om, rbase);
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const long long r = rbase + e4 * 8 + e;
        const long long ro = rwk.part(p.om);
        if (r < p.rows) {
#pragma unroll
          for (int j = 0; j < 2; ++j)
            if (n_ok[j]) p.out[ro + fo[j]] = jg::f32_to_bf16(acc[i][j][e4 * 4 + e] + bv[j]);
        }
        rwk.advance(p.om, e == 3 ? 5 : 1);
      }
    }
  }
}

// ------------------------------------------------------------------------ TN
constexpr int BR = 64;             // tokens per stage
constexpr int TN_PITCH = TILE + TILE / 8;  // slots per chunk of 8 tokens: feature f at f + f / 8
constexpr int TN_OP = 8 * TN_PITCH;
constexpr int TN_STAGE = 2 * TN_OP;
constexpr int TN_LDS = 2 * TN_STAGE * 16;

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

__device__ __forceinline__ float sum_bf16x8(const u32x4& v) {
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    s += __builtin_bit_cast(float, v[j] << 16);
    s += __builtin_bit_cast(float, v[j] & 0xffff0000u);
  }
  return s;
}

__global__ __launch_bounds__(THREADS) void proj_tn_kernel(TnParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  u32x4* lds = reinterpret_cast<u32x4*>(smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int wn = wave & 1, wc = wave >> 1;
  const int tile_c = blockIdx.x % p.tiles_c, tile_n = blockIdx.x / p.tiles_c;
  const int n0 = tile_n * TILE, c0 = tile_c * TILE;
  const int split = blockIdx.y;
  const long long r_first = (long long)split * p.stages_per_split * BR;
  long long r_last = r_first + (long long)p.stages_per_split * BR;
  if (r_last > p.rows) r_last = p.rows;
  const int nst = r_last > r_first ? (int)((r_last - r_first + BR - 1) / BR) : 0;

  // loads: waves 0-1 fetch g, waves 2-3 fetch x; a thread owns an 8 token x 8 feature block
  const int half = tid >> 7, tt = tid & 127;
  const int jc = tt & 15, ro = tt >> 4;
  const Map& mp = half ? p.xm : p.gm;
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

  u32x4 v[8];
  long long r_loaded = 0;
  auto load = [&](int st) {
    // tokens r_first + st*BR + ro*8 + i; `walk` stands at i = 0
    r_loaded = r_first + (long long)st * BR + ro * 8;
    RowWalk w = walk;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // a token past the end is read from token 0 (always there) and zeroed on the way to LDS
      const long long off = (r_loaded + i < p.rows) ? w.part(mp) : 0;
      v[i] = *reinterpret_cast<const u32x4*>(src + off + fpart);
      w.advance(mp, 1);
    }
    walk.advance(mp, BR);
  };
  auto store = [&](int buf) {
    u32x4* dst = lds + buf * TN_STAGE + half * TN_OP + ro * TN_PITCH + jc * 9;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (r_loaded + i >= p.rows) v[i] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int px = 0; px < 8; ++px) {
      const uint32_t sel = (px & 1) ? 0x07060302u : 0x05040100u;
      u32x4 t;
      t.x = __builtin_amdgcn_perm(v[1][px >> 1], v[0][px >> 1], sel);
      t.y = __builtin_amdgcn_perm(v[3][px >> 1], v[2][px >> 1], sel);
      t.z = __builtin_amdgcn_perm(v[5][px >> 1], v[4][px >> 1], sel);
      t.w = __builtin_amdgcn_perm(v[7][px >> 1], v[6][px >> 1], sel);
      dst[px] = t;
      if (want_bias) bsum[px] += sum_bf16x8(t);
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  auto compute = [&](int buf) {
    const u32x4* sg = lds + buf * TN_STAGE;
    const u32x4* sx = sg + TN_OP;
#pragma unroll
    for (int kk = 0; kk < BR / 16; ++kk) {
      const int cc = kk * 2 + kg;
      bf16x8 gf[2], xf[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int fg = wn * 64 + t * 32 + ln, fx = wc * 64 + t * 32 + ln;
        gf[t] = __builtin_bit_cast(bf16x8, sg[cc * TN_PITCH + fg + (fg >> 3)]);
        xf[t] = __builtin_bit_cast(bf16x8, sx[cc * TN_PITCH + fx + (fx >> 3)]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gf[i], xf[j], acc[i][j], 0, 0, 0);
    }
  };

  if (nst > 0) {
    load(0);
    store(0);
  }
  __syncthreads();
  for (int st = 0; st < nst; ++st) {
    if (st + 1 < nst) load(st + 1);
    compute(st & 1);
    if (st + 1 < nst) store((st + 1) & 1);
    __syncthreads();
  }

  // register e of block (i, j): row n0 + wn*64 + i*32 + 8*(e/4) + 4*kg + e%4, column c0 + wc*64 + j*32 + ln
  float* part = p.part + (size_t)split * p.N * p.C;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int n = n0 + wn * 64 + i * 32 + (e >> 2) * 8 + kg * 4 + (e & 3);
      if (n < p.N) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int cidx = c0 + wc * 64 + j * 32 + ln;
          if (cidx < p.C) part[(size_t)n * p.C + cidx] = acc[i][j][e];
        }
      }
    }

  if (p.bias_part != nullptr && tile_c == 0) {  // uniform over the workgroup
    float* red = reinterpret_cast<float*>(smem);  // [8 token octets][128 features]; the stages are done with
    if (half == 0) {
#pragma unroll
      for (int px = 0; px < 8; ++px) red[ro * TILE + jc * 8 + px] = bsum[px];
    }
    __syncthreads();
    if (tid < TILE) {
      float s = 0.0f;
#pragma unroll
      for (int o = 0; o < 8; ++o) s += red[o * TILE + tid];
      // a clamped block would count the last features twice: only features of this tile are written
      if (n0 + tid < p.N && (n0 + (tid & ~7) <= p.N - 8)) p.bias_part[(size_t)split * p.N + n0 + tid] = s;
    }
  }
}

// out[i] (bf16) = sum over the splits of part[split][i], fixed order
__global__ __launch_bounds__(256) void proj_reduce_kernel(uint16_t* __restrict__ out, const float* __restrict__ part,
                                                          int splits, size_t count) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  float s = 0.0f;
  for (int k = 0; k < splits; ++k) s += part[(size_t)k * count + i];
  out[i] = jg::f32_to_bf16(s);
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
    out[i * p.J + j] = Elem<DT>::down(acc);
  } else {
    if (p.bias != nullptr) acc += Elem<DT>::up(static_cast<const T*>(p.bias)[j]);
    out[row_part(p.om, i) + feat_part(p.om, j)] = Elem<DT>::down(acc);
  }
}

// gb[n] = sum over the tokens of g(r, n): one workgroup per feature, fixed order
template <int DT>
__global__ __launch_bounds__(256) void proj_colsum_kernel(void* gb, const void* g, Map gm, long long rows) {
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
  if (threadIdx.x == 0) static_cast<T*>(gb)[n] = Elem<DT>::down(red[0]);
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

int tn_splits(long long rows, int tiles) {
  const long long stages = (rows + BR - 1) / BR;
  long long want = (1024 + tiles - 1) / tiles;  // about four workgroups per compute unit
  if (want > stages) want = stages;
  if (want < 1) want = 1;
  if (want > 64) want = 64;
  return (int)want;
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

int jg_proj_nt(void* out, const void* a, const void* w, const void* bias, int dtype, int64_t rows, int n_out,
               int k_in, int a_heads, int out_heads, int B, int H, int S, int D, void* stream) {
  const char* who = "jg_proj_nt";
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
  const bool fast = dtype == JG_BF16 && map_vec_ok(am, k_in) && aligned16(a) && aligned16(w) &&
                    rows < (1ll << 31) - TILE;
  if (!fast) {
    GenParams gp;
    gp.p = a; gp.q = w; gp.bias = bias; gp.out = out;
    gp.pm = am; gp.qm = am; gp.om = om;
    gp.I = rows; gp.J = n_out; gp.L = k_in;
    return launch_generic<false>(gp, dtype, s, who);
  }
  NtParams p;
  p.a = static_cast<const uint16_t*>(a);
  p.w = static_cast<const uint16_t*>(w);
  p.bias = static_cast<const uint16_t*>(bias);
  p.out = static_cast<uint16_t*>(out);
  p.am = am; p.om = om;
  p.rows = rows; p.N = n_out; p.K = k_in;
  p.tiles_n = jg::cdiv(n_out, TILE);
  const long long tiles = (long long)jg::cdiv(rows, TILE) * p.tiles_n;
  JG_REQUIRE(tiles < (1ll << 31), "%s: too many tiles", who);
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&proj_nt_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, NT_LDS);
  if (e != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS", who, NT_LDS);
  proj_nt_kernel<<<(unsigned)tiles, THREADS, NT_LDS, s>>>(p);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

size_t jg_proj_tn_workspace(int64_t rows, int n, int c) {
  if (rows <= 0 || n <= 0 || c <= 0) return 0;
  const int tiles = jg::cdiv(n, TILE) * jg::cdiv(c, TILE);
  const size_t splits = (size_t)tn_splits(rows, tiles);
  return splits * ((size_t)n * c + n) * sizeof(float);
}

int jg_proj_tn(void* gw, void* gb, const void* g, const void* x, int dtype, int64_t rows, int n, int c, int g_heads,
               int x_heads, int B, int H, int S, int D, void* workspace, size_t workspace_bytes, void* stream) {
  const char* who = "jg_proj_tn";
  JG_REQUIRE(gw && g && x, "%s: null pointer", who);
  JG_REQUIRE(jg::dtype_size(dtype) != 0, "%s: unknown dtype %d", who, dtype);
  JG_REQUIRE(rows > 0 && n > 0 && c > 0, "%s: bad sizes rows=%lld n=%d c=%d", who, (long long)rows, n, c);
  Map gm, xm;
  int rc = make_map(&gm, g_heads, n, rows, B, H, S, D, who, "gradient");
  if (rc) return rc;
  rc = make_map(&xm, x_heads, c, rows, B, H, S, D, who, "input");
  if (rc) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool fast = dtype == JG_BF16 && map_vec_ok(gm, n) && map_vec_ok(xm, c) && aligned16(g) && aligned16(x);
  if (!fast) {
    GenParams gp;
    gp.p = g; gp.q = x; gp.bias = nullptr; gp.out = gw;
    gp.pm = gm; gp.qm = xm; gp.om = gm;
    gp.I = n; gp.J = c; gp.L = rows;
    rc = launch_generic<true>(gp, dtype, s, who);
    if (rc) return rc;
    if (gb != nullptr) {
      switch (dtype) {
        case JG_F32: proj_colsum_kernel<JG_F32><<<n, 256, 0, s>>>(gb, g, gm, rows); break;
        case JG_BF16: proj_colsum_kernel<JG_BF16><<<n, 256, 0, s>>>(gb, g, gm, rows); break;
        default: proj_colsum_kernel<JG_F16><<<n, 256, 0, s>>>(gb, g, gm, rows); break;
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
  p.tiles_c = jg::cdiv(c, TILE);
  const int tiles = jg::cdiv(n, TILE) * p.tiles_c;
  const int splits = tn_splits(rows, tiles);
  const long long stages = (rows + BR - 1) / BR;
  p.stages_per_split = (int)((stages + splits - 1) / splits);
  p.part = static_cast<float*>(workspace);
  p.bias_part = gb != nullptr ? p.part + (size_t)splits * n * c : nullptr;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&proj_tn_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, TN_LDS);
  if (e != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS", who, TN_LDS);
  proj_tn_kernel<<<dim3((unsigned)tiles, (unsigned)splits), THREADS, TN_LDS, s>>>(p);
  JG_CHECK_LAUNCH(who);
  const size_t count = (size_t)n * c;
  proj_reduce_kernel<<<(unsigned)((count + 255) / 256), 256, 0, s>>>(static_cast<uint16_t*>(gw), p.part, splits, count);
  JG_CHECK_LAUNCH(who);
  if (gb != nullptr) {
    proj_reduce_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(static_cast<uint16_t*>(gb), p.bias_part, splits,
                                                                    (size_t)n);
    JG_CHECK_LAUNCH(who);
  }
  return JG_OK;
}

}  // extern "C"
