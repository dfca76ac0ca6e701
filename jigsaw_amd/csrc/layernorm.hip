// Sharded LayerNorm: partial statistics, apply, and the backward partials.
// One wavefront owns one row at a time; lanes stride the columns in 16-byte (or
// 8-byte) vectors so every global access is coalesced; row reductions are
// wavefront butterflies (no LDS), column reductions are per-lane registers plus
// a deterministic two-stage tree (no atomics). Everything is HBM-bound.
//
// Reference behaviour restated here:
//   jigsaw/modules/normalization/_functional.py:45-58   (forward)
//   jigsaw/modules/normalization/_functional.py:141-175 (backward)
#include "jg_common.h"

#include <mutex>
#include <type_traits>

namespace {

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kThreads = kWave * kWavesPerBlock;
constexpr int kVec = 4;        // elements per lane per step
constexpr int kMaxChunks = 8;  // column chunks a lane can own in the backward

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
  // the hardware's conversion: round to nearest even, as jg::f32_to_bf16 (any NaN becomes a quiet one)
  __device__ static __forceinline__ uint16_t down(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }
};
template <>
struct Elem<JG_F16> {
  typedef _Float16 T;
  __device__ static __forceinline__ float up(_Float16 v) { return (float)v; }
  __device__ static __forceinline__ _Float16 down(float v) { return (_Float16)v; }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// Load up to kVec consecutive elements of a row starting at column c (c % kVec == 0).
template <int DT>
__device__ __forceinline__ void load_vec(const typename Elem<DT>::T* row, long long c,
                                         long long cols, bool vec_ok, float out[kVec]) {
  typedef typename Elem<DT>::T T;
  if (vec_ok && c + kVec <= cols) {
    struct alignas(sizeof(T) * kVec) Pack { T v[kVec]; };
    Pack p = *reinterpret_cast<const Pack*>(row + c);
#pragma unroll
    for (int i = 0; i < kVec; ++i) out[i] = Elem<DT>::up(p.v[i]);
  } else {
#pragma unroll
    for (int i = 0; i < kVec; ++i) out[i] = (c + i < cols) ? Elem<DT>::up(row[c + i]) : 0.0f;
  }
}

template <int DT>
__device__ __forceinline__ void store_vec(typename Elem<DT>::T* row, long long c, long long cols,
                                          bool vec_ok, const float in[kVec]) {
  typedef typename Elem<DT>::T T;
  if (vec_ok && c + kVec <= cols) {
    struct alignas(sizeof(T) * kVec) Pack { T v[kVec]; };
    Pack p;
#pragma unroll
    for (int i = 0; i < kVec; ++i) p.v[i] = Elem<DT>::down(in[i]);
    *reinterpret_cast<Pack*>(row + c) = p;
  } else {
#pragma unroll
    for (int i = 0; i < kVec; ++i)
      if (c + i < cols) row[c + i] = Elem<DT>::down(in[i]);
  }
}

// ---------------------------------------------------------- partial statistics
template <int DT>
__global__ __launch_bounds__(kThreads) void ln_partial_fwd_kernel(
    float* __restrict__ mean, float* __restrict__ var, const typename Elem<DT>::T* __restrict__ x,
    long long rows, long long cols, bool vec_ok) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const float inv = 1.0f / (float)cols;
  for (long long r = (long long)blockIdx.x * kWavesPerBlock + wave; r < rows;
       r += (long long)gridDim.x * kWavesPerBlock) {
    const typename Elem<DT>::T* row = x + r * cols;
    float s = 0.0f;
    for (long long c = (long long)lane * kVec; c < cols; c += kWave * kVec) {
      float v[kVec];
      load_vec<DT>(row, c, cols, vec_ok, v);
#pragma unroll
      for (int i = 0; i < kVec; ++i) s += v[i];
    }
    const float m = wave_sum(s) * inv;
    float q = 0.0f;
    for (long long c = (long long)lane * kVec; c < cols; c += kWave * kVec) {
      float v[kVec];
      load_vec<DT>(row, c, cols, vec_ok, v);
#pragma unroll
      for (int i = 0; i < kVec; ++i) {
        float d = (c + i < cols) ? v[i] - m : 0.0f;
        q += d * d;
      }
    }
    q = wave_sum(q) * inv;
    if (lane == 0) {
      mean[r] = m;
      var[r] = q;
    }
  }
}

// ----------------------------------------------------------------------- apply
template <int XDT, int ODT>
__global__ __launch_bounds__(kThreads) void ln_apply_kernel(
    typename Elem<ODT>::T* __restrict__ y, typename Elem<ODT>::T* __restrict__ x_hat,
    float* __restrict__ std_out, const typename Elem<XDT>::T* __restrict__ x,
    const float* __restrict__ mean, const float* __restrict__ var,
    const typename Elem<ODT>::T* __restrict__ w, const typename Elem<ODT>::T* __restrict__ b,
    long long rows, long long cols, float eps, bool vx_ok, bool vo_ok, bool vw_ok) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  for (long long r = (long long)blockIdx.x * kWavesPerBlock + wave; r < rows;
       r += (long long)gridDim.x * kWavesPerBlock) {
    const float m = mean[r];
    const float sd = sqrtf(var[r] + eps);
    if (lane == 0 && std_out != nullptr) std_out[r] = sd;
    for (long long c = (long long)lane * kVec; c < cols; c += kWave * kVec) {
      float v[kVec], wv[kVec], bv[kVec], xh[kVec], out[kVec];
      load_vec<XDT>(x + r * cols, c, cols, vx_ok, v);
      load_vec<ODT>(w, c, cols, vw_ok, wv);
      if (b != nullptr) load_vec<ODT>(b, c, cols, vw_ok, bv);
#pragma unroll
      for (int i = 0; i < kVec; ++i) {
        // x_hat is rounded to the output dtype before the affine map, as the
        // reference materialises x_norm in that dtype and then multiplies.
        xh[i] = Elem<ODT>::up(Elem<ODT>::down((v[i] - m) / sd));
        out[i] = wv[i] * xh[i] + (b != nullptr ? bv[i] : 0.0f);
      }
      if (x_hat != nullptr) store_vec<ODT>(x_hat + r * cols, c, cols, vo_ok, xh);
      store_vec<ODT>(y + r * cols, c, cols, vo_ok, out);
    }
  }
}

// ------------------------------------------------------------ backward partials
// Stage 1: block `blk` walks rows blk*kWavesPerBlock + wave + k*gridDim*kWavesPerBlock.
// Each lane keeps column partials for the columns it touches; they are reduced
// across the block's waves in LDS and written to part[blk][which][col].
template <int DT, int CH>
__global__ __launch_bounds__(kThreads) void ln_partial_bwd_kernel(
    float* __restrict__ mean_gxn, float* __restrict__ dot, float* __restrict__ part,
    const typename Elem<DT>::T* __restrict__ g, const typename Elem<DT>::T* __restrict__ x_hat,
    const typename Elem<DT>::T* __restrict__ w, long long rows, long long cols, bool vec_ok,
    bool vw_ok, bool want_cols) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const float inv = 1.0f / (float)cols;
  float wv[CH][kVec];
  float agw[CH][kVec], agb[CH][kVec];
#pragma unroll
  for (int k = 0; k < CH; ++k) {
    long long c = ((long long)k * kWave + lane) * kVec;
    if (c < cols) load_vec<DT>(w, c, cols, vw_ok, wv[k]);
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
      agw[k][i] = 0.0f;
      agb[k][i] = 0.0f;
      if (c >= cols) wv[k][i] = 0.0f;
    }
  }
  for (long long r = (long long)blockIdx.x * kWavesPerBlock + wave; r < rows;
       r += (long long)gridDim.x * kWavesPerBlock) {
    float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
    for (int k = 0; k < CH; ++k) {
      long long c = ((long long)k * kWave + lane) * kVec;
      if (c < cols) {
        float gv[kVec], xh[kVec];
        load_vec<DT>(g + r * cols, c, cols, vec_ok, gv);
        load_vec<DT>(x_hat + r * cols, c, cols, vec_ok, xh);
#pragma unroll
        for (int i = 0; i < kVec; ++i) {
          // grad_x_norm = g * w is materialised in the tensor dtype by the reference
          float gxn = Elem<DT>::up(Elem<DT>::down(gv[i] * wv[k][i]));
          s1 += gxn;
          s2 += gxn * xh[i];
          agw[k][i] += gv[i] * xh[i];
          agb[k][i] += gv[i];
        }
      }
    }
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    if (lane == 0) {
      mean_gxn[r] = s1 * inv;
      dot[r] = s2;
    }
  }
  if (!want_cols) return;
  __shared__ float red[kWavesPerBlock][2][CH * kWave * kVec];
#pragma unroll
  for (int k = 0; k < CH; ++k)
#pragma unroll
    for (int i = 0; i < kVec; ++i) {
      red[wave][0][(k * kWave + lane) * kVec + i] = agw[k][i];
      red[wave][1][(k * kWave + lane) * kVec + i] = agb[k][i];
    }
  __syncthreads();
  for (long long c = threadIdx.x; c < cols; c += kThreads) {
    float a = 0.0f, b2 = 0.0f;
#pragma unroll
    for (int wv2 = 0; wv2 < kWavesPerBlock; ++wv2) {
      a += red[wv2][0][c];
      b2 += red[wv2][1][c];
    }
    part[((long long)blockIdx.x * 2 + 0) * cols + c] = a;
    part[((long long)blockIdx.x * 2 + 1) * cols + c] = b2;
  }
}

// Stage 2: a block owns 64 consecutive columns (one per lane, so a partial row is read
// coalesced); its 16 wavefronts take the block partials k = w, w + 16, ... in 4 independent
// chains each, and the 64 chain sums are added in a fixed order (deterministic).
constexpr int kReduceWaves = 16;
__global__ __launch_bounds__(kReduceWaves * 64) void ln_colreduce_kernel(float* __restrict__ gw,
                                                                         float* __restrict__ gb,
                                                                         const float* __restrict__ part,
                                                                         int nblocks, long long cols) {
  __shared__ float red[kReduceWaves][2][64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const long long c = (long long)blockIdx.x * 64 + lane;
  float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
  if (c < cols) {
    int k = w;
    for (; k + 3 * kReduceWaves < nblocks; k += 4 * kReduceWaves) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        a[u] += part[((long long)(k + kReduceWaves * u) * 2 + 0) * cols + c];
        b[u] += part[((long long)(k + kReduceWaves * u) * 2 + 1) * cols + c];
      }
    }
    for (; k < nblocks; k += kReduceWaves) {
      a[0] += part[((long long)k * 2 + 0) * cols + c];
      b[0] += part[((long long)k * 2 + 1) * cols + c];
    }
  }
  red[w][0][lane] = (a[0] + a[1]) + (a[2] + a[3]);
  red[w][1][lane] = (b[0] + b[1]) + (b[2] + b[3]);
  __syncthreads();
  if (w != 0 || c >= cols) return;
  float sw = 0.0f, sb = 0.0f;
#pragma unroll
  for (int i = 0; i < kReduceWaves; ++i) {
    sw += red[i][0][lane];
    sb += red[i][1][lane];
  }
  if (gw != nullptr) gw[c] = sw;
  if (gb != nullptr) gb[c] = sb;
}

template <int DT>
__global__ __launch_bounds__(kThreads) void ln_bwd_apply_kernel(
    typename Elem<DT>::T* __restrict__ gx, const typename Elem<DT>::T* __restrict__ g,
    const typename Elem<DT>::T* __restrict__ x_hat, const typename Elem<DT>::T* __restrict__ w,
    const float* __restrict__ mean_gxn, const float* __restrict__ dot,
    const float* __restrict__ stdv, long long rows, long long cols, float inv_n, bool vec_ok,
    bool vw_ok) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  for (long long r = (long long)blockIdx.x * kWavesPerBlock + wave; r < rows;
       r += (long long)gridDim.x * kWavesPerBlock) {
    const float m = mean_gxn[r];
    const float dn = dot[r] * inv_n;
    const float rs = 1.0f / stdv[r];
    for (long long c = (long long)lane * kVec; c < cols; c += kWave * kVec) {
      float gv[kVec], xh[kVec], wv[kVec], out[kVec];
      load_vec<DT>(g + r * cols, c, cols, vec_ok, gv);
      load_vec<DT>(x_hat + r * cols, c, cols, vec_ok, xh);
      load_vec<DT>(w, c, cols, vw_ok, wv);
#pragma unroll
      for (int i = 0; i < kVec; ++i) {
        float gxn = Elem<DT>::up(Elem<DT>::down(gv[i] * wv[i]));
        out[i] = rs * (gxn - m - xh[i] * dn);
      }
      store_vec<DT>(gx + r * cols, c, cols, vec_ok, out);
    }
  }
}

int row_grid(long long rows) {
  long long b = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
  if (b > 65536) b = 65536;
  if (b < 1) b = 1;
  return (int)b;
}

int bwd_blocks(long long rows) {
  long long b = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
  if (b > 1024) b = 1024;  // 4 blocks per CU; bounds the stage-2 sum length
  if (b < 1) b = 1;
  return (int)b;
}

bool vec_aligned(const void* p, long long cols, int dtype) {
  const size_t bytes = jg::dtype_size(dtype) * kVec;
  return (reinterpret_cast<uintptr_t>(p) % bytes) == 0 && (cols % kVec) == 0;
}

bool known(int dt) { return dt == JG_F32 || dt == JG_BF16 || dt == JG_F16; }

// ------------------------------------------------------------------ unsharded
// LayerNorm over rows that one rank holds whole (nn.LayerNorm as the Swin block uses it,
// examples/swin.py:186-188, 209-210): statistics and apply in one pass over x, and a backward
// that recomputes x_hat from (x, mean, rstd). A row is held in registers: G lanes share a row
// (8 columns per lane and chunk, at most kPlainChunks chunks), 64 / G rows per wavefront, so
// narrow rows still use every lane. x, y, g and gx may each have their own dtype; w, b fp32.
constexpr int kPlainVec = 8;
constexpr int kPlainChunks = 4;

template <int DT>
__device__ __forceinline__ void load8(const typename Elem<DT>::T* p, float out[kPlainVec]) {
  typedef typename Elem<DT>::T T;
  struct alignas(16) Pack { T v[16 / sizeof(T)]; };
  constexpr int PER = 16 / sizeof(T);
#pragma unroll
  for (int h = 0; h < kPlainVec / PER; ++h) {
    const Pack q = *reinterpret_cast<const Pack*>(p + h * PER);
#pragma unroll
    for (int i = 0; i < PER; ++i) out[h * PER + i] = Elem<DT>::up(q.v[i]);
  }
}
template <int DT>
__device__ __forceinline__ void store8(typename Elem<DT>::T* p, const float in[kPlainVec]) {
  typedef typename Elem<DT>::T T;
  struct alignas(16) Pack { T v[16 / sizeof(T)]; };
  constexpr int PER = 16 / sizeof(T);
#pragma unroll
  for (int h = 0; h < kPlainVec / PER; ++h) {
    Pack q;
#pragma unroll
    for (int i = 0; i < PER; ++i) q.v[i] = Elem<DT>::down(in[h * PER + i]);
    *reinterpret_cast<Pack*>(p + h * PER) = q;
  }
}

// Sum over the G lanes (a power of two) that share a row, left in every one of them: the butterfly
// v += v[lane ^ o] for o = 1, 2, 4, ..., G / 2, without a trip through the LDS crossbar. Inside a row of
// 16 lanes the partner comes through DPP operands (for o = 4 and 8 the mirror partner holds the bits of the
// lane ^ o partner, because every lane of a finished group holds the same sum); rows of 16 and halves of 32
// change places with the swap instructions. The swaps are written in assembly with their wait states: the
// builtin was seen to be folded into "a + a" when both of its operands hold the same value.
template <int CTRL>
__device__ __forceinline__ float dpp_partner(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float add_row_partner(float v) {  // v[lane] + v[lane ^ 16]
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}
__device__ __forceinline__ float add_half_partner(float v) {  // v[lane] + v[lane ^ 32]
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}
// N such sums at once: the N instructions of a step do not wait for each other
template <int N>
__device__ __forceinline__ void group_sums(float (&v)[N], int G) {
  if (G > 1) {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] += dpp_partner<0xB1>(v[i]);  // quad_perm [1, 0, 3, 2]
  }
  if (G > 2) {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] += dpp_partner<0x4E>(v[i]);  // quad_perm [2, 3, 0, 1]
  }
  if (G > 4) {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] += dpp_partner<0x141>(v[i]);  // row_half_mirror
  }
  if (G > 8) {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] += dpp_partner<0x140>(v[i]);  // row_mirror
  }
  if (G > 16) {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = add_row_partner(v[i]);
  }
  if (G > 32) {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = add_half_partner(v[i]);
  }
}
__device__ __forceinline__ float group_sum(float v, int G) {
  float one[1] = {v};
  group_sums<1>(one, G);
  return one[0];
}

// w (and b) of the columns a lane owns, as 16-byte loads
template <int CH>
__device__ __forceinline__ void load_params(float (&dst)[CH][kPlainVec], const float* src, int G, int sl, int cols) {
#pragma unroll
  for (int k = 0; k < CH; ++k) {
    const int c = (k * G + sl) * kPlainVec;
    if (c < cols && src != nullptr) {
      load8<JG_F32>(src + c, dst[k]);
    } else {
#pragma unroll
      for (int i = 0; i < kPlainVec; ++i) dst[k][i] = 0.0f;
    }
  }
}

// U rows per lane group are in flight at once (their loads and shuffles interleave).
template <int XDT, int YDT, int CH, int U>
__global__ __launch_bounds__(kThreads) void ln_plain_fwd_kernel(
    typename Elem<YDT>::T* __restrict__ y, float* __restrict__ mean, float* __restrict__ rstd,
    const typename Elem<XDT>::T* __restrict__ x, const float* __restrict__ w,
    const float* __restrict__ b, long long rows, int cols, float eps, int G) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sl = lane & (G - 1), sub = lane / G, rpw = kWave / G;
  const float inv = 1.0f / (float)cols;
  // a wavefront's U row sets of a round lie behind each other in memory (U * rpw consecutive rows)
  const long long stride = rpw, round_stride = (long long)gridDim.x * kWavesPerBlock * rpw * U;
  float wv[CH][kPlainVec], bv[CH][kPlainVec];
  load_params<CH>(wv, w, G, sl, cols);
  load_params<CH>(bv, b, G, sl, cols);
  for (long long r0 = ((long long)blockIdx.x * kWavesPerBlock + wave) * rpw * U; r0 < rows; r0 += round_stride) {
    float v[U][CH][kPlainVec], m[U], rs[U];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const long long r = r0 + u * stride + sub;
      live[u] = r < rows;
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const int c = (k * G + sl) * kPlainVec;
        if (live[u] && c < cols) {
          load8<XDT>(x + r * cols + c, v[u][k]);
        } else {
#pragma unroll
          for (int i = 0; i < kPlainVec; ++i) v[u][k][i] = 0.0f;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float s = 0.0f;
#pragma unroll
      for (int k = 0; k < CH; ++k)
#pragma unroll
        for (int i = 0; i < kPlainVec; ++i) s += v[u][k][i];
      m[u] = s;
    }
    group_sums<U>(m, G);
#pragma unroll
    for (int u = 0; u < U; ++u) m[u] *= inv;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float q = 0.0f;
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        if ((k * G + sl) * kPlainVec < cols) {
#pragma unroll
          for (int i = 0; i < kPlainVec; ++i) {
            const float d = v[u][k][i] - m[u];
            q += d * d;
          }
        }
      }
      rs[u] = q;
    }
    group_sums<U>(rs, G);
#pragma unroll
    for (int u = 0; u < U; ++u) rs[u] = rsqrtf(rs[u] * inv + eps);
    // every lane of the wavefront took part in the shuffles above; only now do dead rows drop out
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (!live[u]) continue;
      const long long r = r0 + u * stride + sub;
      if (sl == 0) {
        mean[r] = m[u];
        rstd[r] = rs[u];
      }
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const int c = (k * G + sl) * kPlainVec;
        if (c < cols) {
          float out[kPlainVec];
#pragma unroll
          for (int i = 0; i < kPlainVec; ++i) out[i] = (v[u][k][i] - m[u]) * rs[u] * wv[k][i] + bv[k][i];
          store8<YDT>(y + r * cols + c, out);
        }
      }
    }
  }
}

// gx = rstd * (g w - mean_c(g w) - x_hat * mean_c(g w x_hat)); column partials of g x_hat and g
// per block in part[blk][which][col] (ln_colreduce_kernel finishes them).
template <int GDT, int XDT, int CH, int U>
__global__ __launch_bounds__(kThreads) void ln_plain_bwd_kernel(
    typename Elem<XDT>::T* __restrict__ gx, float* __restrict__ part,
    const typename Elem<GDT>::T* __restrict__ g, const typename Elem<XDT>::T* __restrict__ x,
    const float* __restrict__ mean, const float* __restrict__ rstd, const float* __restrict__ w,
    long long rows, int cols, int G, bool want_cols, const typename Elem<XDT>::T* __restrict__ add) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sl = lane & (G - 1), sub = lane / G, rpw = kWave / G;
  const float inv = 1.0f / (float)cols;
  // a wavefront's U row sets of a round lie behind each other in memory (U * rpw consecutive rows)
  const long long stride = rpw, round_stride = (long long)gridDim.x * kWavesPerBlock * rpw * U;
  float wv[CH][kPlainVec], agw[CH][kPlainVec], agb[CH][kPlainVec];
  load_params<CH>(wv, w, G, sl, cols);
#pragma unroll
  for (int k = 0; k < CH; ++k)
#pragma unroll
    for (int i = 0; i < kPlainVec; ++i) {
      agw[k][i] = 0.0f;
      agb[k][i] = 0.0f;
    }
  for (long long r0 = ((long long)blockIdx.x * kWavesPerBlock + wave) * rpw * U; r0 < rows; r0 += round_stride) {
    float gv[U][CH][kPlainVec], xh[U][CH][kPlainVec], m[U], rs[U], s1[U], s2[U], s12[2 * U];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const long long r = r0 + u * stride + sub;
      live[u] = r < rows;
      m[u] = live[u] ? mean[r] : 0.0f;
      rs[u] = live[u] ? rstd[r] : 0.0f;
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const int c = (k * G + sl) * kPlainVec;
        if (live[u] && c < cols) {
          load8<GDT>(g + r * cols + c, gv[u][k]);
          load8<XDT>(x + r * cols + c, xh[u][k]);
        } else {
#pragma unroll
          for (int i = 0; i < kPlainVec; ++i) {
            gv[u][k][i] = 0.0f;
            xh[u][k][i] = m[u];
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float a1 = 0.0f, a2 = 0.0f;
#pragma unroll
      for (int k = 0; k < CH; ++k)
#pragma unroll
        for (int i = 0; i < kPlainVec; ++i) {
          xh[u][k][i] = (xh[u][k][i] - m[u]) * rs[u];
          const float gxn = gv[u][k][i] * wv[k][i];
          a1 += gxn;
          a2 += gxn * xh[u][k][i];
          agw[k][i] += gv[u][k][i] * xh[u][k][i];
          agb[k][i] += gv[u][k][i];
        }
      s12[u] = a1;
      s12[U + u] = a2;
    }
    group_sums<2 * U>(s12, G);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      s1[u] = s12[u] * inv;
      s2[u] = s12[U + u] * inv;
    }
    if (gx == nullptr) continue;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (!live[u]) continue;
      const long long r = r0 + u * stride + sub;
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const int c = (k * G + sl) * kPlainVec;
        if (c < cols) {
          float out[kPlainVec];
#pragma unroll
          for (int i = 0; i < kPlainVec; ++i)
            out[i] = rs[u] * (gv[u][k][i] * wv[k][i] - s1[u] - xh[u][k][i] * s2[u]);
          if (add != nullptr) {
            // the gradient that reaches x past the normalisation (a residual connection): added
            // to the rounded result, as the separate sum of the two gradient tensors would
            float past[kPlainVec];
            load8<XDT>(add + r * cols + c, past);
#pragma unroll
            for (int i = 0; i < kPlainVec; ++i) out[i] = Elem<XDT>::up(Elem<XDT>::down(out[i])) + past[i];
          }
          store8<XDT>(gx + r * cols + c, out);
        }
      }
    }
  }
  if (!want_cols) return;
  // the rows of a wavefront that share a column set: lanes sl, sl + G, ...
#pragma unroll
  for (int k = 0; k < CH; ++k)
#pragma unroll
    for (int i = 0; i < kPlainVec; ++i)
      for (int o = G; o < kWave; o <<= 1) {
        agw[k][i] += __shfl_xor(agw[k][i], o, kWave);
        agb[k][i] += __shfl_xor(agb[k][i], o, kWave);
      }
  __shared__ float red[kWavesPerBlock][2][kPlainChunks * kWave * kPlainVec];
  if (sub == 0) {
#pragma unroll
    for (int k = 0; k < CH; ++k)
#pragma unroll
      for (int i = 0; i < kPlainVec; ++i) {
        red[wave][0][(k * G + sl) * kPlainVec + i] = agw[k][i];
        red[wave][1][(k * G + sl) * kPlainVec + i] = agb[k][i];
      }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < cols; c += kThreads) {
    float a = 0.0f, b2 = 0.0f;
#pragma unroll
    for (int wv2 = 0; wv2 < kWavesPerBlock; ++wv2) {
      a += red[wv2][0][c];
      b2 += red[wv2][1][c];
    }
    part[((long long)blockIdx.x * 2 + 0) * cols + c] = a;
    part[((long long)blockIdx.x * 2 + 1) * cols + c] = b2;
  }
}

// ------------------------------------------------- sharded, rows held in registers
// The four row kernels of the sharded LayerNorm once more, for local widths that fit the register
// layout of the unsharded kernels (a multiple of 8 columns, at most G * 8 * kPlainChunks): G lanes
// share a row, 64 / G rows per wavefront, 16-byte accesses, U rows of a lane group in flight and
// one pass over the memory. The arithmetic per element is that of the kernels above.
template <int DT, int CH>
__device__ __forceinline__ void load_params_of(float (&dst)[CH][kPlainVec], const typename Elem<DT>::T* src, int G,
                                               int sl, int cols) {
#pragma unroll
  for (int k = 0; k < CH; ++k) {
    const int c = (k * G + sl) * kPlainVec;
    if (c < cols && src != nullptr) {
      load8<DT>(src + c, dst[k]);
    } else {
#pragma unroll
      for (int i = 0; i < kPlainVec; ++i) dst[k][i] = 0.0f;
    }
  }
}

// 8 columns of a row from an address that is always inside the tensor (row and column clamped), zero
// where the lane owns nothing: the loads of a wavefront leave back to back, under no branch.
template <int DT>
__device__ __forceinline__ void load8_or_zero(const typename Elem<DT>::T* base, long long r, long long rows, int c,
                                              int cols, float out[kPlainVec]) {
  const bool ok = r < rows && c < cols;
  load8<DT>(base + (r < rows ? r : rows - 1) * cols + (c < cols ? c : 0), out);
#pragma unroll
  for (int i = 0; i < kPlainVec; ++i) out[i] = ok ? out[i] : 0.0f;
}

// 8 columns as they lie in memory (16 or 32 bytes), converted later: a kernel can then request the rows of its
// next round before it turns to the arithmetic of the current one, and the loads stay in the air meanwhile.
template <int DT>
struct Raw8 {
  typedef typename Elem<DT>::T T;
  static constexpr int PER = 16 / sizeof(T);
  struct alignas(16) Pack { T v[PER]; };
  Pack p[kPlainVec / PER];
};
template <int DT>
__device__ __forceinline__ void load8_raw(const typename Elem<DT>::T* base, long long r, long long rows, int c, int cols,
                                          Raw8<DT>& out) {
  typedef typename Raw8<DT>::Pack Pack;
  // always an address inside the tensor (row and column clamped): no branch around the load
  const typename Elem<DT>::T* p = base + (r < rows ? r : rows - 1) * cols + (c < cols ? c : 0);
#pragma unroll
  for (int h = 0; h < kPlainVec / Raw8<DT>::PER; ++h) out.p[h] = *reinterpret_cast<const Pack*>(p + h * Raw8<DT>::PER);
}
template <int DT>
__device__ __forceinline__ void unpack8(const Raw8<DT>& in, bool ok, float out[kPlainVec]) {
#pragma unroll
  for (int h = 0; h < kPlainVec / Raw8<DT>::PER; ++h)
#pragma unroll
    for (int i = 0; i < Raw8<DT>::PER; ++i) out[h * Raw8<DT>::PER + i] = ok ? Elem<DT>::up(in.p[h].v[i]) : 0.0f;
}

template <int DT, int CH, int U>
__global__ __launch_bounds__(kThreads) void ln_partial_fwd_rows_kernel(
    float* __restrict__ mean, float* __restrict__ var, const typename Elem<DT>::T* __restrict__ x,
    long long rows, int cols, int G) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sl = lane & (G - 1), sub = lane / G, rpw = kWave / G;
  const float inv = 1.0f / (float)cols;
  // a wavefront's U row sets of a round lie behind each other in memory (U * rpw consecutive rows)
  const long long stride = rpw;
  const long long round_stride = (long long)gridDim.x * kWavesPerBlock * rpw * U;
  long long r0 = ((long long)blockIdx.x * kWavesPerBlock + wave) * rpw * U;
  Raw8<DT> raw[U][CH];
  auto request = [&](long long first) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int k = 0; k < CH; ++k) load8_raw<DT>(x, first + u * stride + sub, rows, (k * G + sl) * kPlainVec, cols, raw[u][k]);
  };
  if (r0 < rows) request(r0);
  for (; r0 < rows; r0 += round_stride) {
    float v[U][CH][kPlainVec], m[U], qs[U];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      live[u] = r0 + u * stride + sub < rows;
#pragma unroll
      for (int k = 0; k < CH; ++k) unpack8<DT>(raw[u][k], live[u] && (k * G + sl) * kPlainVec < cols, v[u][k]);
    }
    // the rows of the next round are on their way during the sums and shuffles of this one
    if (r0 + round_stride < rows) request(r0 + round_stride);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float s = 0.0f;
#pragma unroll
      for (int k = 0; k < CH; ++k)
#pragma unroll
        for (int i = 0; i < kPlainVec; ++i) s += v[u][k][i];
      m[u] = s;
    }
    group_sums<U>(m, G);
#pragma unroll
    for (int u = 0; u < U; ++u) m[u] *= inv;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float q = 0.0f;
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        if ((k * G + sl) * kPlainVec < cols) {
#pragma unroll
          for (int i = 0; i < kPlainVec; ++i) {
            const float d = v[u][k][i] - m[u];
            q += d * d;
          }
        }
      }
      qs[u] = q;
    }
    group_sums<U>(qs, G);
    // every lane of the wavefront took part in the shuffles; dead rows drop out only here
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (live[u] && sl == 0) {
        const long long r = r0 + u * stride + sub;
        mean[r] = m[u];
        var[r] = qs[u] * inv;
      }
    }
  }
}

template <int XDT, int ODT, int CH, int U>
__global__ __launch_bounds__(kThreads) void ln_apply_rows_kernel(
    typename Elem<ODT>::T* __restrict__ y, typename Elem<ODT>::T* __restrict__ x_hat,
    float* __restrict__ std_out, const typename Elem<XDT>::T* __restrict__ x,
    const float* __restrict__ mean, const float* __restrict__ var,
    const typename Elem<ODT>::T* __restrict__ w, const typename Elem<ODT>::T* __restrict__ b,
    long long rows, int cols, float eps, int G) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sl = lane & (G - 1), sub = lane / G, rpw = kWave / G;
  // a wavefront's U row sets of a round lie behind each other in memory (U * rpw consecutive rows)
  const long long stride = rpw, round_stride = (long long)gridDim.x * kWavesPerBlock * rpw * U;
  float wv[CH][kPlainVec], bv[CH][kPlainVec];
  load_params_of<ODT, CH>(wv, w, G, sl, cols);
  load_params_of<ODT, CH>(bv, b, G, sl, cols);
  for (long long r0 = ((long long)blockIdx.x * kWavesPerBlock + wave) * rpw * U; r0 < rows; r0 += round_stride) {
    float v[U][CH][kPlainVec], m[U], sd[U];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const long long r = r0 + u * stride + sub;
      live[u] = r < rows;
      const long long rc = live[u] ? r : rows - 1;  // a dead row reads the last one's and stores nothing
      m[u] = mean[rc];
      sd[u] = var[rc];
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const int c = (k * G + sl) * kPlainVec;
        load8_or_zero<XDT>(x, r, rows, c, cols, v[u][k]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (!live[u]) continue;
      const long long r = r0 + u * stride + sub;
      const float s = sqrtf(sd[u] + eps);
      if (sl == 0 && std_out != nullptr) std_out[r] = s;
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const int c = (k * G + sl) * kPlainVec;
        if (c < cols) {
          float xh[kPlainVec], out[kPlainVec];
#pragma unroll
          for (int i = 0; i < kPlainVec; ++i) {
            // x_hat in the output dtype before the affine map (see ln_apply_kernel)
            xh[i] = Elem<ODT>::up(Elem<ODT>::down((v[u][k][i] - m[u]) / s));
            out[i] = wv[k][i] * xh[i] + bv[k][i];
          }
          if (x_hat != nullptr) store8<ODT>(x_hat + r * cols + c, xh);
          store8<ODT>(y + r * cols + c, out);
        }
      }
    }
  }
}

// The column partials leave the kernel as those of ln_partial_bwd_kernel do: part[blk][which][col].
// WAVES wavefronts a block (the number of blocks, and with it of partial rows, is bounded by the workspace
// contract, so more wavefronts per block is how more rows are in flight per CU); a wavefront's U row sets of
// a round lie behind each other in memory. Dynamic LDS: WAVES * 2 * cols floats.
template <int DT, int CH, int U, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void ln_partial_bwd_rows_kernel(
    float* __restrict__ mean_gxn, float* __restrict__ dot, float* __restrict__ part,
    const typename Elem<DT>::T* __restrict__ g, const typename Elem<DT>::T* __restrict__ x_hat,
    const typename Elem<DT>::T* __restrict__ w, long long rows, int cols, int G, bool want_cols) {
  extern __shared__ __attribute__((aligned(16))) float red[];  // [WAVES][2][cols]
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sl = lane & (G - 1), sub = lane / G, rpw = kWave / G;
  const float inv = 1.0f / (float)cols;
  const long long round_stride = (long long)gridDim.x * WAVES * rpw * U;
  float wv[CH][kPlainVec], agw[CH][kPlainVec], agb[CH][kPlainVec];
  load_params_of<DT, CH>(wv, w, G, sl, cols);
#pragma unroll
  for (int k = 0; k < CH; ++k)
#pragma unroll
    for (int i = 0; i < kPlainVec; ++i) {
      agw[k][i] = 0.0f;
      agb[k][i] = 0.0f;
    }
  for (long long r0 = ((long long)blockIdx.x * WAVES + wave) * rpw * U; r0 < rows; r0 += round_stride) {
    float gv[U][CH][kPlainVec], xh[U][CH][kPlainVec], s12[2 * U];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const long long r = r0 + u * rpw + sub;
      live[u] = r < rows;
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const int c = (k * G + sl) * kPlainVec;
        load8_or_zero<DT>(g, r, rows, c, cols, gv[u][k]);
        load8_or_zero<DT>(x_hat, r, rows, c, cols, xh[u][k]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float a1 = 0.0f, a2 = 0.0f;
#pragma unroll
      for (int k = 0; k < CH; ++k)
#pragma unroll
        for (int i = 0; i < kPlainVec; ++i) {
          // g * w in the tensor dtype, as the reference materialises grad_x_norm
          const float gxn = Elem<DT>::up(Elem<DT>::down(gv[u][k][i] * wv[k][i]));
          a1 += gxn;
          a2 += gxn * xh[u][k][i];
          agw[k][i] += gv[u][k][i] * xh[u][k][i];
          agb[k][i] += gv[u][k][i];
        }
      s12[u] = a1;
      s12[U + u] = a2;
    }
    group_sums<2 * U>(s12, G);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (live[u] && sl == 0) {
        const long long r = r0 + u * rpw + sub;
        mean_gxn[r] = s12[u] * inv;
        dot[r] = s12[U + u];
      }
    }
  }
  if (!want_cols) return;
  // the rows of a wavefront that share a column set: lanes sl, sl + G, ...
#pragma unroll
  for (int k = 0; k < CH; ++k)
#pragma unroll
    for (int i = 0; i < kPlainVec; ++i)
      for (int o = G; o < kWave; o <<= 1) {
        agw[k][i] += __shfl_xor(agw[k][i], o, kWave);
        agb[k][i] += __shfl_xor(agb[k][i], o, kWave);
      }
  if (sub == 0) {
#pragma unroll
    for (int k = 0; k < CH; ++k)
#pragma unroll
      for (int i = 0; i < kPlainVec; ++i) {
        const int c = (k * G + sl) * kPlainVec + i;
        if (c < cols) {
          red[(wave * 2 + 0) * cols + c] = agw[k][i];
          red[(wave * 2 + 1) * cols + c] = agb[k][i];
        }
      }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < cols; c += WAVES * kWave) {
    float a = 0.0f, b2 = 0.0f;
#pragma unroll
    for (int wv2 = 0; wv2 < WAVES; ++wv2) {
      a += red[(wv2 * 2 + 0) * cols + c];
      b2 += red[(wv2 * 2 + 1) * cols + c];
    }
    part[((long long)blockIdx.x * 2 + 0) * cols + c] = a;
    part[((long long)blockIdx.x * 2 + 1) * cols + c] = b2;
  }
}

template <int DT, int CH, int U>
__global__ __launch_bounds__(kThreads) void ln_bwd_apply_rows_kernel(
    typename Elem<DT>::T* __restrict__ gx, const typename Elem<DT>::T* __restrict__ g,
    const typename Elem<DT>::T* __restrict__ x_hat, const typename Elem<DT>::T* __restrict__ w,
    const float* __restrict__ mean_gxn, const float* __restrict__ dot, const float* __restrict__ stdv,
    long long rows, int cols, float inv_n, int G) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sl = lane & (G - 1), sub = lane / G, rpw = kWave / G;
  // a wavefront's U row sets of a round lie behind each other in memory (U * rpw consecutive rows)
  const long long stride = rpw, round_stride = (long long)gridDim.x * kWavesPerBlock * rpw * U;
  float wv[CH][kPlainVec];
  load_params_of<DT, CH>(wv, w, G, sl, cols);
  for (long long r0 = ((long long)blockIdx.x * kWavesPerBlock + wave) * rpw * U; r0 < rows; r0 += round_stride) {
    float gv[U][CH][kPlainVec], xh[U][CH][kPlainVec], m[U], dn[U], sd[U];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const long long r = r0 + u * stride + sub;
      live[u] = r < rows;
      const long long rc = live[u] ? r : rows - 1;  // a dead row reads the last one's and stores nothing
      m[u] = mean_gxn[rc];
      dn[u] = dot[rc];
      sd[u] = stdv[rc];
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const int c = (k * G + sl) * kPlainVec;
        load8_or_zero<DT>(g, r, rows, c, cols, gv[u][k]);
        load8_or_zero<DT>(x_hat, r, rows, c, cols, xh[u][k]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (!live[u]) continue;
      const long long r = r0 + u * stride + sub;
      const float rs = 1.0f / sd[u], d = dn[u] * inv_n;
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const int c = (k * G + sl) * kPlainVec;
        if (c < cols) {
          float out[kPlainVec];
#pragma unroll
          for (int i = 0; i < kPlainVec; ++i) {
            const float gxn = Elem<DT>::up(Elem<DT>::down(gv[u][k][i] * wv[k][i]));
            out[i] = rs * (gxn - m[u] - xh[u][k][i] * d);
          }
          store8<DT>(gx + r * cols + c, out);
        }
      }
    }
  }
}

// lanes per row: the power of two that covers cols / 8 columns-octets in the fewest chunks
int plain_group(long long cols) {
  int G = 1;
  while (G < kWave && (long long)G * kPlainVec < cols) G <<= 1;
  return G;
}
int plain_chunks(long long cols) {
  const int G = plain_group(cols);
  return (int)((cols + (long long)G * kPlainVec - 1) / ((long long)G * kPlainVec));
}
bool plain_ok(long long cols) { return cols >= kPlainVec && cols % kPlainVec == 0 && plain_chunks(cols) <= kPlainChunks; }
int plain_blocks(long long rows, long long cols, int most = 1024) {
  const int rpw = kWave / plain_group(cols);
  long long b = (rows + (long long)kWavesPerBlock * rpw - 1) / ((long long)kWavesPerBlock * rpw);  // one row set a wavefront
  if (b > most) b = most;
  if (b < 1) b = 1;
  return (int)b;
}
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Chunks per lane and rows in flight of the rows-in-registers kernels, as compile-time constants:
// f(chunks, rows_in_flight) with std::integral_constant arguments. U1 = rows in flight where a lane
// holds one chunk of a row (the kernels that only read keep more loads in the air).
template <int U1, typename F>
void with_row_shape(long long cols, F&& f) {
  using std::integral_constant;
  switch (plain_chunks(cols)) {
    case 1: f(integral_constant<int, 1>(), integral_constant<int, U1>()); break;
    case 2: f(integral_constant<int, 2>(), integral_constant<int, 2>()); break;
    case 3: f(integral_constant<int, 3>(), integral_constant<int, 1>()); break;
    default: f(integral_constant<int, 4>(), integral_constant<int, 1>()); break;
  }
}

template <int XDT, int YDT>
void launch_plain_fwd(void* y, float* mean, float* rstd, const void* x, const float* w, const float* b,
                      long long rows, int cols, float eps, hipStream_t s) {
  typedef typename Elem<XDT>::T XT;
  typedef typename Elem<YDT>::T YT;
  const int G = plain_group(cols), blocks = plain_blocks(rows, cols, 2048);
#define JG_GO(CH, U)                                                                                   \
  ln_plain_fwd_kernel<XDT, YDT, CH, U><<<blocks, kThreads, 0, s>>>(static_cast<YT*>(y), mean, rstd,     \
                                                                   static_cast<const XT*>(x), w, b, rows, cols, eps, G)
  switch (plain_chunks(cols)) {
    case 1: JG_GO(1, 2); break;
    case 2: JG_GO(2, 2); break;
    case 3: JG_GO(3, 1); break;
    default: JG_GO(4, 1); break;
  }
#undef JG_GO
}

template <int GDT, int XDT>
void launch_plain_bwd(void* gx, float* part, const void* g, const void* x, const float* mean, const float* rstd,
                      const float* w, long long rows, int cols, bool want_cols, const void* add, hipStream_t s) {
  typedef typename Elem<GDT>::T GT;
  typedef typename Elem<XDT>::T XT;
  const int G = plain_group(cols), blocks = plain_blocks(rows, cols);
#define JG_GO(CH, U)                                                                                     \
  ln_plain_bwd_kernel<GDT, XDT, CH, U><<<blocks, kThreads, 0, s>>>(static_cast<XT*>(gx), part,            \
                                                                   static_cast<const GT*>(g),             \
                                                                   static_cast<const XT*>(x), mean, rstd, \
                                                                   w, rows, cols, G, want_cols, static_cast<const XT*>(add))
  switch (plain_chunks(cols)) {
    case 1: JG_GO(1, 2); break;
    case 2: JG_GO(2, 2); break;
    case 3: JG_GO(3, 1); break;
    default: JG_GO(4, 1); break;
  }
#undef JG_GO
}

}  // namespace

extern "C" int jg_ln_partial_fwd(float* mean, float* var, const void* x, int64_t rows,
                                 int64_t cols, int x_dtype, void* stream) {
  JG_REQUIRE(mean && var && x, "jg_ln_partial_fwd: NULL pointer");
  JG_REQUIRE(rows >= 0 && cols >= 1, "jg_ln_partial_fwd: bad shape (%lld, %lld)",
             (long long)rows, (long long)cols);
  JG_REQUIRE(known(x_dtype), "jg_ln_partial_fwd: unknown dtype %d", x_dtype);
  if (rows == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool v = vec_aligned(x, cols, x_dtype);
  const bool in_regs = plain_ok(cols) && aligned16(x);
  const int G = in_regs ? plain_group(cols) : 0, blocks = in_regs ? plain_blocks(rows, cols, 8192) : 0;
#define JG_GO(DT)                                                                                  \
  if (in_regs)                                                                                     \
    with_row_shape<4>(cols, [&](auto ch, auto u) {                                                 \
      ln_partial_fwd_rows_kernel<DT, decltype(ch)::value, decltype(u)::value>                      \
          <<<blocks, kThreads, 0, s>>>(mean, var, static_cast<const Elem<DT>::T*>(x), rows, (int)cols, G); \
    });                                                                                            \
  else                                                                                             \
    ln_partial_fwd_kernel<DT><<<row_grid(rows), kThreads, 0, s>>>(                                 \
        mean, var, static_cast<const Elem<DT>::T*>(x), rows, cols, v)
  if (x_dtype == JG_F32) JG_GO(JG_F32);
  else if (x_dtype == JG_BF16) JG_GO(JG_BF16);
  else JG_GO(JG_F16);
#undef JG_GO
  JG_CHECK_LAUNCH("jg_ln_partial_fwd");
  return JG_OK;
}

template <int XDT, int ODT>
static void launch_apply(void* y, void* x_hat, float* std_out, const void* x, const float* mean,
                         const float* var, const void* w, const void* b, int64_t rows,
                         int64_t cols, float eps, hipStream_t s) {
  typedef typename Elem<XDT>::T XT;
  typedef typename Elem<ODT>::T OT;
  const bool vx = vec_aligned(x, cols, XDT);
  const bool vo = vec_aligned(y, cols, ODT) && (x_hat == nullptr || vec_aligned(x_hat, cols, ODT));
  const bool vw = vec_aligned(w, cols, ODT) && (b == nullptr || vec_aligned(b, cols, ODT));
  if (plain_ok(cols) && aligned16(x) && aligned16(y) && aligned16(x_hat) && aligned16(w) && aligned16(b)) {
    const int G = plain_group(cols), blocks = plain_blocks(rows, cols, 2048);
    with_row_shape<2>(cols, [&](auto ch, auto u) {
      ln_apply_rows_kernel<XDT, ODT, decltype(ch)::value, decltype(u)::value><<<blocks, kThreads, 0, s>>>(
          static_cast<OT*>(y), static_cast<OT*>(x_hat), std_out, static_cast<const XT*>(x), mean, var,
          static_cast<const OT*>(w), static_cast<const OT*>(b), rows, (int)cols, eps, G);
    });
    return;
  }
  ln_apply_kernel<XDT, ODT><<<row_grid(rows), kThreads, 0, s>>>(
      static_cast<OT*>(y), static_cast<OT*>(x_hat), std_out, static_cast<const XT*>(x), mean, var,
      static_cast<const OT*>(w), static_cast<const OT*>(b), rows, cols, eps, vx, vo, vw);
}

extern "C" int jg_ln_apply(void* y, void* x_hat, float* std_out, const void* x,
                           const float* mean, const float* var, const void* w, const void* b,
                           int64_t rows, int64_t cols, float eps, int x_dtype, int out_dtype,
                           void* stream) {
  JG_REQUIRE(y && x && mean && var && w, "jg_ln_apply: NULL pointer");
  JG_REQUIRE(rows >= 0 && cols >= 1, "jg_ln_apply: bad shape");
  JG_REQUIRE(known(x_dtype) && known(out_dtype), "jg_ln_apply: unknown dtype");
  if (rows == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define JG_GO(X, O) launch_apply<X, O>(y, x_hat, std_out, x, mean, var, w, b, rows, cols, eps, s)
  if (x_dtype == out_dtype) {
    if (x_dtype == JG_F32) JG_GO(JG_F32, JG_F32);
    else if (x_dtype == JG_BF16) JG_GO(JG_BF16, JG_BF16);
    else JG_GO(JG_F16, JG_F16);
  } else if (out_dtype == JG_F32) {
    // autocast: low-precision input promoted to fp32 on the fly
    if (x_dtype == JG_BF16) JG_GO(JG_BF16, JG_F32);
    else JG_GO(JG_F16, JG_F32);
  } else {
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_ln_apply: x dtype %d with output dtype %d", x_dtype,
            out_dtype);
  }
#undef JG_GO
  JG_CHECK_LAUNCH("jg_ln_apply");
  return JG_OK;
}

extern "C" size_t jg_ln_bwd_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return (size_t)bwd_blocks(rows) * 2 * (size_t)cols * sizeof(float);
}

template <int DT>
static int launch_partial_bwd(float* mean_gxn, float* dot, float* part, const void* g,
                              const void* x_hat, const void* w, int64_t rows, int64_t cols,
                              bool want_cols, hipStream_t s, int* blocks_used) {
  typedef typename Elem<DT>::T T;
  if (plain_ok(cols) && aligned16(g) && aligned16(x_hat) && aligned16(w)) {
    const int G = plain_group(cols);
    const int rpw = kWave / G;
    long long nb = (rows + (long long)kWavesPerBlock * rpw - 1) / ((long long)kWavesPerBlock * rpw);
    const int blocks = (int)(nb > 1024 ? 1024 : nb);  // never more than bwd_blocks(rows)
    *blocks_used = blocks;
    const size_t lds = (size_t)kWavesPerBlock * 2 * cols * sizeof(float);
    with_row_shape<2>(cols, [&](auto ch, auto u) {
      ln_partial_bwd_rows_kernel<DT, decltype(ch)::value, decltype(u)::value, kWavesPerBlock>
          <<<blocks, kThreads, lds, s>>>(mean_gxn, dot, part, static_cast<const T*>(g), static_cast<const T*>(x_hat),
                                         static_cast<const T*>(w), rows, (int)cols, G, want_cols);
    });
    return JG_OK;
  }
  *blocks_used = bwd_blocks(rows);
  const bool v = vec_aligned(g, cols, DT) && vec_aligned(x_hat, cols, DT);
  const bool vw = vec_aligned(w, cols, DT);
  const int nb = bwd_blocks(rows);
  const long long per = (long long)kWave * kVec;
  const int ch = (int)((cols + per - 1) / per);
#define JG_GO(CH)                                                                        \
  ln_partial_bwd_kernel<DT, CH><<<nb, kThreads, 0, s>>>(                                 \
      mean_gxn, dot, part, static_cast<const T*>(g), static_cast<const T*>(x_hat),       \
      static_cast<const T*>(w), rows, cols, v, vw, want_cols)
  if (ch <= 1) JG_GO(1);
  else if (ch <= 2) JG_GO(2);
  else if (ch <= 4) JG_GO(4);
  else if (ch <= kMaxChunks) JG_GO(8);
  else
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_ln_partial_bwd: local width %lld exceeds %lld",
            (long long)cols, (long long)(per * kMaxChunks));
#undef JG_GO
  return JG_OK;
}

extern "C" int jg_ln_partial_bwd(float* mean_gxn, float* dot_gxn_xhat, float* gw, float* gb,
                                 const void* g, const void* x_hat, const void* w, int64_t rows,
                                 int64_t cols, int dtype, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  JG_REQUIRE(mean_gxn && dot_gxn_xhat && g && x_hat && w, "jg_ln_partial_bwd: NULL pointer");
  JG_REQUIRE(rows >= 0 && cols >= 1, "jg_ln_partial_bwd: bad shape");
  JG_REQUIRE(known(dtype), "jg_ln_partial_bwd: unknown dtype %d", dtype);
  if (rows == 0) return JG_OK;
  const bool want_cols = gw != nullptr || gb != nullptr;
  if (want_cols) {
    JG_REQUIRE(workspace != nullptr, "jg_ln_partial_bwd: workspace is NULL");
    if (workspace_bytes < jg_ln_bwd_workspace_bytes(rows, cols))
      JG_FAIL(JG_ERR_WORKSPACE, "jg_ln_partial_bwd: workspace %zu < %zu bytes", workspace_bytes,
              jg_ln_bwd_workspace_bytes(rows, cols));
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* part = static_cast<float*>(workspace);
  int rc, nparts = 0;
  if (dtype == JG_F32)
    rc = launch_partial_bwd<JG_F32>(mean_gxn, dot_gxn_xhat, part, g, x_hat, w, rows, cols, want_cols, s, &nparts);
  else if (dtype == JG_BF16)
    rc = launch_partial_bwd<JG_BF16>(mean_gxn, dot_gxn_xhat, part, g, x_hat, w, rows, cols, want_cols, s, &nparts);
  else
    rc = launch_partial_bwd<JG_F16>(mean_gxn, dot_gxn_xhat, part, g, x_hat, w, rows, cols, want_cols, s, &nparts);
  if (rc) return rc;
  JG_CHECK_LAUNCH("jg_ln_partial_bwd");
  if (want_cols) {
    ln_colreduce_kernel<<<jg::cdiv(cols, 64), kReduceWaves * 64, 0, s>>>(gw, gb, part, nparts, cols);
    JG_CHECK_LAUNCH("jg_ln_partial_bwd(colreduce)");
  }
  return JG_OK;
}

// ---- jg_ln_partial_bwd for callers that cannot allocate ---------------------------------
// The column partials of stage 1 live in a device array that is part of the library's image
// (every GPU the library runs on holds its own copy until the process ends) instead of a
// caller-supplied workspace. In host code the array's NAME is only a handle: the address a
// kernel can use comes from hipGetSymbolAddress, once per device, with that device current.
constexpr size_t kStaticScratchBytes = JG_LN_BWD_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mu;
void* scratch_ptr[kMaxDevices];  // per device: address of that device's copy of `scratch`

// Address of the current device's scratch array. The first call on a device resolves it
// (under the mutex); later calls read the table only.
int scratch_of_current_device(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "jg_ln_partial_bwd_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_ln_partial_bwd_static: device index %d outside 0..%d", dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(scratch_mu);
  if (scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      JG_FAIL(JG_ERR_LAUNCH, "jg_ln_partial_bwd_static: hipGetSymbolAddress on device %d: %s", dev,
              hipGetErrorString(e));
    scratch_ptr[dev] = p;
  }
  *out = static_cast<float*>(scratch_ptr[dev]);
  return JG_OK;
}
}  // namespace

extern "C" int jg_ln_partial_bwd_static(float* mean_gxn, float* dot_gxn_xhat, float* gw, float* gb,
                                        const void* g, const void* x_hat, const void* w,
                                        int64_t rows, int64_t cols, int dtype, void* stream) {
  JG_REQUIRE(rows >= 0 && cols >= 1, "jg_ln_partial_bwd_static: bad shape");
  const size_t need = (gw != nullptr || gb != nullptr) ? jg_ln_bwd_workspace_bytes(rows, cols) : 0;
  if (need > kStaticScratchBytes)
    JG_FAIL(JG_ERR_WORKSPACE,
            "jg_ln_partial_bwd_static: %lld rows x %lld columns need %zu bytes of column partials, the "
            "built-in scratch holds %zu; use jg_ln_partial_bwd with a workspace",
            (long long)rows, (long long)cols, need, kStaticScratchBytes);
  float* part = nullptr;
  if (need != 0) {
    int rc = scratch_of_current_device(&part);
    if (rc) return rc;
  }
  // Every partial that stage 2 reads is written by stage 1 of the same call, so nothing has
  // to start at zero; the shared kernels take the address as they take a workspace.
  return jg_ln_partial_bwd(mean_gxn, dot_gxn_xhat, gw, gb, g, x_hat, w, rows, cols, dtype, part,
                           kStaticScratchBytes, stream);
}

extern "C" int jg_ln_bwd_apply(void* gx, const void* g, const void* x_hat, const void* w,
                               const float* mean_gxn, const float* dot_gxn_xhat,
                               const float* std, int64_t rows, int64_t cols, int64_t n_global,
                               int dtype, void* stream) {
  JG_REQUIRE(gx && g && x_hat && w && mean_gxn && dot_gxn_xhat && std,
             "jg_ln_bwd_apply: NULL pointer");
  JG_REQUIRE(rows >= 0 && cols >= 1 && n_global >= 1, "jg_ln_bwd_apply: bad shape");
  JG_REQUIRE(known(dtype), "jg_ln_bwd_apply: unknown dtype %d", dtype);
  if (rows == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float inv_n = 1.0f / (float)n_global;
#define JG_GO(DT)                                                                          \
  do {                                                                                     \
    typedef Elem<DT>::T T;                                                                 \
    const bool v = vec_aligned(g, cols, DT) && vec_aligned(x_hat, cols, DT) &&             \
                   vec_aligned(gx, cols, DT);                                              \
    const bool vw = vec_aligned(w, cols, DT);                                              \
    if (plain_ok(cols) && aligned16(gx) && aligned16(g) && aligned16(x_hat) && aligned16(w)) { \
      const int G = plain_group(cols), blocks = plain_blocks(rows, cols, 2048);                  \
      with_row_shape<2>(cols, [&](auto ch, auto u) {                                       \
        ln_bwd_apply_rows_kernel<DT, decltype(ch)::value, decltype(u)::value>              \
            <<<blocks, kThreads, 0, s>>>(static_cast<T*>(gx), static_cast<const T*>(g),    \
                                         static_cast<const T*>(x_hat), static_cast<const T*>(w), \
                                         mean_gxn, dot_gxn_xhat, std, rows, (int)cols, inv_n, G); \
      });                                                                                  \
    } else                                                                                 \
    ln_bwd_apply_kernel<DT><<<row_grid(rows), kThreads, 0, s>>>(                           \
        static_cast<T*>(gx), static_cast<const T*>(g), static_cast<const T*>(x_hat),       \
        static_cast<const T*>(w), mean_gxn, dot_gxn_xhat, std, rows, cols, inv_n, v, vw);  \
  } while (0)
  if (dtype == JG_F32) JG_GO(JG_F32);
  else if (dtype == JG_BF16) JG_GO(JG_BF16);
  else JG_GO(JG_F16);
#undef JG_GO
  JG_CHECK_LAUNCH("jg_ln_bwd_apply");
  return JG_OK;
}


extern "C" int jg_ln_plain_supported(int64_t cols) { return plain_ok(cols) ? 1 : 0; }

extern "C" int jg_ln_plain_fwd(void* y, float* mean, float* rstd, const void* x, const float* w,
                               const float* b, int64_t rows, int64_t cols, float eps, int x_dtype,
                               int y_dtype, void* stream) {
  const char* who = "jg_ln_plain_fwd";
  JG_REQUIRE(y && mean && rstd && x && w, "%s: NULL pointer", who);
  JG_REQUIRE(rows >= 0 && cols >= 1, "%s: bad shape (%lld, %lld)", who, (long long)rows, (long long)cols);
  JG_REQUIRE(known(x_dtype) && known(y_dtype), "%s: unknown dtype", who);
  if (!plain_ok(cols))
    JG_FAIL(JG_ERR_UNSUPPORTED, "%s: %lld columns (needs a multiple of 8, at most %d)", who, (long long)cols,
            kPlainChunks * kWave * kPlainVec);
  JG_REQUIRE(aligned16(y) && aligned16(x) && aligned16(w) && aligned16(b), "%s: x, y, w and b must be 16-byte aligned", who);
  JG_REQUIRE(y_dtype == x_dtype || y_dtype == JG_F32 || x_dtype == JG_F32, "%s: x dtype %d with y dtype %d", who,
             x_dtype, y_dtype);
  if (rows == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define JG_GO(X, Y) launch_plain_fwd<X, Y>(y, mean, rstd, x, w, b, rows, (int)cols, eps, s)
  if (x_dtype == JG_F32) {
    if (y_dtype == JG_F32) JG_GO(JG_F32, JG_F32);
    else if (y_dtype == JG_BF16) JG_GO(JG_F32, JG_BF16);
    else JG_GO(JG_F32, JG_F16);
  } else if (x_dtype == JG_BF16) {
    if (y_dtype == JG_F32) JG_GO(JG_BF16, JG_F32);
    else JG_GO(JG_BF16, JG_BF16);
  } else {
    if (y_dtype == JG_F32) JG_GO(JG_F16, JG_F32);
    else JG_GO(JG_F16, JG_F16);
  }
#undef JG_GO
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

extern "C" size_t jg_ln_plain_bwd_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0 || !plain_ok(cols)) return 0;
  return (size_t)plain_blocks(rows, cols) * 2 * (size_t)cols * sizeof(float);
}

static int plain_bwd_common(const char* who, void* gx, float* gw, float* gb, const void* g, const void* x,
                            const float* mean, const float* rstd, const float* w, int64_t rows, int64_t cols,
                            int g_dtype, int x_dtype, void* workspace, size_t workspace_bytes, const void* add,
                            void* stream) {
  JG_REQUIRE(g && x && mean && rstd && w, "%s: NULL pointer", who);
  JG_REQUIRE(add == nullptr || (gx != nullptr && aligned16(add)), "%s: add needs gx and 16-byte alignment", who);
  JG_REQUIRE(rows >= 0 && cols >= 1, "%s: bad shape (%lld, %lld)", who, (long long)rows, (long long)cols);
  JG_REQUIRE(known(x_dtype) && known(g_dtype), "%s: unknown dtype", who);
  if (!plain_ok(cols))
    JG_FAIL(JG_ERR_UNSUPPORTED, "%s: %lld columns (needs a multiple of 8, at most %d)", who, (long long)cols,
            kPlainChunks * kWave * kPlainVec);
  JG_REQUIRE(aligned16(g) && aligned16(x) && aligned16(w) && (gx == nullptr || aligned16(gx)),
             "%s: g, x, w and gx must be 16-byte aligned", who);
  JG_REQUIRE(g_dtype == x_dtype || g_dtype == JG_F32 || x_dtype == JG_F32, "%s: g dtype %d with x dtype %d", who,
             g_dtype, x_dtype);
  const bool want_cols = gw != nullptr || gb != nullptr;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (rows == 0) {
    // no rows: the column sums are zero (a fill kernel, so that the call can be captured in a graph)
    if (want_cols) {
      ln_colreduce_kernel<<<(unsigned)((cols + 63) / 64), kReduceWaves * 64, 0, s>>>(gw, gb, nullptr, 0, cols);
      JG_CHECK_LAUNCH(who);
    }
    return JG_OK;
  }
  float* part = static_cast<float*>(workspace);
  if (want_cols) {
    const size_t need = jg_ln_plain_bwd_workspace_bytes(rows, cols);
    if (workspace == nullptr || workspace_bytes < need)
      JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, workspace_bytes, need);
  }
#define JG_GO(G_, X) launch_plain_bwd<G_, X>(gx, part, g, x, mean, rstd, w, rows, (int)cols, want_cols, add, s)
  if (x_dtype == JG_F32) {
    if (g_dtype == JG_F32) JG_GO(JG_F32, JG_F32);
    else if (g_dtype == JG_BF16) JG_GO(JG_BF16, JG_F32);
    else JG_GO(JG_F16, JG_F32);
  } else if (x_dtype == JG_BF16) {
    if (g_dtype == JG_F32) JG_GO(JG_F32, JG_BF16);
    else JG_GO(JG_BF16, JG_BF16);
  } else {
    if (g_dtype == JG_F32) JG_GO(JG_F32, JG_F16);
    else JG_GO(JG_F16, JG_F16);
  }
#undef JG_GO
  JG_CHECK_LAUNCH(who);
  if (want_cols) {
    ln_colreduce_kernel<<<(unsigned)((cols + 63) / 64), kReduceWaves * 64, 0, s>>>(gw, gb, part, plain_blocks(rows, cols), cols);
    JG_CHECK_LAUNCH(who);
  }
  return JG_OK;
}

extern "C" int jg_ln_plain_bwd(void* gx, float* gw, float* gb, const void* g, const void* x,
                               const float* mean, const float* rstd, const float* w, int64_t rows,
                               int64_t cols, int g_dtype, int x_dtype, void* workspace,
                               size_t workspace_bytes, void* stream) {
  return plain_bwd_common("jg_ln_plain_bwd", gx, gw, gb, g, x, mean, rstd, w, rows, cols, g_dtype, x_dtype, workspace,
                          workspace_bytes, nullptr, stream);
}

extern "C" int jg_ln_plain_bwd_add(void* gx, float* gw, float* gb, const void* g, const void* x,
                                   const float* mean, const float* rstd, const float* w, int64_t rows,
                                   int64_t cols, int g_dtype, int x_dtype, void* workspace,
                                   size_t workspace_bytes, const void* add, void* stream) {
  const char* who = "jg_ln_plain_bwd_add";
  JG_REQUIRE(add != nullptr && gx != nullptr, "%s: NULL pointer", who);
  return plain_bwd_common(who, gx, gw, gb, g, x, mean, rstd, w, rows, cols, g_dtype, x_dtype, workspace,
                          workspace_bytes, add, stream);
}
