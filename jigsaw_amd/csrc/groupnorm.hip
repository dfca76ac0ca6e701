// GroupNorm over a spatially sharded input: the per-(sample, group) partial sums that
// the ranks add up, the normalise + affine pass, and the backward partials and pass.
// x is (N, C, S) contiguous (S = product of the local spatial extents); a group is
// C / G consecutive channels, so the elements of one (sample, group) are one contiguous
// span. Everything is HBM-bound: 16-byte loads, fp32 accumulation, block partials that a
// second small kernel adds up in a fixed order (deterministic, no atomics).
//
// Reference behaviour restated here:
//   jigsaw/modules/normalization/_functional.py:352-385 (forward: sum, centred squares, apply)
//   jigsaw/modules/normalization/_functional.py:431-468 (backward)
#include "jg_common.h"

namespace {

constexpr int kThreads = 256;
constexpr long long kChunk = 32768;  // elements a block reduces
constexpr int kMaxChunks = 64;

template <int DT>
struct Elem;
template <>
struct Elem<JG_F32> {
  typedef float T;
  static constexpr int VEC = 4;
  __device__ static __forceinline__ float up(float v) { return v; }
  __device__ static __forceinline__ float down(float v) { return v; }
};
template <>
struct Elem<JG_BF16> {
  typedef uint16_t T;
  static constexpr int VEC = 8;
  __device__ static __forceinline__ float up(uint16_t v) { return jg::bf16_to_f32(v); }
  __device__ static __forceinline__ uint16_t down(float v) { return jg::f32_to_bf16(v); }
};
template <>
struct Elem<JG_F16> {
  typedef _Float16 T;
  static constexpr int VEC = 8;
  __device__ static __forceinline__ float up(_Float16 v) { return (float)v; }
  __device__ static __forceinline__ _Float16 down(float v) { return (_Float16)v; }
};

template <int DT>
struct alignas(16) Pack {
  typename Elem<DT>::T v[Elem<DT>::VEC];
};

// Elements [i, i + VEC) of a span of `len` elements; zeros past the end.
template <int DT>
__device__ __forceinline__ void load_vec(const typename Elem<DT>::T* p, long long i, long long len, bool vec_ok,
                                         float out[Elem<DT>::VEC]) {
  constexpr int V = Elem<DT>::VEC;
  if (vec_ok && i + V <= len) {
    const Pack<DT> q = *reinterpret_cast<const Pack<DT>*>(p + i);
#pragma unroll
    for (int t = 0; t < V; ++t) out[t] = Elem<DT>::up(q.v[t]);
  } else {
#pragma unroll
    for (int t = 0; t < V; ++t) out[t] = (i + t < len) ? Elem<DT>::up(p[i + t]) : 0.0f;
  }
}

template <int DT>
__device__ __forceinline__ void store_vec(typename Elem<DT>::T* p, long long i, long long len, bool vec_ok,
                                          const float in[Elem<DT>::VEC]) {
  constexpr int V = Elem<DT>::VEC;
  if (vec_ok && i + V <= len) {
    Pack<DT> q;
#pragma unroll
    for (int t = 0; t < V; ++t) q.v[t] = Elem<DT>::down(in[t]);
    *reinterpret_cast<Pack<DT>*>(p + i) = q;
  } else {
#pragma unroll
    for (int t = 0; t < V; ++t)
      if (i + t < len) p[i + t] = Elem<DT>::down(in[t]);
  }
}

// Sum of two per-thread values over the block, fixed order; valid in thread 0.
__device__ __forceinline__ void block_sum2(float& a, float& b) {
  __shared__ float red[2][kThreads / 64];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    a += __shfl_xor(a, o, 64);
    b += __shfl_xor(b, o, 64);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    red[0][wave] = a;
    red[1][wave] = b;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    a = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
    b = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
  }
}

// MODE 0: part[0] = sum x                      over a chunk of a (sample, group) span
// MODE 1: part[0] = sum (x - mean[unit])^2      "
// MODE 2: part[0] = sum g, part[1] = sum g * y  over a chunk of a (sample, channel) row
// Block b handles chunk b % chunks of unit b / chunks; partials at part[(b) * 2 + {0, 1}].
template <int DT, int MODE>
__global__ __launch_bounds__(kThreads) void gn_reduce_kernel(float* __restrict__ part,
                                                             const typename Elem<DT>::T* __restrict__ x,
                                                             const typename Elem<DT>::T* __restrict__ y,
                                                             const float* __restrict__ mean, long long len,
                                                             int chunks, long long chunk_len, bool vec_ok) {
  constexpr int V = Elem<DT>::VEC;
  const long long unit = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const typename Elem<DT>::T* xs = x + unit * len;
  const typename Elem<DT>::T* ys = MODE == 2 ? y + unit * len : nullptr;
  const float m = MODE == 1 ? mean[unit] : 0.0f;
  const long long lo = chunk * chunk_len;
  long long hi = lo + chunk_len;
  if (hi > len) hi = len;
  float a = 0.0f, b = 0.0f;
  for (long long i = lo + (long long)threadIdx.x * V; i < hi; i += (long long)kThreads * V) {
    float v[V];
    load_vec<DT>(xs, i, hi, vec_ok, v);
    if (MODE == 0) {
#pragma unroll
      for (int t = 0; t < V; ++t) a += v[t];
    } else if (MODE == 1) {
#pragma unroll
      for (int t = 0; t < V; ++t) {
        const float d = (i + t < hi) ? v[t] - m : 0.0f;
        a += d * d;
      }
    } else {
      float w[V];
      load_vec<DT>(ys, i, hi, vec_ok, w);
#pragma unroll
      for (int t = 0; t < V; ++t) {
        a += v[t];
        b += v[t] * w[t];
      }
    }
  }
  block_sum2(a, b);
  if (threadIdx.x == 0) {
    part[(size_t)blockIdx.x * 2 + 0] = a;
    part[(size_t)blockIdx.x * 2 + 1] = b;
  }
}

// out0[u] (and out1[u]) = sum over the chunks of unit u, in chunk order
__global__ __launch_bounds__(kThreads) void gn_finish_kernel(float* __restrict__ out0, float* __restrict__ out1,
                                                             const float* __restrict__ part, long long units,
                                                             int chunks) {
  const long long u = (long long)blockIdx.x * kThreads + threadIdx.x;
  if (u >= units) return;
  float a = 0.0f, b = 0.0f;
  for (int k = 0; k < chunks; ++k) {
    a += part[((size_t)u * chunks + k) * 2 + 0];
    b += part[((size_t)u * chunks + k) * 2 + 1];
  }
  out0[u] = a;
  if (out1 != nullptr) out1[u] = b;
}

// From the row sums a[n][c] = sum g, b[n][c] = sum g * x_norm:
//   threads [0, N*G):       gsum[n][grp] = sum_c w[c] a[n][c], gxsum[n][grp] = sum_c w[c] b[n][c]
//   threads [N*G, N*G + C): gb[c] = sum_n a[n][c], gw[c] = sum_n b[n][c]
template <int DT>
__global__ __launch_bounds__(kThreads) void gn_bwd_finish_kernel(float* __restrict__ gsum, float* __restrict__ gxsum,
                                                                 float* __restrict__ gw, float* __restrict__ gb,
                                                                 const float* __restrict__ ra,
                                                                 const float* __restrict__ rb,
                                                                 const typename Elem<DT>::T* __restrict__ weight,
                                                                 long long N, long long C, long long G) {
  const long long t = (long long)blockIdx.x * kThreads + threadIdx.x;
  const long long cpg = C / G;
  if (t < N * G) {
    const long long n = t / G, grp = t % G;
    float s0 = 0.0f, s1 = 0.0f;
    for (long long c = grp * cpg; c < (grp + 1) * cpg; ++c) {
      const float w = weight != nullptr ? Elem<DT>::up(weight[c]) : 1.0f;
      s0 += w * ra[n * C + c];
      s1 += w * rb[n * C + c];
    }
    gsum[t] = s0;
    gxsum[t] = s1;
  } else if (t < N * G + C) {
    const long long c = t - N * G;
    float s0 = 0.0f, s1 = 0.0f;
    for (long long n = 0; n < N; ++n) {
      s0 += ra[n * C + c];
      s1 += rb[n * C + c];
    }
    if (gb != nullptr) gb[c] = s0;
    if (gw != nullptr) gw[c] = s1;
  }
}

// Forward:  x_norm = (x - mean) * rstd, y = x_norm * w[c] + b[c]
// Backward: gx = rstd * (g * w[c] - gsum / cnt - x_norm * gxsum / cnt)
// Block b handles chunk b % chunks of row (n, c) = b / chunks.
template <int DT, bool BWD>
__global__ __launch_bounds__(kThreads) void gn_apply_kernel(
    typename Elem<DT>::T* __restrict__ out, typename Elem<DT>::T* __restrict__ out_norm,
    const typename Elem<DT>::T* __restrict__ in, const typename Elem<DT>::T* __restrict__ in_norm,
    const float* __restrict__ s0, const float* __restrict__ s1, const float* __restrict__ s2,
    const float* __restrict__ cnt, const typename Elem<DT>::T* __restrict__ weight,
    const typename Elem<DT>::T* __restrict__ bias, long long C, long long G, long long S, int chunks,
    long long chunk_len, bool vec_ok) {
  constexpr int V = Elem<DT>::VEC;
  const long long row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const long long n = row / C, c = row % C;
  const long long seg = n * G + c / (C / G);
  const float w = weight != nullptr ? Elem<DT>::up(weight[c]) : 1.0f;
  const float bv = (!BWD && bias != nullptr) ? Elem<DT>::up(bias[c]) : 0.0f;
  // forward: s0 = mean, s1 = rstd; backward: s0 = rstd, s1 = gsum, s2 = gxsum
  const float p0 = s0[seg], p1 = s1[seg];
  const float inv = BWD ? 1.0f / cnt[seg] : 0.0f;
  const float q1 = BWD ? p1 * inv : 0.0f, q2 = BWD ? s2[seg] * inv : 0.0f;
  const long long lo = chunk * chunk_len;
  long long hi = lo + chunk_len;
  if (hi > S) hi = S;
  const typename Elem<DT>::T* src = in + row * S;
  const typename Elem<DT>::T* srcn = BWD ? in_norm + row * S : nullptr;
  typename Elem<DT>::T* dst = out + row * S;
  typename Elem<DT>::T* dstn = BWD ? nullptr : out_norm + row * S;
  for (long long i = lo + (long long)threadIdx.x * V; i < hi; i += (long long)kThreads * V) {
    float v[V], r[V];
    load_vec<DT>(src, i, hi, vec_ok, v);
    if (!BWD) {
      float xn[V];
#pragma unroll
      for (int t = 0; t < V; ++t) {
        // x_norm is stored in the compute dtype and y is computed from the stored value,
        // as the reference computes y from the x_norm tensor
        xn[t] = Elem<DT>::up(Elem<DT>::down((v[t] - p0) * p1));
        r[t] = xn[t] * w + bv;
      }
      store_vec<DT>(dstn, i, hi, vec_ok, xn);
    } else {
      float xn[V];
      load_vec<DT>(srcn, i, hi, vec_ok, xn);
#pragma unroll
      for (int t = 0; t < V; ++t) r[t] = p0 * (v[t] * w - q1 - xn[t] * q2);
    }
    store_vec<DT>(dst, i, hi, vec_ok, r);
  }
}

int chunks_of(long long len) {
  long long c = (len + kChunk - 1) / kChunk;
  if (c < 1) c = 1;
  if (c > kMaxChunks) c = kMaxChunks;
  return (int)c;
}

// chunk length: a multiple of 8 elements, so that chunk starts keep the 16-byte alignment
long long chunk_len_of(long long len, int chunks) {
  long long l = (len + chunks - 1) / chunks;
  return (l + 7) / 8 * 8;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check(const char* who, int64_t N, int64_t C, int64_t S, int64_t G, int dtype) {
  JG_REQUIRE(dtype == JG_F32 || dtype == JG_BF16 || dtype == JG_F16, "%s: unknown dtype %d", who, dtype);
  JG_REQUIRE(N >= 0 && C >= 1 && S >= 0 && G >= 1, "%s: bad shape", who);
  JG_REQUIRE(C % G == 0, "%s: %lld channels do not divide into %lld groups", who, (long long)C, (long long)G);
  JG_REQUIRE(N * C * (int64_t)kMaxChunks < (1ll << 31), "%s: too many rows", who);
  return JG_OK;
}

size_t ws_need(int64_t N, int64_t C, int64_t S) {
  // the larger of: per-row partials + row sums (backward), per-group partials (forward)
  const size_t rows = (size_t)N * (size_t)C;
  return (rows * (size_t)chunks_of(S) * 2 + rows * 2) * sizeof(float) + 256;
}

template <int DT, int MODE>
int reduce_launch(float* out0, float* out1, const void* x, const void* y, const float* mean, long long units,
                  long long len, float* ws, hipStream_t s, const char* who) {
  typedef typename Elem<DT>::T T;
  if (units == 0) return JG_OK;
  const int chunks = chunks_of(len);
  const long long cl = chunk_len_of(len, chunks);
  const bool vec_ok = aligned16(x) && (MODE != 2 || aligned16(y)) && (len * (long long)sizeof(T)) % 16 == 0;
  gn_reduce_kernel<DT, MODE><<<(unsigned)(units * chunks), kThreads, 0, s>>>(
      ws, static_cast<const T*>(x), static_cast<const T*>(y), mean, len, chunks, cl, vec_ok);
  JG_CHECK_LAUNCH(who);
  gn_finish_kernel<<<(unsigned)((units + kThreads - 1) / kThreads), kThreads, 0, s>>>(out0, out1, ws, units, chunks);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

}  // namespace

extern "C" size_t jg_gn_workspace_bytes(int64_t batch, int64_t channels, int64_t spatial) {
  if (batch <= 0 || channels <= 0 || spatial <= 0) return 256;
  return ws_need(batch, channels, spatial);
}

#define JG_GN_DISPATCH(CALL)                    \
  switch (dtype) {                              \
    case JG_F32: return CALL(JG_F32);           \
    case JG_BF16: return CALL(JG_BF16);         \
    default: return CALL(JG_F16);               \
  }

extern "C" int jg_gn_partial_sum(float* sum, const void* x, int64_t batch, int64_t channels, int64_t spatial,
                                 int64_t groups, int dtype, void* workspace, size_t workspace_bytes,
                                 void* stream) {
  const char* who = "jg_gn_partial_sum";
  int rc = check(who, batch, channels, spatial, groups, dtype);
  if (rc) return rc;
  JG_REQUIRE(sum && x, "%s: NULL pointer", who);
  if (workspace == nullptr || workspace_bytes < jg_gn_workspace_bytes(batch, channels, spatial))
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, workspace_bytes,
            jg_gn_workspace_bytes(batch, channels, spatial));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long long units = batch * groups, len = channels / groups * spatial;
#define CALL(DT) reduce_launch<DT, 0>(sum, nullptr, x, nullptr, nullptr, units, len, static_cast<float*>(workspace), s, who)
  JG_GN_DISPATCH(CALL)
#undef CALL
}

extern "C" int jg_gn_partial_sqdev(float* sq, const void* x, const float* mean, int64_t batch, int64_t channels,
                                   int64_t spatial, int64_t groups, int dtype, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  const char* who = "jg_gn_partial_sqdev";
  int rc = check(who, batch, channels, spatial, groups, dtype);
  if (rc) return rc;
  JG_REQUIRE(sq && x && mean, "%s: NULL pointer", who);
  if (workspace == nullptr || workspace_bytes < jg_gn_workspace_bytes(batch, channels, spatial))
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, workspace_bytes,
            jg_gn_workspace_bytes(batch, channels, spatial));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long long units = batch * groups, len = channels / groups * spatial;
#define CALL(DT) reduce_launch<DT, 1>(sq, nullptr, x, nullptr, mean, units, len, static_cast<float*>(workspace), s, who)
  JG_GN_DISPATCH(CALL)
#undef CALL
}

namespace {
template <int DT, bool BWD>
int apply_launch(void* out, void* out_norm, const void* in, const void* in_norm, const float* s0, const float* s1,
                 const float* s2, const float* cnt, const void* weight, const void* bias, long long N,
                 long long C, long long S, long long G, hipStream_t s, const char* who) {
  typedef typename Elem<DT>::T T;
  const long long rows = N * C;
  if (rows == 0 || S == 0) return JG_OK;
  const int chunks = chunks_of(S);
  const long long cl = chunk_len_of(S, chunks);
  const bool vec_ok = aligned16(out) && aligned16(in) && (BWD ? aligned16(in_norm) : aligned16(out_norm)) &&
                      (S * (long long)sizeof(T)) % 16 == 0;
  gn_apply_kernel<DT, BWD><<<(unsigned)(rows * chunks), kThreads, 0, s>>>(
      static_cast<T*>(out), static_cast<T*>(out_norm), static_cast<const T*>(in), static_cast<const T*>(in_norm), s0,
      s1, s2, cnt, static_cast<const T*>(weight), static_cast<const T*>(bias), C, G, S, chunks, cl, vec_ok);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}
}  // namespace

extern "C" int jg_gn_apply(void* y, void* x_norm, const void* x, const float* mean, const float* rstd,
                           const void* weight, const void* bias, int64_t batch, int64_t channels,
                           int64_t spatial, int64_t groups, int dtype, void* stream) {
  const char* who = "jg_gn_apply";
  int rc = check(who, batch, channels, spatial, groups, dtype);
  if (rc) return rc;
  JG_REQUIRE(y && x_norm && x && mean && rstd, "%s: NULL pointer", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define CALL(DT) \
  apply_launch<DT, false>(y, x_norm, x, nullptr, mean, rstd, nullptr, nullptr, weight, bias, batch, channels, spatial, groups, s, who)
  JG_GN_DISPATCH(CALL)
#undef CALL
}

extern "C" int jg_gn_partial_bwd(float* gsum, float* gxsum, float* gw, float* gb, const void* g,
                                 const void* x_norm, const void* weight, int64_t batch, int64_t channels,
                                 int64_t spatial, int64_t groups, int dtype, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  const char* who = "jg_gn_partial_bwd";
  int rc = check(who, batch, channels, spatial, groups, dtype);
  if (rc) return rc;
  JG_REQUIRE(gsum && gxsum && g && x_norm, "%s: NULL pointer", who);
  if (workspace == nullptr || workspace_bytes < jg_gn_workspace_bytes(batch, channels, spatial))
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, workspace_bytes,
            jg_gn_workspace_bytes(batch, channels, spatial));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long long rows = batch * channels;
  if (rows == 0) return JG_OK;
  float* part = static_cast<float*>(workspace);
  float* ra = part + (size_t)rows * chunks_of(spatial) * 2;  // row sums behind the chunk partials
  float* rb = ra + rows;
  const unsigned fin = (unsigned)((batch * groups + channels + kThreads - 1) / kThreads);
#define CALL(DT)                                                                                          \
  [&]() -> int {                                                                                          \
    int r2 = reduce_launch<DT, 2>(ra, rb, g, x_norm, nullptr, rows, spatial, part, s, who);               \
    if (r2) return r2;                                                                                    \
    gn_bwd_finish_kernel<DT><<<fin, kThreads, 0, s>>>(gsum, gxsum, gw, gb, ra, rb,                        \
                                                      static_cast<const Elem<DT>::T*>(weight), batch,     \
                                                      channels, groups);                                  \
    JG_CHECK_LAUNCH(who);                                                                                 \
    return JG_OK;                                                                                         \
  }()
  JG_GN_DISPATCH(CALL)
#undef CALL
}

extern "C" int jg_gn_bwd_apply(void* gx, const void* g, const void* x_norm, const void* weight, const float* rstd,
                               const float* gsum, const float* gxsum, const float* count, int64_t batch,
                               int64_t channels, int64_t spatial, int64_t groups, int dtype, void* stream) {
  const char* who = "jg_gn_bwd_apply";
  int rc = check(who, batch, channels, spatial, groups, dtype);
  if (rc) return rc;
  JG_REQUIRE(gx && g && x_norm && rstd && gsum && gxsum && count, "%s: NULL pointer", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define CALL(DT) \
  apply_launch<DT, true>(gx, nullptr, g, x_norm, rstd, gsum, gxsum, count, weight, nullptr, batch, channels, spatial, groups, s, who)
  JG_GN_DISPATCH(CALL)
#undef CALL
}
