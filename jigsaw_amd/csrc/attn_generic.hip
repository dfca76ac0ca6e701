// Attention core for any sequence length and head size up to 128, with an
// optional additive bias / mask: forward (output + natural-log LSE) and backward
// from a given (global) output and LSE. One thread owns one query row (forward,
// dQ) or one key row (dK/dV); the other side is streamed through LDS in tiles
// and read as broadcasts. fp32 arithmetic throughout. This is the path for
// shapes the MFMA flash kernels do not cover (short or ragged sequences, head
// sizes other than 64, windowed attention with a relative-position bias).
//
// Reference behaviour restated here:
//   jigsaw/modules/attention/_functional/cores/math.py:69-78   (forward)
//   jigsaw/modules/attention/_functional/cores/math.py:125-149 (backward)
//   examples/swin.py:148-151 (softmax(q k^T / sqrt(d) + bias) v)
#include "jg_common.h"

namespace {

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

constexpr int kRows = 64;   // rows (queries or keys) per workgroup, one per thread
constexpr int kTile = 32;   // rows of the streamed side per LDS tile

struct AttnArgs {
  long long batch;   // b * h (flattened leading axes)
  int sq, sk, d;
  float scale;
  const float* bias; // (bias_period, sq, sk) fp32 or NULL
  long long bias_period;
};

// Stage `rows` x D values (row-major, zero beyond `valid` rows) into LDS as fp32.
template <int DT, int D>
__device__ __forceinline__ void stage_rows(float* dst, const typename Elem<DT>::T* src, int valid) {
  for (int i = threadIdx.x; i < kTile * D; i += kRows) {
    const int r = i / D;
    dst[i] = (r < valid) ? Elem<DT>::up(src[i]) : 0.0f;
  }
}

// ------------------------------------------------------------------- forward
template <int DT, int D>
__global__ __launch_bounds__(kRows) void attn_fwd_generic(typename Elem<DT>::T* __restrict__ out,
                                                          float* __restrict__ lse,
                                                          const typename Elem<DT>::T* __restrict__ q,
                                                          const typename Elem<DT>::T* __restrict__ k,
                                                          const typename Elem<DT>::T* __restrict__ v,
                                                          AttnArgs a) {
  __shared__ float ks[kTile * D];
  __shared__ float vs[kTile * D];
  const long long b = blockIdx.y;
  const int row = blockIdx.x * kRows + threadIdx.x;
  const bool live = row < a.sq;
  float qr[D], acc[D];
#pragma unroll
  for (int i = 0; i < D; ++i) {
    qr[i] = live ? Elem<DT>::up(q[(b * a.sq + row) * D + i]) * a.scale : 0.0f;
    acc[i] = 0.0f;
  }
  const float* brow = (a.bias != nullptr && live)
                          ? a.bias + ((b % a.bias_period) * a.sq + row) * (long long)a.sk
                          : nullptr;
  float m = -INFINITY, l = 0.0f;
  for (int k0 = 0; k0 < a.sk; k0 += kTile) {
    const int valid = min(kTile, a.sk - k0);
    __syncthreads();
    stage_rows<DT, D>(ks, k + (b * a.sk + k0) * D, valid);
    stage_rows<DT, D>(vs, v + (b * a.sk + k0) * D, valid);
    __syncthreads();
    for (int j = 0; j < valid; ++j) {
      float s = 0.0f;
#pragma unroll
      for (int i = 0; i < D; ++i) s += qr[i] * ks[j * D + i];
      if (brow != nullptr) s += brow[k0 + j];
      const float mn = fmaxf(m, s);
      // a fully masked prefix keeps m = -inf; exp(-inf - -inf) must not produce NaN
      const float alpha = (mn == -INFINITY) ? 1.0f : __expf(m - mn);
      const float p = (mn == -INFINITY) ? 0.0f : __expf(s - mn);
      l = l * alpha + p;
#pragma unroll
      for (int i = 0; i < D; ++i) acc[i] = acc[i] * alpha + p * vs[j * D + i];
      m = mn;
    }
  }
  if (live) {
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < D; ++i) out[(b * a.sq + row) * D + i] = Elem<DT>::down(acc[i] * inv);
    lse[b * a.sq + row] = m + __logf(l);
  }
}

// ------------------------------------------------------------ backward: dQ
// Also writes delta[q] = rowsum(dO * O) for the dK/dV kernel, and optionally the
// gradient of the additive bias, ds_bias[b][q][k] = p * (dp - delta).
template <int DT, int D>
__global__ __launch_bounds__(kRows) void attn_bwd_dq_generic(
    typename Elem<DT>::T* __restrict__ dq, float* __restrict__ delta, float* __restrict__ dbias,
    const typename Elem<DT>::T* __restrict__ dout, const typename Elem<DT>::T* __restrict__ q,
    const typename Elem<DT>::T* __restrict__ k, const typename Elem<DT>::T* __restrict__ v,
    const typename Elem<DT>::T* __restrict__ out, const float* __restrict__ lse, AttnArgs a) {
  __shared__ float ks[kTile * D];
  __shared__ float vs[kTile * D];
  const long long b = blockIdx.y;
  const int row = blockIdx.x * kRows + threadIdx.x;
  const bool live = row < a.sq;
  float qr[D], dor[D], acc[D];
  float dl = 0.0f;
#pragma unroll
  for (int i = 0; i < D; ++i) {
    qr[i] = live ? Elem<DT>::up(q[(b * a.sq + row) * D + i]) * a.scale : 0.0f;
    dor[i] = live ? Elem<DT>::up(dout[(b * a.sq + row) * D + i]) : 0.0f;
    const float o = live ? Elem<DT>::up(out[(b * a.sq + row) * D + i]) : 0.0f;
    dl += dor[i] * o;
    acc[i] = 0.0f;
  }
  const float L = live ? lse[b * a.sq + row] : 0.0f;
  if (live) delta[b * a.sq + row] = dl;
  const float* brow = (a.bias != nullptr && live)
                          ? a.bias + ((b % a.bias_period) * a.sq + row) * (long long)a.sk
                          : nullptr;
  float* dbrow = (dbias != nullptr && live) ? dbias + (b * a.sq + row) * (long long)a.sk : nullptr;
  for (int k0 = 0; k0 < a.sk; k0 += kTile) {
    const int valid = min(kTile, a.sk - k0);
    __syncthreads();
    stage_rows<DT, D>(ks, k + (b * a.sk + k0) * D, valid);
    stage_rows<DT, D>(vs, v + (b * a.sk + k0) * D, valid);
    __syncthreads();
    for (int j = 0; j < valid; ++j) {
      float s = 0.0f, dp = 0.0f;
#pragma unroll
      for (int i = 0; i < D; ++i) {
        s += qr[i] * ks[j * D + i];
        dp += dor[i] * vs[j * D + i];
      }
      if (brow != nullptr) s += brow[k0 + j];
      const float p = __expf(s - L);
      const float dsb = p * (dp - dl);
      if (dbrow != nullptr) dbrow[k0 + j] = dsb;
      const float ds = dsb * a.scale;
#pragma unroll
      for (int i = 0; i < D; ++i) acc[i] += ds * ks[j * D + i];
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < D; ++i) dq[(b * a.sq + row) * D + i] = Elem<DT>::down(acc[i]);
  }
}

// --------------------------------------------------------- backward: dK, dV
template <int DT, int D>
__global__ __launch_bounds__(kRows) void attn_bwd_dkv_generic(
    typename Elem<DT>::T* __restrict__ dk, typename Elem<DT>::T* __restrict__ dv,
    const typename Elem<DT>::T* __restrict__ dout, const typename Elem<DT>::T* __restrict__ q,
    const typename Elem<DT>::T* __restrict__ k, const typename Elem<DT>::T* __restrict__ v,
    const float* __restrict__ lse, const float* __restrict__ delta, AttnArgs a) {
  __shared__ float qs[kTile * D];
  __shared__ float dos[kTile * D];
  __shared__ float ls[kTile];
  __shared__ float dls[kTile];
  const long long b = blockIdx.y;
  const int row = blockIdx.x * kRows + threadIdx.x;  // key row
  const bool live = row < a.sk;
  float kr[D], vr[D], gk[D], gv[D];
#pragma unroll
  for (int i = 0; i < D; ++i) {
    kr[i] = live ? Elem<DT>::up(k[(b * a.sk + row) * D + i]) : 0.0f;
    vr[i] = live ? Elem<DT>::up(v[(b * a.sk + row) * D + i]) : 0.0f;
    gk[i] = 0.0f;
    gv[i] = 0.0f;
  }
  const float* bcol =
      (a.bias != nullptr && live) ? a.bias + (b % a.bias_period) * (long long)a.sq * a.sk + row : nullptr;
  for (int q0 = 0; q0 < a.sq; q0 += kTile) {
    const int valid = min(kTile, a.sq - q0);
    __syncthreads();
    stage_rows<DT, D>(qs, q + (b * a.sq + q0) * D, valid);
    stage_rows<DT, D>(dos, dout + (b * a.sq + q0) * D, valid);
    if (threadIdx.x < kTile) {
      ls[threadIdx.x] = threadIdx.x < valid ? lse[b * a.sq + q0 + threadIdx.x] : 0.0f;
      dls[threadIdx.x] = threadIdx.x < valid ? delta[b * a.sq + q0 + threadIdx.x] : 0.0f;
    }
    __syncthreads();
    for (int j = 0; j < valid; ++j) {
      float s = 0.0f, dp = 0.0f;
#pragma unroll
      for (int i = 0; i < D; ++i) {
        s += qs[j * D + i] * kr[i];
        dp += dos[j * D + i] * vr[i];
      }
      s *= a.scale;
      if (bcol != nullptr) s += bcol[(long long)(q0 + j) * a.sk];
      const float p = __expf(s - ls[j]);
      const float ds = p * (dp - dls[j]) * a.scale;
#pragma unroll
      for (int i = 0; i < D; ++i) {
        gv[i] += p * dos[j * D + i];
        gk[i] += ds * qs[j * D + i];
      }
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < D; ++i) {
      dk[(b * a.sk + row) * D + i] = Elem<DT>::down(gk[i]);
      dv[(b * a.sk + row) * D + i] = Elem<DT>::down(gv[i]);
    }
  }
}

}  // namespace

namespace jg {

bool attn_generic_supported(int d) { return d == 8 || d == 16 || d == 32 || d == 64 || d == 96 || d == 128; }

#define JG_ATTN_DISPATCH(CALL)                                   \
  do {                                                           \
    switch (d) {                                                 \
      case 8: CALL(8); break;                                    \
      case 16: CALL(16); break;                                  \
      case 32: CALL(32); break;                                  \
      case 64: CALL(64); break;                                  \
      case 96: CALL(96); break;                                  \
      default: CALL(128); break;                                 \
    }                                                            \
  } while (0)

template <int DT>
static void fwd_t(void* out, float* lse, const void* q, const void* k, const void* v, AttnArgs a,
                  hipStream_t s) {
  typedef typename Elem<DT>::T T;
  const int d = a.d;
  dim3 grid((a.sq + kRows - 1) / kRows, (unsigned)a.batch, 1);
#define CALL(D)                                                                          \
  attn_fwd_generic<DT, D><<<grid, kRows, 0, s>>>(static_cast<T*>(out), lse,              \
                                                 static_cast<const T*>(q),               \
                                                 static_cast<const T*>(k),               \
                                                 static_cast<const T*>(v), a)
  JG_ATTN_DISPATCH(CALL);
#undef CALL
}

template <int DT>
static void bwd_t(void* dq, void* dk, void* dv, float* delta, float* dbias, const void* dout,
                  const void* q, const void* k, const void* v, const void* out, const float* lse,
                  AttnArgs a, hipStream_t s) {
  typedef typename Elem<DT>::T T;
  const int d = a.d;
  dim3 gq((a.sq + kRows - 1) / kRows, (unsigned)a.batch, 1);
  dim3 gk((a.sk + kRows - 1) / kRows, (unsigned)a.batch, 1);
#define CALL(D)                                                                               \
  do {                                                                                        \
    attn_bwd_dq_generic<DT, D><<<gq, kRows, 0, s>>>(                                          \
        static_cast<T*>(dq), delta, dbias, static_cast<const T*>(dout),                       \
        static_cast<const T*>(q), static_cast<const T*>(k), static_cast<const T*>(v),         \
        static_cast<const T*>(out), lse, a);                                                  \
    attn_bwd_dkv_generic<DT, D><<<gk, kRows, 0, s>>>(                                         \
        static_cast<T*>(dk), static_cast<T*>(dv), static_cast<const T*>(dout),                \
        static_cast<const T*>(q), static_cast<const T*>(k), static_cast<const T*>(v), lse,    \
        delta, a);                                                                            \
  } while (0)
  JG_ATTN_DISPATCH(CALL);
#undef CALL
}

int attn_generic_fwd(void* out, float* lse, const void* q, const void* k, const void* v,
                     long long batch, int sq, int sk, int d, float scale, const float* bias,
                     long long bias_period, int dtype, hipStream_t s) {
  JG_REQUIRE(batch <= 65535, "attention (generic): batch*heads = %lld exceeds 65535", batch);
  AttnArgs a{batch, sq, sk, d, scale, bias, bias_period > 0 ? bias_period : 1};
  if (dtype == JG_F32) fwd_t<JG_F32>(out, lse, q, k, v, a, s);
  else if (dtype == JG_BF16) fwd_t<JG_BF16>(out, lse, q, k, v, a, s);
  else fwd_t<JG_F16>(out, lse, q, k, v, a, s);
  JG_CHECK_LAUNCH("jg_attn_fwd(generic)");
  return JG_OK;
}

int attn_generic_bwd(void* dq, void* dk, void* dv, float* delta, float* dbias, const void* dout,
                     const void* q, const void* k, const void* v, const void* out,
                     const float* lse, long long batch, int sq, int sk, int d, float scale,
                     const float* bias, long long bias_period, int dtype, hipStream_t s) {
  JG_REQUIRE(batch <= 65535, "attention (generic): batch*heads = %lld exceeds 65535", batch);
  AttnArgs a{batch, sq, sk, d, scale, bias, bias_period > 0 ? bias_period : 1};
  if (dtype == JG_F32) bwd_t<JG_F32>(dq, dk, dv, delta, dbias, dout, q, k, v, out, lse, a, s);
  else if (dtype == JG_BF16) bwd_t<JG_BF16>(dq, dk, dv, delta, dbias, dout, q, k, v, out, lse, a, s);
  else bwd_t<JG_F16>(dq, dk, dv, delta, dbias, dout, q, k, v, out, lse, a, s);
  JG_CHECK_LAUNCH("jg_attn_bwd(generic)");
  return JG_OK;
}

}  // namespace jg
