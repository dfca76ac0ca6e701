// Online-softmax / log-sum-exp merge of two partial attention results.
// One thread owns 4 consecutive head-dim elements of one row; the row's two
// log-sum-exp values are read once per thread (they hit in cache across the
// d/4 threads of a row). HBM-bound: reads o1, o2, writes o1.
//
// Reference behaviour restated here:
//   jigsaw/modules/attention/_functional/_merge_kernel.py:37-82
//   jigsaw/modules/attention/_functional/forward.py:23-61
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

template <int D1, int D2, int V>
__global__ __launch_bounds__(256) void merge_kernel(typename Elem<D1>::T* __restrict__ o1,
                                                    const float* l1,
                                                    const typename Elem<D2>::T* __restrict__ o2,
                                                    const float* __restrict__ l2, float* l_new,
                                                    long long n_rows, long long N, long long H,
                                                    int d, bool bshd) {
  typedef typename Elem<D1>::T T1;
  typedef typename Elem<D2>::T T2;
  const int per_row = d / V;
  const long long total = n_rows * per_row;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (long long)gridDim.x * 256) {
    const long long row = i / per_row;
    const int c = (int)(i - row * per_row) * V;
    long long l_off = row;
    if (bshd) {
      // o rows run (b, n, h); the log-sum-exp is (b, h, n)
      long long b = row / (N * H);
      long long rem = row - b * N * H;
      long long n = rem / H;
      long long h = rem - n * H;
      l_off = (b * H + h) * N + n;
    }
    const float a = l1[l_off];
    const float b2 = l2[l_off];
    const float w = 1.0f / (1.0f + __expf(a - b2));  // sigmoid(l2 - l1)
    struct alignas(sizeof(T1) * V) P1 { T1 v[V]; };
    struct alignas(sizeof(T2) * V) P2 { T2 v[V]; };
    P1 x = *reinterpret_cast<const P1*>(o1 + row * d + c);
    const P2 y = *reinterpret_cast<const P2*>(o2 + row * d + c);
#pragma unroll
    for (int k = 0; k < V; ++k) {
      const float xa = Elem<D1>::up(x.v[k]);
      const float yb = Elem<D2>::up(y.v[k]);
      x.v[k] = Elem<D1>::down(xa + w * (yb - xa));
    }
    *reinterpret_cast<P1*>(o1 + row * d + c) = x;
    if (c == 0) {
      const float mx = fmaxf(a, b2);
      l_new[l_off] = mx + log1pf(__expf(-fabsf(a - b2)));
    }
  }
}

template <int D1, int D2>
int launch(void* o1, const float* l1, const void* o2, const float* l2, float* l_new,
           long long rows, long long N, long long H, int d, bool bshd, hipStream_t s) {
  typedef typename Elem<D1>::T T1;
  typedef typename Elem<D2>::T T2;
  const bool v4 = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(o1) % (4 * sizeof(T1)) == 0) &&
                  (reinterpret_cast<uintptr_t>(o2) % (4 * sizeof(T2)) == 0);
  const long long total = rows * (v4 ? d / 4 : d);
  long long blocks = (total + 255) / 256;
  if (blocks > (1 << 20)) blocks = 1 << 20;
  if (v4)
    merge_kernel<D1, D2, 4><<<(int)blocks, 256, 0, s>>>(static_cast<T1*>(o1), l1,
                                                        static_cast<const T2*>(o2), l2, l_new,
                                                        rows, N, H, d, bshd);
  else
    merge_kernel<D1, D2, 1><<<(int)blocks, 256, 0, s>>>(static_cast<T1*>(o1), l1,
                                                        static_cast<const T2*>(o2), l2, l_new,
                                                        rows, N, H, d, bshd);
  return JG_OK;
}

}  // namespace

extern "C" int jg_lse_merge(void* o1, const float* l1, const void* o2, const float* l2,
                            float* l_new, int64_t b, int64_t h, int64_t n, int64_t d, int bshd,
                            int o1_dtype, int o2_dtype, void* stream) {
  JG_REQUIRE(o1 && l1 && o2 && l2 && l_new, "jg_lse_merge: NULL pointer");
  JG_REQUIRE(b >= 0 && h >= 0 && n >= 0 && d >= 1 && d <= (1 << 20), "jg_lse_merge: bad shape");
  const long long rows = (long long)b * h * n;
  if (rows == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define JG_GO(A, B) launch<A, B>(o1, l1, o2, l2, l_new, rows, n, h, (int)d, bshd != 0, s)
  if (o1_dtype == JG_F32 && o2_dtype == JG_F32) JG_GO(JG_F32, JG_F32);
  else if (o1_dtype == JG_F32 && o2_dtype == JG_BF16) JG_GO(JG_F32, JG_BF16);
  else if (o1_dtype == JG_F32 && o2_dtype == JG_F16) JG_GO(JG_F32, JG_F16);
  else if (o1_dtype == JG_BF16 && o2_dtype == JG_BF16) JG_GO(JG_BF16, JG_BF16);
  else if (o1_dtype == JG_F16 && o2_dtype == JG_F16) JG_GO(JG_F16, JG_F16);
  else
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_lse_merge: dtype pair (%d, %d) not supported", o1_dtype,
            o2_dtype);
#undef JG_GO
  JG_CHECK_LAUNCH("jg_lse_merge");
  return JG_OK;
}
