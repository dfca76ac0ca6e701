// DistributedRoll: the local cyclic roll and the wrapped-slab pack / unpack.
// Pure copies, destination-driven, 16-byte vectors whenever the run of
// unrolled trailing axes allows it.
//
// Reference behaviour restated here:
//   jigsaw/modules/roll/_distributed_roll.py:99     (torch.roll of the tile)
//   jigsaw/modules/roll/_distributed_roll.py:44-59  (slab cut and write-back)
#include "jg_common.h"

namespace {

constexpr int kMaxDims = 6;

struct RollArgs {
  int nd;                      // axes after collapsing
  long long size[kMaxDims];    // extent in units of the copy word
  long long shift[kMaxDims];   // normalised to [0, size)
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
__global__ __launch_bounds__(256) void roll_kernel(T* __restrict__ dst,
                                                   const T* __restrict__ src, RollArgs a,
                                                   long long total) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (long long)gridDim.x * 256) {
    long long rem = i, so = 0, stride = 1;
#pragma unroll
    for (int k = kMaxDims - 1; k >= 0; --k) {
      if (k < a.nd) {
        long long q = rem / a.size[k];
        long long c = rem - q * a.size[k];
        rem = q;
        long long sc = c - a.shift[k];
        if (sc < 0) sc += a.size[k];
        so += sc * stride;
        stride *= a.size[k];
      }
    }
    dst[i] = src[so];
  }
}

// Slab copy between x viewed as (outer, len, inner) and a dense (outer, win, inner).
template <typename T, bool PACK>
__global__ __launch_bounds__(256) void slab_kernel(T* __restrict__ x_or_strip_dst,
                                                   const T* __restrict__ src, long long outer,
                                                   long long len, long long inner,
                                                   long long start, long long win) {
  const long long total = outer * win * inner;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (long long)gridDim.x * 256) {
    long long r = i / inner;
    long long ci = i - r * inner;
    long long o = r / win;
    long long a = r - o * win;
    long long xo = (o * len + start + a) * inner + ci;
    if (PACK)
      x_or_strip_dst[i] = src[xo];
    else
      x_or_strip_dst[xo] = src[i];
  }
}

int grid_for(long long n) {
  long long b = (n + 255) / 256;
  if (b > (1 << 20)) b = 1 << 20;
  if (b < 1) b = 1;
  return (int)b;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int slab_common(void* dst, const void* src, const void* x, int ndim, const int64_t* sizes,
                int axis, int64_t window, int elem_size, void* stream, bool pack,
                const char* who) {
  JG_REQUIRE(dst != nullptr && src != nullptr && sizes != nullptr, "%s: NULL pointer", who);
  JG_REQUIRE(ndim >= 1 && ndim <= 8, "%s: ndim %d out of range", who, ndim);
  JG_REQUIRE(axis >= 0 && axis < ndim, "%s: axis %d out of range", who, axis);
  JG_REQUIRE(elem_size == 2 || elem_size == 4, "%s: elem_size %d not in {2, 4}", who,
             elem_size);
  long long outer = 1, inner = 1;
  for (int i = 0; i < ndim; ++i) {
    JG_REQUIRE(sizes[i] >= 0, "%s: negative size", who);
    if (i < axis) outer *= sizes[i];
    if (i > axis) inner *= sizes[i];
  }
  const long long len = sizes[axis];
  const long long win = window < 0 ? -window : window;
  JG_REQUIRE(win <= len, "%s: |window| = %lld exceeds the local size %lld", who, win, len);
  const long long start = window > 0 ? 0 : len - win;
  if (outer * win * inner == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long long inner_bytes = inner * elem_size;
  const void* strip = pack ? dst : src;
  if (inner_bytes % 16 == 0 && aligned16(x) && aligned16(strip)) {
    const long long iv = inner_bytes / 16;
    const long long total = outer * win * iv;
    if (pack)
      slab_kernel<u32x4, true><<<grid_for(total), 256, 0, s>>>(
          static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), outer, len, iv, start, win);
    else
      slab_kernel<u32x4, false><<<grid_for(total), 256, 0, s>>>(
          static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), outer, len, iv, start, win);
  } else {
    const long long total = outer * win * inner;
#define JG_SLAB(T)                                                                         \
  do {                                                                                     \
    if (pack)                                                                              \
      slab_kernel<T, true><<<grid_for(total), 256, 0, s>>>(                                \
          static_cast<T*>(dst), static_cast<const T*>(src), outer, len, inner, start, win); \
    else                                                                                   \
      slab_kernel<T, false><<<grid_for(total), 256, 0, s>>>(                               \
          static_cast<T*>(dst), static_cast<const T*>(src), outer, len, inner, start, win); \
  } while (0)
    if (elem_size == 2) JG_SLAB(uint16_t);
    else JG_SLAB(uint32_t);
#undef JG_SLAB
  }
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

}  // namespace

extern "C" int jg_roll(void* dst, const void* src, int ndim, const int64_t* sizes,
                       const int64_t* shifts, int elem_size, void* stream) {
  JG_REQUIRE(dst != nullptr && src != nullptr && sizes != nullptr && shifts != nullptr,
             "jg_roll: NULL pointer");
  JG_REQUIRE(dst != src, "jg_roll: dst must not alias src");
  JG_REQUIRE(ndim >= 1 && ndim <= kMaxDims, "jg_roll: ndim %d not in [1, %d]", ndim, kMaxDims);
  JG_REQUIRE(elem_size == 2 || elem_size == 4, "jg_roll: elem_size %d not in {2, 4}",
             elem_size);
  long long total = 1;
  for (int i = 0; i < ndim; ++i) {
    JG_REQUIRE(sizes[i] >= 0, "jg_roll: negative size");
    total *= sizes[i];
  }
  if (total == 0) return JG_OK;
  // Normalise the shifts, then merge the trailing axes that are not rolled into
  // one contiguous run, copied in the widest word that divides it.
  long long sz[kMaxDims], sh[kMaxDims];
  for (int i = 0; i < ndim; ++i) {
    sz[i] = sizes[i];
    long long m = shifts[i] % sizes[i];
    if (m < 0) m += sizes[i];
    sh[i] = m;
  }
  int last = ndim;  // axes [last, ndim) are unrolled
  while (last > 0 && sh[last - 1] == 0) --last;
  long long run = 1;
  for (int i = last; i < ndim; ++i) run *= sz[i];
  RollArgs a;
  a.nd = 0;
  // Also merge neighbouring unrolled leading axes (cheap, fewer divisions).
  for (int i = 0; i < last; ++i) {
    if (a.nd > 0 && sh[i] == 0 && a.shift[a.nd - 1] == 0) {
      a.size[a.nd - 1] *= sz[i];
    } else {
      a.size[a.nd] = sz[i];
      a.shift[a.nd] = sh[i];
      ++a.nd;
    }
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long long run_bytes = run * elem_size;
  if (run_bytes % 16 == 0 && aligned16(dst) && aligned16(src)) {
    a.size[a.nd] = run_bytes / 16;
    a.shift[a.nd] = 0;
    ++a.nd;
    const long long n = total * elem_size / 16;
    roll_kernel<u32x4><<<grid_for(n), 256, 0, s>>>(static_cast<u32x4*>(dst),
                                                   static_cast<const u32x4*>(src), a, n);
  } else {
    if (run > 1 || a.nd == 0) {
      a.size[a.nd] = run;
      a.shift[a.nd] = 0;
      ++a.nd;
    }
    if (elem_size == 2)
      roll_kernel<uint16_t><<<grid_for(total), 256, 0, s>>>(
          static_cast<uint16_t*>(dst), static_cast<const uint16_t*>(src), a, total);
    else
      roll_kernel<uint32_t><<<grid_for(total), 256, 0, s>>>(
          static_cast<uint32_t*>(dst), static_cast<const uint32_t*>(src), a, total);
  }
  JG_CHECK_LAUNCH("jg_roll");
  return JG_OK;
}

extern "C" int jg_roll_pack(void* strip, const void* x, int ndim, const int64_t* sizes,
                            int axis, int64_t window, int elem_size, void* stream) {
  return slab_common(strip, x, x, ndim, sizes, axis, window, elem_size, stream, true,
                     "jg_roll_pack");
}

extern "C" int jg_roll_unpack(void* x, const void* strip, int ndim, const int64_t* sizes,
                              int axis, int64_t window, int elem_size, void* stream) {
  return slab_common(x, strip, x, ndim, sizes, axis, window, elem_size, stream, false,
                     "jg_roll_unpack");
}
