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

// I: the index arithmetic's type, int where the word count allows it: a 64-bit division is some
// hundred instructions, and with one per axis and word they, not the memory, set the kernel's time.
template <typename I>
__device__ __forceinline__ I rolled_source(const RollArgs& a, I i) {
  I rem = i, so = 0, stride = 1;
#pragma unroll
  for (int k = kMaxDims - 1; k >= 0; --k) {
    if (k < a.nd) {
      const I size = (I)a.size[k];
      const I q = rem / size;
      const I c = rem - q * size;
      rem = q;
      I sc = c - (I)a.shift[k];
      if (sc < 0) sc += size;
      so += sc * stride;
      stride *= size;
    }
  }
  return so;
}

template <typename T, typename I>
__global__ __launch_bounds__(256) void roll_kernel(T* __restrict__ dst,
                                                   const T* __restrict__ src, RollArgs a,
                                                   long long total) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (long long)gridDim.x * 256)
    dst[i] = src[rolled_source<I>(a, (I)i)];
}

// Slab copy between x viewed as (outer, len, inner) and a dense (outer, win, inner).
template <typename T, bool PACK, typename I>
__global__ __launch_bounds__(256) void slab_kernel(T* __restrict__ x_or_strip_dst,
                                                   const T* __restrict__ src, long long outer,
                                                   long long len_, long long inner_,
                                                   long long start_, long long win_) {
  const long long total = outer * win_ * inner_;
  const I len = (I)len_, inner = (I)inner_, start = (I)start_, win = (I)win_;
  for (long long i_ = (long long)blockIdx.x * 256 + threadIdx.x; i_ < total;
       i_ += (long long)gridDim.x * 256) {
    const I i = (I)i_;
    I r = i / inner;
    I ci = i - r * inner;
    I o = r / win;
    I a = r - o * win;
    I xo = (o * len + start + a) * inner + ci;
    if (PACK)
      x_or_strip_dst[i] = src[xo];
    else
      x_or_strip_dst[xo] = src[i];
  }
}

// x viewed as (outer, len, inner) along one axis; the slab is rows [start, start + win) of it.
struct SlabView {
  long long len, inner, start, win;
  template <typename I>
  __device__ __forceinline__ bool holds(I idx, I* strip_idx) const {
    const I inner_ = (I)inner, len_ = (I)len, start_ = (I)start, win_ = (I)win;
    const I r = idx / inner_, ci = idx - r * inner_;
    const I o = r / len_, l = r - o * len_;
    *strip_idx = (o * win_ + (l - start_)) * inner_ + ci;
    return l >= start_ && l < start_ + win_;
  }
  template <typename I>
  __device__ __forceinline__ I place(I strip_idx) const {
    const I inner_ = (I)inner, len_ = (I)len, start_ = (I)start, win_ = (I)win;
    const I r = strip_idx / inner_, ci = strip_idx - r * inner_;
    const I o = r / win_, a = r - o * win_;
    return (o * len_ + start_ + a) * inner_ + ci;
  }
};

// The local roll, and on the way the wrapped slab of the ROLLED tensor along one axis cut into
// `strip`, with the buffer the neighbour's slab will be received in cleared (what the reference
// does in three passes: torch.roll, x[sl].contiguous(), torch.zeros_like).
template <typename T, typename I>
__global__ __launch_bounds__(256) void roll_pack_kernel(T* __restrict__ dst, const T* __restrict__ src, RollArgs a,
                                                        long long total, T* __restrict__ strip, T* __restrict__ clear,
                                                        SlabView v) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
    const T val = src[rolled_source<I>(a, (I)i)];
    dst[i] = val;
    I j;
    if (v.holds<I>((I)i, &j)) {
      strip[j] = val;
      if (clear != nullptr) clear[j] = T{};
    }
  }
}

// Between two exchanges: the slab received along the first axis goes into x, and the slab to
// send along the second axis is cut from x as it will be AFTER that write: where the two slabs
// cross, the cut takes the received values directly, so the two steps do not wait for each other.
// The buffer for the second exchange is cleared on the way.
template <typename T, typename I>
__global__ __launch_bounds__(256) void unpack_pack_kernel(T* __restrict__ x, const T* __restrict__ recv1, SlabView v1,
                                                          long long n1, T* __restrict__ strip2, T* __restrict__ clear2,
                                                          SlabView v2, long long n2) {
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n1 + n2; i += (long long)gridDim.x * 256) {
    if (i < n1) {
      x[v1.place<I>((I)i)] = recv1[i];
    } else {
      const I j = (I)(i - n1);
      const I idx = v2.place<I>(j);
      I j1;
      strip2[j] = v1.holds<I>(idx, &j1) ? recv1[j1] : x[idx];
      if (clear2 != nullptr) clear2[j] = T{};
    }
  }
}

int grid_for(long long n) {
  long long b = (n + 255) / 256;
  if (b > (1 << 20)) b = 1 << 20;
  if (b < 1) b = 1;
  return (int)b;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
// whether every index of a tensor of `words` copy words fits the 32-bit arithmetic
bool small(long long words) { return words < (1ll << 30); }

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
    const bool i32 = small(outer * len * iv);
    if (pack && i32)
      slab_kernel<u32x4, true, int><<<grid_for(total), 256, 0, s>>>(
          static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), outer, len, iv, start, win);
    else if (pack)
      slab_kernel<u32x4, true, long long><<<grid_for(total), 256, 0, s>>>(
          static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), outer, len, iv, start, win);
    else if (i32)
      slab_kernel<u32x4, false, int><<<grid_for(total), 256, 0, s>>>(
          static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), outer, len, iv, start, win);
    else
      slab_kernel<u32x4, false, long long><<<grid_for(total), 256, 0, s>>>(
          static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), outer, len, iv, start, win);
  } else {
    const long long total = outer * win * inner;
#define JG_SLAB(T)                                                                         \
  do {                                                                                     \
    if (pack)                                                                              \
      slab_kernel<T, true, long long><<<grid_for(total), 256, 0, s>>>(                     \
          static_cast<T*>(dst), static_cast<const T*>(src), outer, len, inner, start, win); \
    else                                                                                   \
      slab_kernel<T, false, long long><<<grid_for(total), 256, 0, s>>>(                    \
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
    if (small(n))
      roll_kernel<u32x4, int><<<grid_for(n), 256, 0, s>>>(static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), a, n);
    else
      roll_kernel<u32x4, long long><<<grid_for(n), 256, 0, s>>>(static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), a, n);
  } else {
    if (run > 1 || a.nd == 0) {
      a.size[a.nd] = run;
      a.shift[a.nd] = 0;
      ++a.nd;
    }
    if (elem_size == 2)
      roll_kernel<uint16_t, long long><<<grid_for(total), 256, 0, s>>>(
          static_cast<uint16_t*>(dst), static_cast<const uint16_t*>(src), a, total);
    else
      roll_kernel<uint32_t, long long><<<grid_for(total), 256, 0, s>>>(
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


namespace {
struct Axis {
  long long outer, len, inner, start, win;
};
int axis_view(Axis* v, int ndim, const int64_t* sizes, int axis, int64_t window, const char* who) {
  JG_REQUIRE(axis >= 0 && axis < ndim, "%s: axis %d out of range", who, axis);
  v->outer = v->inner = 1;
  for (int i = 0; i < ndim; ++i) {
    JG_REQUIRE(sizes[i] >= 0, "%s: negative size", who);
    if (i < axis) v->outer *= sizes[i];
    if (i > axis) v->inner *= sizes[i];
  }
  v->len = sizes[axis];
  v->win = window < 0 ? -window : window;
  JG_REQUIRE(v->win <= v->len, "%s: |window| = %lld exceeds the local size %lld", who, v->win, v->len);
  v->start = window > 0 ? 0 : v->len - v->win;
  return JG_OK;
}
}  // namespace

// jg_roll, jg_roll_pack of the rolled tensor along `axis` and the clearing of the receive buffer in
// one pass (_distributed_roll.py:99 followed by 44-49 of the first exchange). 16-byte runs only:
// the trailing axes that are not rolled (and lie behind `axis`) must make up a multiple of 16 bytes.
extern "C" int jg_roll_pack_fused(void* dst, void* strip, void* clear, const void* src, int ndim, const int64_t* sizes,
                                  const int64_t* shifts, int axis, int64_t window, int elem_size, void* stream) {
  const char* who = "jg_roll_pack_fused";
  JG_REQUIRE(dst && strip && src && sizes && shifts, "%s: NULL pointer", who);
  JG_REQUIRE(dst != src, "%s: dst must not alias src", who);
  JG_REQUIRE(ndim >= 1 && ndim <= kMaxDims, "%s: ndim %d not in [1, %d]", who, ndim, kMaxDims);
  JG_REQUIRE(elem_size == 2 || elem_size == 4, "%s: elem_size %d not in {2, 4}", who, elem_size);
  Axis ax;
  int rc = axis_view(&ax, ndim, sizes, axis, window, who);
  if (rc) return rc;
  long long total = 1;
  for (int i = 0; i < ndim; ++i) total *= sizes[i];
  if (total == 0) return JG_OK;
  int last = ndim;  // axes [last, ndim) are not rolled
  while (last > 0 && (shifts[last - 1] % sizes[last - 1]) == 0) --last;
  if (last <= axis) last = axis + 1;  // the slab axis keeps an index of its own
  long long run = 1;
  for (int i = last; i < ndim; ++i) run *= sizes[i];
  const long long run_bytes = run * elem_size;
  if (run_bytes % 16 != 0 || !aligned16(dst) || !aligned16(src) || !aligned16(strip) || (clear && !aligned16(clear)))
    JG_FAIL(JG_ERR_UNSUPPORTED, "%s: needs 16-byte aligned tensors whose unrolled trailing axes span a multiple of 16 bytes", who);
  JG_REQUIRE(last + 1 <= kMaxDims, "%s: too many rolled axes", who);
  RollArgs a;
  a.nd = 0;
  for (int i = 0; i < last; ++i) {
    long long m = shifts[i] % sizes[i];
    if (m < 0) m += sizes[i];
    a.size[a.nd] = sizes[i];
    a.shift[a.nd] = m;
    ++a.nd;
  }
  const long long words = run_bytes / 16;
  a.size[a.nd] = words;
  a.shift[a.nd] = 0;
  ++a.nd;
  // the slab view in 16-byte words: inner = (axes between `axis` and `last`) * words
  SlabView v;
  v.len = ax.len; v.start = ax.start; v.win = ax.win;
  v.inner = ax.inner / run * words;
  const long long n = total / run * words;
  if (small(n))
    roll_pack_kernel<u32x4, int><<<grid_for(n), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), a, n, static_cast<u32x4*>(strip),
        static_cast<u32x4*>(clear), v);
  else
    roll_pack_kernel<u32x4, long long><<<grid_for(n), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<u32x4*>(dst), static_cast<const u32x4*>(src), a, n, static_cast<u32x4*>(strip),
        static_cast<u32x4*>(clear), v);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

// jg_roll_unpack of the slab received along axis1 and jg_roll_pack of the slab to send along axis2
// (with its receive buffer cleared) in one pass (_distributed_roll.py:59 of one exchange, 44-49 of
// the next). The innermost axis must span a multiple of 16 bytes and lie behind both axes.
extern "C" int jg_roll_unpack_pack(void* x, const void* recv1, int axis1, int64_t window1, void* strip2, void* clear2,
                                   int axis2, int64_t window2, int ndim, const int64_t* sizes, int elem_size,
                                   void* stream) {
  const char* who = "jg_roll_unpack_pack";
  JG_REQUIRE(x && recv1 && strip2 && sizes, "%s: NULL pointer", who);
  JG_REQUIRE(ndim >= 1 && ndim <= 8, "%s: ndim %d out of range", who, ndim);
  JG_REQUIRE(elem_size == 2 || elem_size == 4, "%s: elem_size %d not in {2, 4}", who, elem_size);
  JG_REQUIRE(axis1 != axis2, "%s: the two axes must differ", who);
  Axis a1, a2;
  int rc = axis_view(&a1, ndim, sizes, axis1, window1, who);
  if (rc) return rc;
  rc = axis_view(&a2, ndim, sizes, axis2, window2, who);
  if (rc) return rc;
  const int deeper = axis1 > axis2 ? axis1 : axis2;
  long long run = 1;
  for (int i = deeper + 1; i < ndim; ++i) run *= sizes[i];
  const long long run_bytes = run * elem_size;
  if (run_bytes % 16 != 0 || !aligned16(x) || !aligned16(recv1) || !aligned16(strip2) || (clear2 && !aligned16(clear2)))
    JG_FAIL(JG_ERR_UNSUPPORTED, "%s: needs 16-byte aligned tensors whose axes behind both slab axes span a multiple of 16 bytes", who);
  const long long words = run_bytes / 16;
  SlabView v1, v2;
  v1.len = a1.len; v1.start = a1.start; v1.win = a1.win; v1.inner = a1.inner / run * words;
  v2.len = a2.len; v2.start = a2.start; v2.win = a2.win; v2.inner = a2.inner / run * words;
  const long long n1 = a1.outer * a1.win * v1.inner, n2 = a2.outer * a2.win * v2.inner;
  if (n1 + n2 == 0) return JG_OK;
  // indices run over x (in words), the largest of the three tensors
  if (small(a1.outer * a1.len * v1.inner))
    unpack_pack_kernel<u32x4, int><<<grid_for(n1 + n2), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<u32x4*>(x), static_cast<const u32x4*>(recv1), v1, n1, static_cast<u32x4*>(strip2),
        static_cast<u32x4*>(clear2), v2, n2);
  else
    unpack_pack_kernel<u32x4, long long><<<grid_for(n1 + n2), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<u32x4*>(x), static_cast<const u32x4*>(recv1), v1, n1, static_cast<u32x4*>(strip2),
        static_cast<u32x4*>(clear2), v2, n2);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}
