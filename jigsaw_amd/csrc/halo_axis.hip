// Halo exchange along ONE split axis for need spans of any shape: spans that leave out rows the
// rank owns (stride 2 without padding on an odd tile) or reach ranks that are not adjacent (a
// kernel wider than the tile). This is the per-peer overlap loop of the reference as it stands:
//
//   gather        x_need = zeros(span); for peer: x_need[off : off + cnt] = rows of peer's tile
//                 jigsaw/modules/convolution/_conv/halo.py:112-114, 134-154
//   scatter-add   g_local = zeros(n); for peer = 0 .. G-1: g_local[off : off + cnt] += peer's part
//                 jigsaw/modules/convolution/_conv/halo.py:207, 217-249 (each add rounded to the dtype)
//
// A tensor is seen as (outer, rows, inner) around the axis. A segment names `count` rows of a
// source and where they land in the destination; the gather copies bytes (rows no segment covers
// are zero, later segments overwrite earlier ones, as successive copies would), the scatter-add
// visits the segments in the order given. One thread per 16-byte vector of the destination where
// rows are made of whole, aligned vectors, per element otherwise. Plain HBM-bound passes: the
// spans this serves are the unusual ones, the fused 8 / 26-strip kernels keep the common case.
#include "jg_common.h"

namespace {

constexpr int MAX_SEGS = JG_HALO_AXIS_MAX_SEGMENTS;

struct Segs {
  const void* src[MAX_SEGS];
  long long src_rows[MAX_SEGS], src_start[MAX_SEGS], dst_start[MAX_SEGS], count[MAX_SEGS];
  int n;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ T zero_of() { return T(0); }
template <>
__device__ __forceinline__ u32x4 zero_of<u32x4>() { return u32x4{0u, 0u, 0u, 0u}; }

// `inner` counts units of T
template <typename T>
__global__ __launch_bounds__(256) void axis_gather_kernel(T* __restrict__ dst, Segs segs, long long dst_rows,
                                                          long long inner, long long total) {
  for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long long)gridDim.x * 256) {
    const long long line = idx / inner, i = idx - line * inner;
    const long long o = line / dst_rows, r = line - o * dst_rows;
    // constant segment indices (the list is a kernel argument: no per-lane copy of it); the last
    // segment that covers the row wins
    const T* from = nullptr;
#pragma unroll
    for (int s = 0; s < MAX_SEGS; ++s) {
      const long long k = r - segs.dst_start[s];
      if (s < segs.n && k >= 0 && k < segs.count[s])
        from = static_cast<const T*>(segs.src[s]) + (o * segs.src_rows[s] + segs.src_start[s] + k) * inner + i;
    }
    dst[idx] = from != nullptr ? *from : zero_of<T>();
  }
}

template <int DT>
struct Num;
template <>
struct Num<JG_F32> {
  typedef float T;
  __device__ static __forceinline__ float up(float v) { return v; }
  __device__ static __forceinline__ float down(float v) { return v; }
};
template <>
struct Num<JG_BF16> {
  typedef uint16_t T;
  __device__ static __forceinline__ float up(uint16_t v) { return jg::bf16_to_f32(v); }
  __device__ static __forceinline__ uint16_t down(float v) { return jg::f32_to_bf16(v); }
};
template <>
struct Num<JG_F16> {
  typedef _Float16 T;
  __device__ static __forceinline__ float up(_Float16 v) { return (float)v; }
  __device__ static __forceinline__ _Float16 down(float v) { return (_Float16)v; }
};

// V elements per thread (V * sizeof(T) = 16 with vector accesses, V = 1 per element)
template <int DT, int V>
__global__ __launch_bounds__(256) void axis_scatter_add_kernel(typename Num<DT>::T* __restrict__ dst, Segs segs,
                                                               long long dst_rows, long long inner_v,
                                                               long long total_v) {
  typedef typename Num<DT>::T T;
  struct alignas(V * sizeof(T)) Pack { T v[V]; };
  for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < total_v; idx += (long long)gridDim.x * 256) {
    const long long line = idx / inner_v, i = idx - line * inner_v;
    const long long o = line / dst_rows, r = line - o * dst_rows;
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = 0.0f;
#pragma unroll
    for (int s = 0; s < MAX_SEGS; ++s) {  // constant indices into the kernel argument
      const long long k = r - segs.dst_start[s];
      if (s >= segs.n || k < 0 || k >= segs.count[s]) continue;
      const Pack in = reinterpret_cast<const Pack*>(segs.src[s])[(o * segs.src_rows[s] + segs.src_start[s] + k) * inner_v + i];
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = Num<DT>::up(Num<DT>::down(acc[e] + Num<DT>::up(in.v[e])));
    }
    Pack out;
#pragma unroll
    for (int e = 0; e < V; ++e) out.v[e] = Num<DT>::down(acc[e]);
    reinterpret_cast<Pack*>(dst)[idx] = out;
  }
}

int check_segments(const char* who, const jg_axis_segment* segs, int n_segs, int64_t dst_rows, Segs* out) {
  JG_REQUIRE(n_segs >= 0 && n_segs <= MAX_SEGS, "%s: %d segments, at most %d a call", who, n_segs, MAX_SEGS);
  JG_REQUIRE(n_segs == 0 || segs != nullptr, "%s: NULL segment list", who);
  *out = Segs{};
  for (int s = 0; s < n_segs; ++s) {
    const jg_axis_segment& g = segs[s];
    JG_REQUIRE(g.count >= 0 && g.src_start >= 0 && g.dst_start >= 0 && g.src_rows >= 0, "%s: segment %d has a negative field", who, s);
    if (g.count == 0) continue;
    JG_REQUIRE(g.src != nullptr, "%s: segment %d has no source", who, s);
    JG_REQUIRE(g.src_start + g.count <= g.src_rows, "%s: segment %d reads rows [%lld, %lld) of a source with %lld", who, s,
               (long long)g.src_start, (long long)(g.src_start + g.count), (long long)g.src_rows);
    JG_REQUIRE(g.dst_start + g.count <= dst_rows, "%s: segment %d writes rows [%lld, %lld) of a destination with %lld", who, s,
               (long long)g.dst_start, (long long)(g.dst_start + g.count), (long long)dst_rows);
    const int k = out->n++;
    out->src[k] = g.src;
    out->src_rows[k] = g.src_rows;
    out->src_start[k] = g.src_start;
    out->dst_start[k] = g.dst_start;
    out->count[k] = g.count;
  }
  return JG_OK;
}

bool all_aligned16(const void* dst, const Segs& s) {
  if ((reinterpret_cast<uintptr_t>(dst) & 15) != 0) return false;
  for (int k = 0; k < s.n; ++k)
    if ((reinterpret_cast<uintptr_t>(s.src[k]) & 15) != 0) return false;
  return true;
}

unsigned grid_for(long long total) {
  long long b = (total + 255) / 256;
  if (b > 65536) b = 65536;
  return (unsigned)(b < 1 ? 1 : b);
}

}  // namespace

extern "C" int jg_halo_axis_gather(void* dst, int64_t outer, int64_t dst_rows, int64_t inner,
                                   const jg_axis_segment* segs, int n_segs, int elem_size, void* stream) {
  const char* who = "jg_halo_axis_gather";
  JG_REQUIRE(outer >= 0 && dst_rows >= 0 && inner >= 0, "%s: bad shape", who);
  JG_REQUIRE(elem_size == 2 || elem_size == 4, "%s: elem_size %d not in {2, 4}", who, elem_size);
  Segs s;
  int rc = check_segments(who, segs, n_segs, dst_rows, &s);
  if (rc) return rc;
  const long long total = (long long)outer * dst_rows * inner;
  if (total == 0) return JG_OK;
  JG_REQUIRE(dst != nullptr, "%s: NULL destination", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const long long row_bytes = (long long)inner * elem_size;
  if (row_bytes % 16 == 0 && all_aligned16(dst, s)) {
    const long long tv = total * elem_size / 16;
    axis_gather_kernel<u32x4><<<grid_for(tv), 256, 0, st>>>(static_cast<u32x4*>(dst), s, dst_rows, row_bytes / 16, tv);
  } else if (elem_size == 4) {
    axis_gather_kernel<uint32_t><<<grid_for(total), 256, 0, st>>>(static_cast<uint32_t*>(dst), s, dst_rows, inner, total);
  } else {
    axis_gather_kernel<uint16_t><<<grid_for(total), 256, 0, st>>>(static_cast<uint16_t*>(dst), s, dst_rows, inner, total);
  }
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

extern "C" int jg_halo_axis_scatter_add(void* dst, int64_t outer, int64_t dst_rows, int64_t inner,
                                        const jg_axis_segment* segs, int n_segs, int dtype, void* stream) {
  const char* who = "jg_halo_axis_scatter_add";
  JG_REQUIRE(outer >= 0 && dst_rows >= 0 && inner >= 0, "%s: bad shape", who);
  JG_REQUIRE(dtype == JG_F32 || dtype == JG_BF16 || dtype == JG_F16, "%s: unknown dtype %d", who, dtype);
  Segs s;
  int rc = check_segments(who, segs, n_segs, dst_rows, &s);
  if (rc) return rc;
  const long long total = (long long)outer * dst_rows * inner;
  if (total == 0) return JG_OK;
  JG_REQUIRE(dst != nullptr, "%s: NULL destination", who);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int es = (int)jg::dtype_size(dtype);
  const bool vec = ((long long)inner * es) % 16 == 0 && all_aligned16(dst, s);
#define JG_GO(DT)                                                                                                   \
  if (vec)                                                                                                          \
    axis_scatter_add_kernel<DT, 16 / sizeof(Num<DT>::T)><<<grid_for(total * es / 16), 256, 0, st>>>(                \
        static_cast<Num<DT>::T*>(dst), s, dst_rows, (long long)inner * es / 16, total * es / 16);                   \
  else                                                                                                              \
    axis_scatter_add_kernel<DT, 1><<<grid_for(total), 256, 0, st>>>(static_cast<Num<DT>::T*>(dst), s, dst_rows, inner, total)
  if (dtype == JG_F32) JG_GO(JG_F32);
  else if (dtype == JG_BF16) JG_GO(JG_BF16);
  else JG_GO(JG_F16);
#undef JG_GO
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}
