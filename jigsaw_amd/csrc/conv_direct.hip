// Direct (FMA, fp32-accumulate) convolution kernels for any 1-D / 2-D / 3-D
// geometry: forward, input gradient, weight gradient and bias gradient. They
// cover every shape the implicit-GEMM MFMA kernels do not (few channels, fp32
// tensors, strides, dilations) and are the path of the fp32 configuration.
// Layouts: x (N, Cin, D, H, W), w (Cout, Cin, kd, kh, kw), y (N, Cout, Do, Ho, Wo).
//
// Reference operators these stand in for (table at
// jigsaw/modules/convolution/_conv/config.py:27-29): F.conv{1,2,3}d,
// torch.nn.grad.conv{1,2,3}d_input, conv{1,2,3}d_weight, and the bias sum of
// config.py:117-120.
#include "conv_common.h"

namespace {

using jg::ConvGeom;

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

constexpr int kCB = 8;  // output channels (fwd) / input channels (dgrad) per thread

// -------------------------------------------------------------------- forward
template <int DT>
__global__ __launch_bounds__(256) void direct_fwd_kernel(typename Elem<DT>::T* __restrict__ y,
                                                         const typename Elem<DT>::T* __restrict__ x,
                                                         const typename Elem<DT>::T* __restrict__ w,
                                                         const typename Elem<DT>::T* __restrict__ bias,
                                                         ConvGeom g) {
  const long long so = (long long)g.out[0] * g.out[1] * g.out[2];
  const long long si = (long long)g.in[0] * g.in[1] * g.in[2];
  const int taps = g.k[0] * g.k[1] * g.k[2];
  const long long sp = (long long)blockIdx.x * 256 + threadIdx.x;
  // blockIdx.y = (group, block of kCB of the group's output channels)
  const int cin_g = g.cin / g.groups, cout_g = g.cout / g.groups;
  const int blocks_g = (cout_g + kCB - 1) / kCB;
  const int grp = blockIdx.y / blocks_g;
  const int co0 = grp * cout_g + (blockIdx.y - grp * blocks_g) * kCB, co_end = (grp + 1) * cout_g;
  const long long n = blockIdx.z;
  if (sp >= so) return;
  const int ow = (int)(sp % g.out[2]);
  const long long t = sp / g.out[2];
  const int oh = (int)(t % g.out[1]);
  const int od = (int)(t / g.out[1]);
  float acc[kCB];
#pragma unroll
  for (int j = 0; j < kCB; ++j)
    acc[j] = (bias != nullptr && co0 + j < co_end) ? Elem<DT>::up(bias[co0 + j]) : 0.0f;
  const typename Elem<DT>::T* xn = x + (n * g.cin + (long long)grp * cin_g) * si;
  for (int ci = 0; ci < cin_g; ++ci) {
    for (int kd = 0; kd < g.k[0]; ++kd) {
      const int id = od * g.s[0] - g.p[0] + kd * g.d[0];
      if (id < 0 || id >= g.in[0]) continue;
      for (int kh = 0; kh < g.k[1]; ++kh) {
        const int ih = oh * g.s[1] - g.p[1] + kh * g.d[1];
        if (ih < 0 || ih >= g.in[1]) continue;
        for (int kw = 0; kw < g.k[2]; ++kw) {
          const int iw = ow * g.s[2] - g.p[2] + kw * g.d[2];
          if (iw < 0 || iw >= g.in[2]) continue;
          const float xv =
              Elem<DT>::up(xn[ci * si + ((long long)id * g.in[1] + ih) * g.in[2] + iw]);
          const int tap = (kd * g.k[1] + kh) * g.k[2] + kw;
#pragma unroll
          for (int j = 0; j < kCB; ++j) {
            if (co0 + j < co_end)
              acc[j] += xv * Elem<DT>::up(w[((long long)(co0 + j) * cin_g + ci) * taps + tap]);
          }
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < kCB; ++j)
    if (co0 + j < co_end) y[(n * g.cout + co0 + j) * so + sp] = Elem<DT>::down(acc[j]);
}

// --------------------------------------------------------------------- dgrad
template <int DT>
__global__ __launch_bounds__(256) void direct_dgrad_kernel(
    typename Elem<DT>::T* __restrict__ gx, const typename Elem<DT>::T* __restrict__ w,
    const typename Elem<DT>::T* __restrict__ go, ConvGeom g) {
  const long long so = (long long)g.out[0] * g.out[1] * g.out[2];
  const long long si = (long long)g.in[0] * g.in[1] * g.in[2];
  const int taps = g.k[0] * g.k[1] * g.k[2];
  const long long sp = (long long)blockIdx.x * 256 + threadIdx.x;
  // blockIdx.y = (group, block of kCB of the group's input channels)
  const int cin_g = g.cin / g.groups, cout_g = g.cout / g.groups;
  const int blocks_g = (cin_g + kCB - 1) / kCB;
  const int grp = blockIdx.y / blocks_g;
  const int cl0 = (blockIdx.y - grp * blocks_g) * kCB;  // first channel of the block inside its group
  const int ci0 = grp * cin_g + cl0;
  const long long n = blockIdx.z;
  if (sp >= si) return;
  const int iw = (int)(sp % g.in[2]);
  const long long t = sp / g.in[2];
  const int ih = (int)(t % g.in[1]);
  const int id = (int)(t / g.in[1]);
  float acc[kCB];
#pragma unroll
  for (int j = 0; j < kCB; ++j) acc[j] = 0.0f;
  const typename Elem<DT>::T* gn = go + (n * g.cout + (long long)grp * cout_g) * so;
  for (int kd = 0; kd < g.k[0]; ++kd) {
    const int td = id + g.p[0] - kd * g.d[0];
    if (td < 0 || td % g.s[0]) continue;
    const int od = td / g.s[0];
    if (od >= g.out[0]) continue;
    for (int kh = 0; kh < g.k[1]; ++kh) {
      const int th = ih + g.p[1] - kh * g.d[1];
      if (th < 0 || th % g.s[1]) continue;
      const int oh = th / g.s[1];
      if (oh >= g.out[1]) continue;
      for (int kw = 0; kw < g.k[2]; ++kw) {
        const int tw = iw + g.p[2] - kw * g.d[2];
        if (tw < 0 || tw % g.s[2]) continue;
        const int ow = tw / g.s[2];
        if (ow >= g.out[2]) continue;
        const int tap = (kd * g.k[1] + kh) * g.k[2] + kw;
        const long long po = ((long long)od * g.out[1] + oh) * g.out[2] + ow;
        for (int co = 0; co < cout_g; ++co) {
          const float gv = Elem<DT>::up(gn[co * so + po]);
#pragma unroll
          for (int j = 0; j < kCB; ++j)
            if (cl0 + j < cin_g)
              acc[j] += gv * Elem<DT>::up(w[((long long)(grp * cout_g + co) * cin_g + cl0 + j) * taps + tap]);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < kCB; ++j)
    if (cl0 + j < cin_g) gx[(n * g.cin + ci0 + j) * si + sp] = Elem<DT>::down(acc[j]);
}

// --------------------------------------------------------------------- wgrad
__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// Stage 1: block (chunk, ci inside the group of co, co) reduces its share of the N*Do*Ho*Wo
// domain for every tap; part[chunk][co][ci in group][tap].
template <int DT>
__global__ __launch_bounds__(256) void direct_wgrad_kernel(float* __restrict__ part,
                                                           const typename Elem<DT>::T* __restrict__ x,
                                                           const typename Elem<DT>::T* __restrict__ go,
                                                           ConvGeom g, long long chunk_len) {
  __shared__ float red[4];
  const long long so = (long long)g.out[0] * g.out[1] * g.out[2];
  const long long si = (long long)g.in[0] * g.in[1] * g.in[2];
  const long long dom = g.batch * so;
  const int taps = g.k[0] * g.k[1] * g.k[2];
  const int cin_g = g.cin / g.groups;
  const int co = blockIdx.z, cil = blockIdx.y;  // cil: channel inside the group
  const int ci = (co / (g.cout / g.groups)) * cin_g + cil;
  const long long r0 = (long long)blockIdx.x * chunk_len;
  long long r1 = r0 + chunk_len;
  if (r1 > dom) r1 = dom;
  for (int kd = 0; kd < g.k[0]; ++kd)
    for (int kh = 0; kh < g.k[1]; ++kh)
      for (int kw = 0; kw < g.k[2]; ++kw) {
        float s = 0.0f;
        for (long long r = r0 + threadIdx.x; r < r1; r += 256) {
          const long long n = r / so;
          const long long sp = r - n * so;
          const int ow = (int)(sp % g.out[2]);
          const long long t = sp / g.out[2];
          const int oh = (int)(t % g.out[1]);
          const int od = (int)(t / g.out[1]);
          const int id = od * g.s[0] - g.p[0] + kd * g.d[0];
          const int ih = oh * g.s[1] - g.p[1] + kh * g.d[1];
          const int iw = ow * g.s[2] - g.p[2] + kw * g.d[2];
          if (id < 0 || id >= g.in[0] || ih < 0 || ih >= g.in[1] || iw < 0 || iw >= g.in[2])
            continue;
          const float gv = Elem<DT>::up(go[(n * g.cout + co) * so + sp]);
          const float xv = Elem<DT>::up(
              x[(n * g.cin + ci) * si + ((long long)id * g.in[1] + ih) * g.in[2] + iw]);
          s += gv * xv;
        }
        s = block_sum(s, red);
        const int tap = (kd * g.k[1] + kh) * g.k[2] + kw;
        if (threadIdx.x == 0)
          part[(((long long)blockIdx.x * g.cout + co) * cin_g + cil) * taps + tap] = s;
      }
}

// Stage 2: fixed-order sum over the chunk partials (deterministic). One wavefront per
// output: lane j adds partials j, j + 64, ... and a butterfly adds the lanes.
template <int DT>
__global__ __launch_bounds__(256) void reduce_parts_kernel(typename Elem<DT>::T* __restrict__ out,
                                                           const float* __restrict__ part,
                                                           long long count, int nparts) {
  const long long i = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (i >= count) return;
  float s = 0.0f;
  for (int k = lane; k < nparts; k += 64) s += part[(long long)k * count + i];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if (lane == 0) out[i] = Elem<DT>::down(s);
}

// ----------------------------------------------------------------- bias grad
// Stage 1: block (chunk, c) sums a contiguous slice of the (n, spatial) domain
// of channel c; part[chunk][c].
template <int DT>
__global__ __launch_bounds__(256) void bias_grad_kernel(float* __restrict__ part,
                                                        const typename Elem<DT>::T* __restrict__ go,
                                                        long long batch, int channels,
                                                        long long spatial, long long chunk_len) {
  __shared__ float red[4];
  typedef typename Elem<DT>::T T;
  constexpr int V = 16 / sizeof(T);
  const int c = blockIdx.y;
  const long long dom = batch * spatial;
  const long long r0 = (long long)blockIdx.x * chunk_len;
  long long r1 = r0 + chunk_len;
  if (r1 > dom) r1 = dom;
  float s = 0.0f;
  // chunk_len divides `spatial` or is a multiple of it, so a chunk never straddles
  // a plane boundary in the middle of a vector when the vector path is taken.
  const bool vec = (spatial % V == 0) && (chunk_len % V == 0) &&
                   (reinterpret_cast<uintptr_t>(go) % 16 == 0);
  if (vec) {
    for (long long r = r0 + (long long)threadIdx.x * V; r < r1; r += 256 * V) {
      const long long n = r / spatial;
      const long long sp = r - n * spatial;
      struct alignas(16) Pack { T v[V]; };
      const Pack p = *reinterpret_cast<const Pack*>(go + (n * channels + c) * spatial + sp);
#pragma unroll
      for (int i = 0; i < V; ++i) s += Elem<DT>::up(p.v[i]);
    }
  } else {
    for (long long r = r0 + threadIdx.x; r < r1; r += 256) {
      const long long n = r / spatial;
      const long long sp = r - n * spatial;
      s += Elem<DT>::up(go[(n * channels + c) * spatial + sp]);
    }
  }
  s = block_sum(s, red);
  if (threadIdx.x == 0) part[(long long)blockIdx.x * channels + c] = s;
}

bool known(int dt) { return dt == JG_F32 || dt == JG_BF16 || dt == JG_F16; }

int wgrad_chunks(long long dom, long long* chunk_len) {
  long long len = (dom + 127) / 128;
  if (len < 1024) len = 1024;
  *chunk_len = len;
  return (int)((dom + len - 1) / len);
}

int bias_chunks(long long batch, long long spatial, long long* chunk_len) {
  // about 64K elements per block, aligned to whole vectors
  long long dom = batch * spatial;
  long long len = 65536;
  if (len > dom) len = ((dom + 7) / 8) * 8;
  if (len < 8) len = 8;
  *chunk_len = len;
  return (int)((dom + len - 1) / len);
}

}  // namespace

namespace jg {

size_t direct_wgrad_workspace(const ConvGeom& g) {
  long long len;
  const long long so = (long long)g.out[0] * g.out[1] * g.out[2];
  const int chunks = wgrad_chunks(g.batch * so, &len);
  return (size_t)chunks * g.cout * (g.cin / g.groups) * g.k[0] * g.k[1] * g.k[2] * sizeof(float);
}

int direct_fwd(void* y, const void* x, const void* w, const void* bias, const ConvGeom& g,
               int dtype, hipStream_t s) {
  const long long so = (long long)g.out[0] * g.out[1] * g.out[2];
  if (g.batch == 0 || so == 0) return JG_OK;
  JG_REQUIRE(g.batch <= 65535, "conv fwd (direct): batch %lld exceeds 65535", (long long)g.batch);
  dim3 grid((unsigned)((so + 255) / 256), (unsigned)(g.groups * ((g.cout / g.groups + kCB - 1) / kCB)), (unsigned)g.batch);
#define JG_GO(DT)                                                                           \
  direct_fwd_kernel<DT><<<grid, 256, 0, s>>>(                                               \
      static_cast<Elem<DT>::T*>(y), static_cast<const Elem<DT>::T*>(x),                     \
      static_cast<const Elem<DT>::T*>(w), static_cast<const Elem<DT>::T*>(bias), g)
  if (dtype == JG_F32) JG_GO(JG_F32);
  else if (dtype == JG_BF16) JG_GO(JG_BF16);
  else JG_GO(JG_F16);
#undef JG_GO
  JG_CHECK_LAUNCH("jg_conv_fwd(direct)");
  return JG_OK;
}

int direct_dgrad(void* gx, const void* w, const void* go, const ConvGeom& g, int dtype,
                 hipStream_t s) {
  const long long si = (long long)g.in[0] * g.in[1] * g.in[2];
  if (g.batch == 0 || si == 0) return JG_OK;
  JG_REQUIRE(g.batch <= 65535, "conv dgrad (direct): batch %lld exceeds 65535",
             (long long)g.batch);
  dim3 grid((unsigned)((si + 255) / 256), (unsigned)(g.groups * ((g.cin / g.groups + kCB - 1) / kCB)), (unsigned)g.batch);
#define JG_GO(DT)                                                                           \
  direct_dgrad_kernel<DT><<<grid, 256, 0, s>>>(                                             \
      static_cast<Elem<DT>::T*>(gx), static_cast<const Elem<DT>::T*>(w),                    \
      static_cast<const Elem<DT>::T*>(go), g)
  if (dtype == JG_F32) JG_GO(JG_F32);
  else if (dtype == JG_BF16) JG_GO(JG_BF16);
  else JG_GO(JG_F16);
#undef JG_GO
  JG_CHECK_LAUNCH("jg_conv_dgrad(direct)");
  return JG_OK;
}

int direct_wgrad(void* gw, const void* x, const void* go, const ConvGeom& g, int dtype, void* ws,
                 size_t ws_bytes, hipStream_t s) {
  const long long so = (long long)g.out[0] * g.out[1] * g.out[2];
  const long long count = (long long)g.cout * (g.cin / g.groups) * g.k[0] * g.k[1] * g.k[2];
  if (count == 0) return JG_OK;
  JG_REQUIRE(g.cin <= 65535 && g.cout <= 65535, "conv wgrad (direct): too many channels");
  long long len;
  const int chunks = wgrad_chunks(g.batch * so, &len);
  if (ws == nullptr || ws_bytes < direct_wgrad_workspace(g))
    JG_FAIL(JG_ERR_WORKSPACE, "jg_conv_wgrad: workspace %zu < %zu bytes", ws_bytes,
            direct_wgrad_workspace(g));
  float* part = static_cast<float*>(ws);
  const bool empty = (g.batch * so == 0);  // nothing to reduce: the gradient is zero
  dim3 grid((unsigned)chunks, (unsigned)(g.cin / g.groups), (unsigned)g.cout);
#define JG_GO(DT)                                                                          \
  do {                                                                                     \
    if (!empty)                                                                            \
      direct_wgrad_kernel<DT><<<grid, 256, 0, s>>>(part, static_cast<const Elem<DT>::T*>(x), \
                                                   static_cast<const Elem<DT>::T*>(go), g, len); \
    reduce_parts_kernel<DT><<<(unsigned)((count + 3) / 4), 256, 0, s>>>(               \
        static_cast<Elem<DT>::T*>(gw), part, count, empty ? 0 : chunks);                   \
  } while (0)
  if (dtype == JG_F32) JG_GO(JG_F32);
  else if (dtype == JG_BF16) JG_GO(JG_BF16);
  else JG_GO(JG_F16);
#undef JG_GO
  JG_CHECK_LAUNCH("jg_conv_wgrad(direct)");
  return JG_OK;
}

}  // namespace jg

extern "C" size_t jg_bias_grad_workspace_bytes(int64_t batch, int64_t channels, int64_t spatial) {
  if (batch <= 0 || channels <= 0 || spatial <= 0) return 0;
  long long len;
  const int chunks = bias_chunks(batch, spatial, &len);
  return (size_t)chunks * channels * sizeof(float);
}

extern "C" int jg_bias_grad(void* gb, const void* g, int64_t batch, int64_t channels,
                            int64_t spatial, int dtype, void* workspace, size_t workspace_bytes,
                            void* stream) {
  JG_REQUIRE(gb && g, "jg_bias_grad: NULL pointer");
  JG_REQUIRE(batch >= 0 && channels >= 1 && channels <= 65535 && spatial >= 0,
             "jg_bias_grad: bad shape");
  JG_REQUIRE(known(dtype), "jg_bias_grad: unknown dtype %d", dtype);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool empty = (batch * spatial == 0);
  if (!empty && (workspace == nullptr || workspace_bytes < jg_bias_grad_workspace_bytes(batch, channels, spatial)))
    JG_FAIL(JG_ERR_WORKSPACE, "jg_bias_grad: workspace %zu < %zu bytes", workspace_bytes,
            jg_bias_grad_workspace_bytes(batch, channels, spatial));
  long long len = 8;
  const int chunks = empty ? 1 : bias_chunks(batch, spatial, &len);
  float* part = static_cast<float*>(workspace);
  dim3 grid((unsigned)chunks, (unsigned)channels, 1);
#define JG_GO(DT)                                                                             \
  do {                                                                                        \
    if (!empty)                                                                               \
      bias_grad_kernel<DT><<<grid, 256, 0, s>>>(part, static_cast<const Elem<DT>::T*>(g), batch, \
                                                (int)channels, spatial, len);                 \
    reduce_parts_kernel<DT><<<(unsigned)((channels + 3) / 4), 256, 0, s>>>(               \
        static_cast<Elem<DT>::T*>(gb), part, channels, empty ? 0 : chunks);                   \
  } while (0)
  if (dtype == JG_F32) JG_GO(JG_F32);
  else if (dtype == JG_BF16) JG_GO(JG_BF16);
  else JG_GO(JG_F16);
#undef JG_GO
  JG_CHECK_LAUNCH("jg_bias_grad");
  return JG_OK;
}
