// fp32 attention core on the matrix cores (v_mfma_f32_32x32x2_f32): forward with the natural-log
// LSE and, optionally, the merge into a running (out_acc, lse_acc) pair of a ring of chunks.
// Any sequence lengths, head size 32, 64 or 128, no bias. fp32 inputs took the one-thread-per-row
// kernels before (LDS broadcasts, 4 % of the fp32 peak); here a wavefront owns 32 queries and
// walks the keys 32 at a time:
//
//   S^T = K Q^T      A = K (row = key), B = Q^T (column = query); the two contraction slots of an
//                    MFMA step belong to the two halves of the wavefront, and half g owns the
//                    head-size slice [g D/2, (g + 1) D/2), so a lane reads its K slice as 16-byte
//                    words and keeps its Q slice in registers, scaled by scale * log2(e).
//   softmax          a lane holds 16 keys of ONE query (column = lane % 32): the row maximum and
//                    sum are 16 values in registers plus one exchange with the other half.
//   O^T = V^T P^T    A = V^T (row = head-size index), B = P^T: step i contracts the two keys whose
//                    probabilities the two halves hold in element i, so P never moves.
//
// Reference behaviour restated here:
//   jigsaw/modules/attention/_functional/cores/math.py:69-78   (forward, lse = logsumexp of the scaled scores)
//   jigsaw/modules/attention/_functional/forward.py (merge of a chunk into the running output by its LSE)
#include "jg_common.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kWaves = 4;
constexpr int kThreads = 64 * kWaves;
constexpr int kBQ = 32 * kWaves;  // queries per workgroup
constexpr int kBK = 32;           // keys per step

struct F32Params {
  float* out;          // (batch, sq, D) or NULL
  float* lse;          // (batch, sq) or NULL
  const float* q;      // (batch, sq, D)
  const float* k;      // (batch, sk, D)
  const float* v;      // (batch, sk, D)
  float* out_acc;      // (batch, sq, D) merged in place, or NULL
  float* lse_acc;      // (batch, sq) merged in place, or NULL
  int sq, sk, q_blocks;
  float scale_log2;    // scale * log2(e)
};

// key row (inside a 32-key step) of accumulator element i in half g: the 32x32 result layout
__device__ __forceinline__ int row_of(int i, int g) { return (i >> 2) * 8 + g * 4 + (i & 3); }

template <int D>
__global__ __launch_bounds__(kThreads) void attn_f32_mfma_fwd_kernel(F32Params p) {
  constexpr int H = D / 2;        // contraction slots of one half
  constexpr int PITCH = D + 4;    // LDS row pitch in floats: 16-byte rows, the b128 reads of 16 rows cover all banks
  constexpr int PIECES = D / 32;  // 16-byte pieces of a 32 x D tile per thread
  constexpr int NT = D / 32;      // 32-wide head-size tiles of the output
  __shared__ float Ks[kBK * PITCH];
  __shared__ float Vs[kBK * PITCH];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, n = lane & 31;
  const long long b = blockIdx.x / p.q_blocks;
  const int q0 = (int)(blockIdx.x % p.q_blocks) * kBQ;
  const int qrow = q0 + wave * 32 + n;
  const bool q_live = qrow < p.sq;
  const float* kb_base = p.k + b * (long long)p.sk * D;
  const float* vb_base = p.v + b * (long long)p.sk * D;

  // this lane's slice of its query, scaled
  float qf[H];
  {
    const float* qp = p.q + (b * p.sq + (q_live ? qrow : p.sq - 1)) * (long long)D + g * H;
#pragma unroll
    for (int j = 0; j < H; j += 4) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(qp + j);
      qf[j] = t.x * p.scale_log2;
      qf[j + 1] = t.y * p.scale_log2;
      qf[j + 2] = t.z * p.scale_log2;
      qf[j + 3] = t.w * p.scale_log2;
    }
  }

  f32x16 o[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[t][i] = 0.0f;
  float m = -INFINITY, l = 0.0f;

  const int steps = (p.sk + kBK - 1) / kBK;
  f32x4 kreg[PIECES], vreg[PIECES];
  auto fetch = [&](int step) {
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int e = tid + kThreads * i, row = e / (D / 4), c4 = e % (D / 4);
      const int key = step * kBK + row;
      const long long at = (long long)(key < p.sk ? key : p.sk - 1) * D + 4 * c4;
      kreg[i] = *reinterpret_cast<const f32x4*>(kb_base + at);
      const f32x4 t = *reinterpret_cast<const f32x4*>(vb_base + at);
      const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
      vreg[i] = key < p.sk ? t : zero;  // a key past the end weighs 0; its V row must not be 0 * anything
    }
  };
  fetch(0);
  for (int step = 0; step < steps; ++step) {
    __syncthreads();  // every wavefront is done with the previous tile
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int e = tid + kThreads * i, row = e / (D / 4), c4 = e % (D / 4);
      *reinterpret_cast<f32x4*>(Ks + row * PITCH + 4 * c4) = kreg[i];
      *reinterpret_cast<f32x4*>(Vs + row * PITCH + 4 * c4) = vreg[i];
    }
    __syncthreads();
    if (step + 1 < steps) fetch(step + 1);

    // S^T[key][query], in units of log2
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.0f;
#pragma unroll
    for (int j = 0; j < H; j += 4) {
      const f32x4 kv = *reinterpret_cast<const f32x4*>(Ks + n * PITCH + g * H + j);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qf[j], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qf[j + 1], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qf[j + 2], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qf[j + 3], s, 0, 0, 0);
    }
    if ((step + 1) * kBK > p.sk) {  // the last, ragged step
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (step * kBK + row_of(i, g) >= p.sk) s[i] = -INFINITY;
    }
    float mx = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);  // finite: key 0 of every step exists
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = __builtin_amdgcn_exp2f(s[i] - m_new);
      sum += s[i];
    }
    sum += __shfl_xor(sum, 32, 64);
    l = l * alpha + sum;
    m = m_new;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[t][i] *= alpha;

    // O^T[dv][query] += V^T P^T
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float* vrow = Vs + row_of(i, g) * PITCH + n;
#pragma unroll
      for (int t = 0; t < NT; ++t) o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[32 * t], s[i], o[t], 0, 0, 0);
    }
  }

  if (!q_live) return;
  const float inv = 1.0f / l;
  const float lse_j = (m + __builtin_amdgcn_logf(l)) * 0.6931471805599453f;  // v_log_f32 is log2
  const long long qi = b * p.sq + qrow;
  float w = 0.0f;
  if (p.out_acc != nullptr) {
    const float l_old = p.lse_acc[qi];
    w = 1.0f / (1.0f + expf(l_old - lse_j));  // sigmoid(lse_j - l_old); l_old = -inf -> 1
    if (g == 0) p.lse_acc[qi] = fmaxf(l_old, lse_j) + log1pf(expf(-fabsf(l_old - lse_j)));
  }
  if (g == 0 && p.lse != nullptr) p.lse[qi] = lse_j;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const long long at = qi * D + 32 * t + 8 * i4 + 4 * g;
      f32x4 val = {o[t][4 * i4] * inv, o[t][4 * i4 + 1] * inv, o[t][4 * i4 + 2] * inv, o[t][4 * i4 + 3] * inv};
      if (p.out != nullptr) *reinterpret_cast<f32x4*>(p.out + at) = val;
      if (p.out_acc != nullptr) {
        f32x4 a = *reinterpret_cast<const f32x4*>(p.out_acc + at);
        a.x += w * (val.x - a.x);
        a.y += w * (val.y - a.y);
        a.z += w * (val.z - a.z);
        a.w += w * (val.w - a.w);
        *reinterpret_cast<f32x4*>(p.out_acc + at) = a;
      }
    }
}

// ------------------------------------------------------------------ backward
// From the global output and LSE (cores/math.py:125-149): delta = rowsum(dO * O),
// P = exp(S - lse), dS = P * (dO V^T - delta), dQ = scale dS K, dK = scale dS^T Q, dV = P^T dO.
// Two kernels with the forward's operand placement. attn_f32_mfma_dq_kernel: a wavefront owns 32
// queries (a lane: one query, 16 keys a step), S^T = K Q^T and dP^T = V dO^T with the Q and dO
// slices in registers, then dQ^T += K^T dS^T with dS^T as it lies in the registers.
// attn_f32_mfma_dkv_kernel: a wavefront owns 32 keys (a lane: one key, 16 queries a step),
// S = Q K^T and dP = dO V^T with the K and V slices in registers, then dV^T += dO^T P and
// dK^T += Q^T dS. Both recompute S and dP (6 + 8 matrix products of 32 x 32 x D per tile pair for
// the 5 the mathematics needs once).
struct F32BwdParams {
  float* dq;           // (batch, sq, D)
  float* dk;           // (batch, sk, D)
  float* dv;           // (batch, sk, D)
  const float* dout;   // (batch, sq, D)
  const float* q;
  const float* k;
  const float* v;
  const float* lse;    // (batch, sq) natural log
  const float* delta;  // (batch, sq)
  int sq, sk, blocks_per_batch;
  float scale, scale_log2;
};

template <int D>
__global__ __launch_bounds__(kThreads) void attn_f32_delta_kernel(float* __restrict__ delta,
                                                                  const float* __restrict__ dout,
                                                                  const float* __restrict__ out, long long rows) {
  const long long r = (long long)blockIdx.x * (kThreads / 16) + threadIdx.x / 16;
  const int sl = threadIdx.x & 15;
  float a = 0.0f;
  if (r < rows) {
    for (int c = sl * 4; c < D; c += 64) {
      const f32x4 x = *reinterpret_cast<const f32x4*>(dout + r * D + c);
      const f32x4 y = *reinterpret_cast<const f32x4*>(out + r * D + c);
      a += x.x * y.x + x.y * y.y + x.z * y.z + x.w * y.w;
    }
  }
  for (int o = 8; o > 0; o >>= 1) a += __shfl_xor(a, o, 64);
  if (r < rows && sl == 0) delta[r] = a;
}

// A 32 x D tile of two tensors into registers (rows past `rows` read the last row; those of the
// second tensor become zero), and from there into LDS.
template <int D>
__device__ __forceinline__ void fetch_tiles(f32x4 (&a)[D / 32], f32x4 (&b)[D / 32], const float* abase,
                                            const float* bbase, int row0, int rows, int tid) {
#pragma unroll
  for (int i = 0; i < D / 32; ++i) {
    const int e = tid + kThreads * i, row = e / (D / 4), c4 = e % (D / 4);
    const int r = row0 + row;
    const long long at = (long long)(r < rows ? r : rows - 1) * D + 4 * c4;
    a[i] = *reinterpret_cast<const f32x4*>(abase + at);
    const f32x4 t = *reinterpret_cast<const f32x4*>(bbase + at);
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    b[i] = r < rows ? t : zero;
  }
}
template <int D>
__device__ __forceinline__ void store_tiles(float* as, float* bs, const f32x4 (&a)[D / 32], const f32x4 (&b)[D / 32],
                                            int tid) {
#pragma unroll
  for (int i = 0; i < D / 32; ++i) {
    const int e = tid + kThreads * i, row = e / (D / 4), c4 = e % (D / 4);
    *reinterpret_cast<f32x4*>(as + row * (D + 4) + 4 * c4) = a[i];
    *reinterpret_cast<f32x4*>(bs + row * (D + 4) + 4 * c4) = b[i];
  }
}

template <int D>
__global__ __launch_bounds__(kThreads) void attn_f32_mfma_dq_kernel(F32BwdParams p) {
  constexpr int H = D / 2, PITCH = D + 4, NT = D / 32;
  __shared__ float Ks[kBK * PITCH];
  __shared__ float Vs[kBK * PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, n = lane & 31;
  const long long b = blockIdx.x / p.blocks_per_batch;
  const int qrow = (int)(blockIdx.x % p.blocks_per_batch) * kBQ + wave * 32 + n;
  const bool q_live = qrow < p.sq;
  const long long qi = b * p.sq + (q_live ? qrow : p.sq - 1);
  const float* kb_base = p.k + b * (long long)p.sk * D;
  const float* vb_base = p.v + b * (long long)p.sk * D;

  float qf[H], dof[H];
#pragma unroll
  for (int j = 0; j < H; j += 4) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p.q + qi * D + g * H + j);
    const f32x4 u = *reinterpret_cast<const f32x4*>(p.dout + qi * D + g * H + j);
    qf[j] = t.x * p.scale_log2;
    qf[j + 1] = t.y * p.scale_log2;
    qf[j + 2] = t.z * p.scale_log2;
    qf[j + 3] = t.w * p.scale_log2;
    dof[j] = u.x;
    dof[j + 1] = u.y;
    dof[j + 2] = u.z;
    dof[j + 3] = u.w;
  }
  const float lse2 = p.lse[qi] * 1.4426950408889634f, dl = p.delta[qi];

  f32x16 dq[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[t][i] = 0.0f;

  const int steps = (p.sk + kBK - 1) / kBK;
  f32x4 kreg[NT], vreg[NT];
  fetch_tiles<D>(kreg, vreg, kb_base, vb_base, 0, p.sk, tid);
  for (int step = 0; step < steps; ++step) {
    __syncthreads();
    store_tiles<D>(Ks, Vs, kreg, vreg, tid);
    __syncthreads();
    if (step + 1 < steps) fetch_tiles<D>(kreg, vreg, kb_base, vb_base, (step + 1) * kBK, p.sk, tid);

    f32x16 s, dp;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = 0.0f;
      dp[i] = 0.0f;
    }
#pragma unroll
    for (int j = 0; j < H; j += 4) {
      const f32x4 kv = *reinterpret_cast<const f32x4*>(Ks + n * PITCH + g * H + j);
      const f32x4 vv = *reinterpret_cast<const f32x4*>(Vs + n * PITCH + g * H + j);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qf[j], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.x, dof[j], dp, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qf[j + 1], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.y, dof[j + 1], dp, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qf[j + 2], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.z, dof[j + 2], dp, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qf[j + 3], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.w, dof[j + 3], dp, 0, 0, 0);
    }
    const bool ragged = (step + 1) * kBK > p.sk;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float pr = __builtin_amdgcn_exp2f(s[i] - lse2);
      if (ragged && step * kBK + row_of(i, g) >= p.sk) pr = 0.0f;
      s[i] = pr * (dp[i] - dl);  // dS^T
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float* krow = Ks + row_of(i, g) * PITCH + n;
#pragma unroll
      for (int t = 0; t < NT; ++t) dq[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(krow[32 * t], s[i], dq[t], 0, 0, 0);
    }
  }
  if (!q_live) return;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const f32x4 val = {dq[t][4 * i4] * p.scale, dq[t][4 * i4 + 1] * p.scale, dq[t][4 * i4 + 2] * p.scale,
                         dq[t][4 * i4 + 3] * p.scale};
      *reinterpret_cast<f32x4*>(p.dq + qi * D + 32 * t + 8 * i4 + 4 * g) = val;
    }
}

template <int D>
__global__ __launch_bounds__(kThreads) void attn_f32_mfma_dkv_kernel(F32BwdParams p) {
  constexpr int H = D / 2, PITCH = D + 4, NT = D / 32;
  __shared__ float Qs[kBK * PITCH];
  __shared__ float dOs[kBK * PITCH];
  __shared__ float lse2s[kBK];
  __shared__ float deltas[kBK];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, n = lane & 31;
  const long long b = blockIdx.x / p.blocks_per_batch;
  const int krow = (int)(blockIdx.x % p.blocks_per_batch) * kBQ + wave * 32 + n;
  const bool k_live = krow < p.sk;
  const long long ki = b * p.sk + (k_live ? krow : p.sk - 1);
  const float* qb_base = p.q + b * (long long)p.sq * D;
  const float* dob_base = p.dout + b * (long long)p.sq * D;
  const float* lse_base = p.lse + b * (long long)p.sq;
  const float* delta_base = p.delta + b * (long long)p.sq;

  float kf[H], vf[H];
#pragma unroll
  for (int j = 0; j < H; j += 4) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p.k + ki * D + g * H + j);
    const f32x4 u = *reinterpret_cast<const f32x4*>(p.v + ki * D + g * H + j);
    kf[j] = t.x * p.scale_log2;
    kf[j + 1] = t.y * p.scale_log2;
    kf[j + 2] = t.z * p.scale_log2;
    kf[j + 3] = t.w * p.scale_log2;
    vf[j] = u.x;
    vf[j + 1] = u.y;
    vf[j + 2] = u.z;
    vf[j + 3] = u.w;
  }
  f32x16 dk[NT], dv[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dk[t][i] = 0.0f;
      dv[t][i] = 0.0f;
    }

  const int steps = (p.sq + kBK - 1) / kBK;
  f32x4 qreg[NT], doreg[NT];
  float lreg = 0.0f, dreg = 0.0f;
  auto fetch_rows = [&](int step) {  // the 32 queries' lse (in log2 units) and delta; 0 past the end
    if (tid < kBK) {
      const int r = step * kBK + tid;
      lreg = r < p.sq ? lse_base[r] * 1.4426950408889634f : 0.0f;
      dreg = r < p.sq ? delta_base[r] : 0.0f;
    }
  };
  fetch_tiles<D>(qreg, doreg, qb_base, dob_base, 0, p.sq, tid);
  fetch_rows(0);
  for (int step = 0; step < steps; ++step) {
    __syncthreads();
    store_tiles<D>(Qs, dOs, qreg, doreg, tid);
    if (tid < kBK) {
      lse2s[tid] = lreg;
      deltas[tid] = dreg;
    }
    __syncthreads();
    if (step + 1 < steps) {
      fetch_tiles<D>(qreg, doreg, qb_base, dob_base, (step + 1) * kBK, p.sq, tid);
      fetch_rows(step + 1);
    }

    f32x16 s, dp;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = 0.0f;
      dp[i] = 0.0f;
    }
#pragma unroll
    for (int j = 0; j < H; j += 4) {
      const f32x4 qv = *reinterpret_cast<const f32x4*>(Qs + n * PITCH + g * H + j);
      const f32x4 gv = *reinterpret_cast<const f32x4*>(dOs + n * PITCH + g * H + j);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(qv.x, kf[j], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(gv.x, vf[j], dp, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(qv.y, kf[j + 1], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(gv.y, vf[j + 1], dp, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(qv.z, kf[j + 2], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(gv.z, vf[j + 2], dp, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(qv.w, kf[j + 3], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x2f32(gv.w, vf[j + 3], dp, 0, 0, 0);
    }
    const bool ragged = (step + 1) * kBK > p.sq;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int qr = row_of(i, g);
      float pr = __builtin_amdgcn_exp2f(s[i] - lse2s[qr]);
      if (ragged && step * kBK + qr >= p.sq) pr = 0.0f;
      s[i] = pr;                          // P
      dp[i] = pr * (dp[i] - deltas[qr]);  // dS
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float* gorow = dOs + row_of(i, g) * PITCH + n;
      const float* qrow_ = Qs + row_of(i, g) * PITCH + n;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        dv[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(gorow[32 * t], s[i], dv[t], 0, 0, 0);
        dk[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(qrow_[32 * t], dp[i], dk[t], 0, 0, 0);
      }
    }
  }
  if (!k_live) return;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const long long at = ki * D + 32 * t + 8 * i4 + 4 * g;
      const f32x4 a = {dk[t][4 * i4] * p.scale, dk[t][4 * i4 + 1] * p.scale, dk[t][4 * i4 + 2] * p.scale,
                       dk[t][4 * i4 + 3] * p.scale};
      const f32x4 c = {dv[t][4 * i4], dv[t][4 * i4 + 1], dv[t][4 * i4 + 2], dv[t][4 * i4 + 3]};
      *reinterpret_cast<f32x4*>(p.dk + at) = a;
      *reinterpret_cast<f32x4*>(p.dv + at) = c;
    }
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

}  // namespace

namespace jg {

bool attn_f32_mfma_fwd_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias) {
  if (dtype != JG_F32 || has_bias || batch <= 0 || sq <= 0 || sk <= 0) return false;
  if (d != 32 && d != 64 && d != 128) return false;
  const long long blocks = batch * ((sq + kBQ - 1) / kBQ);
  return blocks <= 0x7fffffffLL;
}

int attn_f32_mfma_fwd(void* out, float* lse, const void* q, const void* k, const void* v, long long batch, int sq,
                      int sk, int d, float scale, float* out_acc, float* lse_acc, hipStream_t s) {
  for (const void* ptr : {static_cast<const void*>(out), q, k, v, static_cast<const void*>(out_acc)})
    JG_REQUIRE(aligned16(ptr), "jg_attn_fwd: the fp32 matrix-core kernel needs 16-byte aligned tensors");
  F32Params p;
  p.out = static_cast<float*>(out);
  p.lse = lse;
  p.q = static_cast<const float*>(q);
  p.k = static_cast<const float*>(k);
  p.v = static_cast<const float*>(v);
  p.out_acc = out_acc;
  p.lse_acc = lse_acc;
  p.sq = sq;
  p.sk = sk;
  p.q_blocks = (sq + kBQ - 1) / kBQ;
  p.scale_log2 = scale * 1.4426950408889634f;
  const unsigned blocks = (unsigned)(batch * p.q_blocks);
  if (d == 32) attn_f32_mfma_fwd_kernel<32><<<blocks, kThreads, 0, s>>>(p);
  else if (d == 64) attn_f32_mfma_fwd_kernel<64><<<blocks, kThreads, 0, s>>>(p);
  else attn_f32_mfma_fwd_kernel<128><<<blocks, kThreads, 0, s>>>(p);
  JG_CHECK_LAUNCH("jg_attn_fwd(fp32 mfma)");
  return JG_OK;
}

bool attn_f32_mfma_bwd_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias) {
  if (!attn_f32_mfma_fwd_supported(batch, sq, sk, d, dtype, has_bias)) return false;
  return batch * ((sk + kBQ - 1) / kBQ) <= 0x7fffffffLL;
}

// workspace: (batch, sq) floats for delta
int attn_f32_mfma_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q, const void* k, const void* v,
                      const void* out, const float* lse, long long batch, int sq, int sk, int d, float scale,
                      void* workspace, hipStream_t s) {
  for (const void* ptr : {static_cast<const void*>(dq), static_cast<const void*>(dk), static_cast<const void*>(dv),
                          dout, q, k, v, out})
    JG_REQUIRE(aligned16(ptr), "jg_attn_bwd: the fp32 matrix-core kernels need 16-byte aligned tensors");
  F32BwdParams p;
  p.dq = static_cast<float*>(dq);
  p.dk = static_cast<float*>(dk);
  p.dv = static_cast<float*>(dv);
  p.dout = static_cast<const float*>(dout);
  p.q = static_cast<const float*>(q);
  p.k = static_cast<const float*>(k);
  p.v = static_cast<const float*>(v);
  p.lse = lse;
  float* delta = static_cast<float*>(workspace);
  p.delta = delta;
  p.sq = sq;
  p.sk = sk;
  p.scale = scale;
  p.scale_log2 = scale * 1.4426950408889634f;
  const long long rows = batch * sq;
  const unsigned delta_blocks = (unsigned)((rows + kThreads / 16 - 1) / (kThreads / 16));
  const unsigned q_blocks = (unsigned)(batch * ((sq + kBQ - 1) / kBQ)), k_blocks = (unsigned)(batch * ((sk + kBQ - 1) / kBQ));
#define JG_GO(DD)                                                                                          \
  do {                                                                                                     \
    attn_f32_delta_kernel<DD><<<delta_blocks, kThreads, 0, s>>>(delta, p.dout, static_cast<const float*>(out), rows); \
    p.blocks_per_batch = (sq + kBQ - 1) / kBQ;                                                             \
    attn_f32_mfma_dq_kernel<DD><<<q_blocks, kThreads, 0, s>>>(p);                                          \
    p.blocks_per_batch = (sk + kBQ - 1) / kBQ;                                                             \
    attn_f32_mfma_dkv_kernel<DD><<<k_blocks, kThreads, 0, s>>>(p);                                         \
  } while (0)
  if (d == 32) JG_GO(32);
  else if (d == 64) JG_GO(64);
  else JG_GO(128);
#undef JG_GO
  JG_CHECK_LAUNCH("jg_attn_bwd(fp32 mfma)");
  return JG_OK;
}

}  // namespace jg
