// Attention inside small windows on the bf16 matrix cores: 64 queries x 64 keys,
// head size 32, additive fp32 bias (relative-position bias plus shift mask), as the
// Swin example runs it (examples/swin.py:129-170: F.scaled_dot_product_attention with
// attn_mask over (B, nW, heads, 64, 32) windows). Forward and backward.
//
//   Work split    one wavefront per (window, head) entry, four entries per workgroup.
//                 An entry is 4 KB per operand, so q, k, v, dout go from memory
//                 straight into MFMA fragments (a lane's 8 consecutive d values are 16
//                 contiguous bytes) and each is read once.
//   S^T = K Q^T   MFMA 32x32x16, A = K rows, B = Q rows: an accumulator lane owns ONE
//                 query and 16 of the 32 keys of a block, so max / sum / lse are per
//                 lane with one exchange between the two lanes that share a query.
//   O^T = V^T P^T the probabilities of a lane are already a B fragment if the 16 keys
//                 of a K-step are taken in the order the accumulator holds them
//                 (key = 16 t + 8 (j / 4) + 4 (lane / 32) + j % 4 for slot j); the A
//                 fragment is read from an LDS copy of V with that same key order,
//                 element by element (a transposed read: lane = d, slots = keys).
//   Backward      pass A (lane = query): P^T, dP^T = V dO^T, dS^T = P^T (dP^T - delta),
//                 dbias = dS^T, dQ^T = K^T dS^T. Pass B (lane = key) recomputes
//                 S = Q K^T and dP = dO V^T from the same fragments with the operands
//                 swapped, then dV^T = dO^T P, dK^T = Q^T dS. K, Q and dO sit in LDS
//                 for the transposed A fragments; lse and delta cross from the query
//                 lanes to the key lanes through LDS.
//   Numerics      scores, softmax and all accumulation in fp32; P and dS rounded to
//                 bf16 for the second matmuls (as the flash kernels do). lse is the
//                 natural-log sum-exp of scale * q k^T + bias.
//
// Reference behaviour restated here:
//   jigsaw/modules/attention/_functional/cores/math.py:31-149 (core forward / backward)
#include "attn_window_common.h"

namespace {

struct FwdArgs {
  const uint16_t *q, *k, *v;  // (batch, 64, 32)
  uint16_t* out;              // (batch, 64, 32)
  float* lse;                 // (batch, 64)
  const float* bias;          // (period, 64, 64) or NULL
  long long period, batch;
  float scale;
};

struct BwdArgs {
  const uint16_t *q, *k, *v, *dout, *out;
  const float* lse;
  const float* bias;
  long long period, batch;
  uint16_t *dq, *dk, *dv;
  float* dbias;  // (batch, 64, 64) or NULL
  float scale;
};

template <bool BIAS>
__global__ __launch_bounds__(WAVES * 64) void attn_window_fwd_kernel(FwdArgs p) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[WAVES * TILE];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  long long e = (long long)blockIdx.x * WAVES + wave;
  const bool valid = e < p.batch;
  if (!valid) e = p.batch - 1;  // computed again, not stored: every wavefront reaches the barrier
  const uint16_t* qe = p.q + e * (N * D);
  const uint16_t* ke = p.k + e * (N * D);
  const uint16_t* ve = p.v + e * (N * D);
  unsigned char* vt = smem + wave * TILE;

  bf16x8 kf[2][2], qf[2][2], vf[2][2];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      kf[b][ks] = load_frag(ke, b * 32 + ln, ks, kg);
      qf[b][ks] = load_frag(qe, b * 32 + ln, ks, kg);
      vf[b][ks] = load_frag(ve, b * 32 + ln, ks, kg);
    }
  store_tile(vt, vf, ln, kg);
  __syncthreads();

  const float c2 = p.scale * LOG2E;  // scores in base 2
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int qi = nb * 32 + ln;
    f32x16 s[2] = {zero16(), zero16()};
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
        s[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[mb][ks], qf[nb][ks], s[mb], 0, 0, 0);
    const float* be = BIAS ? p.bias + (e % p.period) * (N * N) + qi * N : nullptr;
    float x[2][16];
    float mx = -INFINITY;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        f32x4 bv = {0.0f, 0.0f, 0.0f, 0.0f};
        if (BIAS) bv = *reinterpret_cast<const f32x4*>(be + mb * 32 + i4 * 8 + kg * 4);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float t = s[mb][i4 * 4 + r] * c2 + bv[r] * LOG2E;
          x[mb][i4 * 4 + r] = t;
          mx = fmaxf(mx, t);
        }
      }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float ms = mx == -INFINITY ? 0.0f : mx;
    float sum = 0.0f;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        x[mb][i] = __builtin_amdgcn_exp2f(x[mb][i] - ms);
        sum += x[mb][i];
      }
    sum += __shfl_xor(sum, 32, 64);
    f32x16 o = zero16();
#pragma unroll
    for (int t = 0; t < 4; ++t)
      o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(vt, t, ln, kg), pack_half(x[t >> 1], t & 1), o, 0, 0, 0);
    if (valid) {
      const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
      uint16_t* orow = p.out + e * (N * D) + qi * D;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) *reinterpret_cast<u32x2*>(orow + i4 * 8 + kg * 4) = pack_rows(o, i4, inv);
      if (kg == 0) p.lse[e * N + qi] = sum > 0.0f ? ms * LN2 + __logf(sum) : -INFINITY;
    }
  }
}

template <bool BIAS, bool DBIAS>
__global__ __launch_bounds__(WAVES * 64) void attn_window_bwd_kernel(BwdArgs p) {
  constexpr int PER_WAVE = 3 * TILE + 2 * N * 4;
  __shared__ __attribute__((aligned(16))) unsigned char smem[WAVES * PER_WAVE];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  long long e = (long long)blockIdx.x * WAVES + wave;
  const bool valid = e < p.batch;
  if (!valid) e = p.batch - 1;
  const long long eo = e * (N * D);
  unsigned char* kt = smem + wave * PER_WAVE;
  unsigned char* qt = kt + TILE;
  unsigned char* dot = qt + TILE;
  float* lse_s = reinterpret_cast<float*>(dot + TILE);
  float* delta_s = lse_s + N;

  bf16x8 kf[2][2], qf[2][2], vf[2][2], dof[2][2];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      kf[b][ks] = load_frag(p.k + eo, b * 32 + ln, ks, kg);
      qf[b][ks] = load_frag(p.q + eo, b * 32 + ln, ks, kg);
      vf[b][ks] = load_frag(p.v + eo, b * 32 + ln, ks, kg);
      dof[b][ks] = load_frag(p.dout + eo, b * 32 + ln, ks, kg);
    }
  store_tile(kt, kf, ln, kg);
  store_tile(qt, qf, ln, kg);
  store_tile(dot, dof, ln, kg);

  // delta = rowsum(dout * out) and lse (in base 2) of this lane's queries
  float delta_q[2], lse_q[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int qi = nb * 32 + ln;
    float part = 0.0f;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const bf16x8 of = load_frag(p.out + eo, qi, ks, kg);
#pragma unroll
      for (int j = 0; j < 8; ++j) part += (float)dof[nb][ks][j] * (float)of[j];
    }
    part += __shfl_xor(part, 32, 64);
    delta_q[nb] = part;
    lse_q[nb] = p.lse[e * N + qi] * LOG2E;
    if (kg == 0) {
      delta_s[qi] = part;
      lse_s[qi] = lse_q[nb];
    }
  }
  __syncthreads();

  const float c2 = p.scale * LOG2E;
  const float* bias_e = BIAS ? p.bias + (e % p.period) * (N * N) : nullptr;

  // ---- pass A: lane = query
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int qi = nb * 32 + ln;
    f32x16 s[2] = {zero16(), zero16()}, dp[2] = {zero16(), zero16()};
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        s[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[mb][ks], qf[nb][ks], s[mb], 0, 0, 0);
        dp[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[mb][ks], dof[nb][ks], dp[mb], 0, 0, 0);
      }
    f32x16 dqa = zero16();
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      float ds[16];
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int key0 = mb * 32 + i4 * 8 + kg * 4;
        f32x4 bv = {0.0f, 0.0f, 0.0f, 0.0f};
        if (BIAS) bv = *reinterpret_cast<const f32x4*>(bias_e + qi * N + key0);
        f32x4 dsv;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = i4 * 4 + r;
          const float pr = __builtin_amdgcn_exp2f(s[mb][i] * c2 + bv[r] * LOG2E - lse_q[nb]);
          dsv[r] = pr * (dp[mb][i] - delta_q[nb]);
          ds[i] = dsv[r];
        }
        if (DBIAS && valid) *reinterpret_cast<f32x4*>(p.dbias + e * (N * N) + qi * N + key0) = dsv;
      }
#pragma unroll
      for (int h = 0; h < 2; ++h)
        dqa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(kt, mb * 2 + h, ln, kg), pack_half(ds, h), dqa, 0, 0, 0);
    }
    if (valid) {
      uint16_t* row = p.dq + eo + qi * D;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) *reinterpret_cast<u32x2*>(row + i4 * 8 + kg * 4) = pack_rows(dqa, i4, p.scale);
    }
  }

  // ---- pass B: lane = key
#pragma unroll
  for (int nbk = 0; nbk < 2; ++nbk) {
    const int ki = nbk * 32 + ln;
    f32x16 s[2] = {zero16(), zero16()}, dp[2] = {zero16(), zero16()};
#pragma unroll
    for (int mbq = 0; mbq < 2; ++mbq)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        s[mbq] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf[mbq][ks], kf[nbk][ks], s[mbq], 0, 0, 0);
        dp[mbq] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dof[mbq][ks], vf[nbk][ks], dp[mbq], 0, 0, 0);
      }
    f32x16 dva = zero16(), dka = zero16();
#pragma unroll
    for (int mbq = 0; mbq < 2; ++mbq) {
      float pr[16], ds[16];
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int q0 = mbq * 32 + i4 * 8 + kg * 4;
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(lse_s + q0);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(delta_s + q0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = i4 * 4 + r;
          const float bv = BIAS ? bias_e[(q0 + r) * N + ki] * LOG2E : 0.0f;
          pr[i] = __builtin_amdgcn_exp2f(s[mbq][i] * c2 + bv - l4[r]);
          ds[i] = pr[i] * (dp[mbq][i] - d4[r]);
        }
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        dva = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(dot, mbq * 2 + h, ln, kg), pack_half(pr, h), dva, 0, 0, 0);
        dka = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(qt, mbq * 2 + h, ln, kg), pack_half(ds, h), dka, 0, 0, 0);
      }
    }
    if (valid) {
      uint16_t* vrow = p.dv + eo + ki * D;
      uint16_t* krow = p.dk + eo + ki * D;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        *reinterpret_cast<u32x2*>(vrow + i4 * 8 + kg * 4) = pack_rows(dva, i4, 1.0f);
        *reinterpret_cast<u32x2*>(krow + i4 * 8 + kg * 4) = pack_rows(dka, i4, p.scale);
      }
    }
  }
}

}  // namespace

namespace jg {

bool attn_window_supported(long long batch, int sq, int sk, int d, int dtype) {
  return dtype == JG_BF16 && sq == N && sk == N && d == D && batch > 0 && batch < (1ll << 31) * WAVES;
}

int attn_window_fwd(void* out, float* lse, const void* q, const void* k, const void* v,
                    long long batch, float scale, const float* bias, long long bias_period,
                    hipStream_t s) {
  FwdArgs a;
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k);
  a.v = static_cast<const uint16_t*>(v);
  a.out = static_cast<uint16_t*>(out);
  a.lse = lse;
  a.bias = bias;
  a.period = bias ? bias_period : 1;
  a.batch = batch;
  a.scale = scale;
  const dim3 grid((unsigned)((batch + WAVES - 1) / WAVES)), block(WAVES * 64);
  if (bias)
    attn_window_fwd_kernel<true><<<grid, block, 0, s>>>(a);
  else
    attn_window_fwd_kernel<false><<<grid, block, 0, s>>>(a);
  JG_CHECK_LAUNCH("attn_window_fwd_kernel");
  return JG_OK;
}

int attn_window_bwd(void* dq, void* dk, void* dv, float* dbias, const void* dout, const void* q,
                    const void* k, const void* v, const void* out, const float* lse,
                    long long batch, float scale, const float* bias, long long bias_period,
                    hipStream_t s) {
  BwdArgs a;
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k);
  a.v = static_cast<const uint16_t*>(v);
  a.dout = static_cast<const uint16_t*>(dout);
  a.out = static_cast<const uint16_t*>(out);
  a.lse = lse;
  a.bias = bias;
  a.period = bias ? bias_period : 1;
  a.batch = batch;
  a.dq = static_cast<uint16_t*>(dq);
  a.dk = static_cast<uint16_t*>(dk);
  a.dv = static_cast<uint16_t*>(dv);
  a.dbias = dbias;
  a.scale = scale;
  const dim3 grid((unsigned)((batch + WAVES - 1) / WAVES)), block(WAVES * 64);
  if (bias && dbias)
    attn_window_bwd_kernel<true, true><<<grid, block, 0, s>>>(a);
  else if (bias)
    attn_window_bwd_kernel<true, false><<<grid, block, 0, s>>>(a);
  else if (dbias)
    attn_window_bwd_kernel<false, true><<<grid, block, 0, s>>>(a);
  else
    attn_window_bwd_kernel<false, false><<<grid, block, 0, s>>>(a);
  JG_CHECK_LAUNCH("attn_window_bwd_kernel");
  return JG_OK;
}

}  // namespace jg
