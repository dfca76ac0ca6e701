// Blockwise (flash-style) attention of one K/V chunk on the bf16 matrix cores,
// head size 64, non-causal, with the ring's log-sum-exp merge fused into the
// epilogue. Forward kernel.
//
//   S^T = K Q^T      MFMA 32x32x16: A = K rows (32 keys x 16 d, natural layout),
//                    B = Q rows (16 d x 32 queries, natural layout, kept in
//                    registers for the whole kernel). An accumulator lane then owns
//                    ONE query and 16 keys, so the running max / sum of the online
//                    softmax live in that lane's registers (one cross-lane exchange
//                    per 64 keys, between the two lanes that share a query).
//   O^T = V^T P^T    A = V^T (32 dv x 16 keys, from a transposed LDS copy), B = P^T:
//                    the probabilities of a lane are already in B-fragment position
//                    (the 16 keys of a K-step are taken in the order the accumulator
//                    holds them, and V^T is stored in LDS in that same order), so P
//                    never leaves registers. O^T keeps lane = query, so the rescale
//                    by exp(m_old - m_new) is per lane too.
//   Workgroup        512 threads = 8 wavefronts = 4 query blocks (32 queries) x 2
//                    key halves; the halves stream disjoint K/V tiles (64 keys,
//                    double buffered in LDS, prefetched through registers) and are
//                    combined through LDS at the end. 2 wavefronts per SIMD let the
//                    exp-heavy softmax of one overlap the MFMAs of the other.
//   Epilogue         out_j = O / l (bf16), lse_j = m*scale + ln l; optionally merged
//                    in place into the ring's fp32 accumulator:
//                    w = sigmoid(lse_j - lse), out += w (out_j - out), lse = logaddexp.
//
// Reference behaviour restated here:
//   jigsaw/modules/attention/_functional/cores/math.py:69-78 (per-chunk core)
//   jigsaw/modules/attention/_functional/forward.py:23-96    (merge per step)
#include "jg_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int D = 64;
constexpr int BM = 128;           // queries per workgroup
constexpr int BN = 64;            // keys per tile
constexpr int THREADS = 512;
constexpr int ROWB = 144;         // LDS row pitch in bytes (128 + 16: odd multiple of 16)
constexpr int KT_BYTES = BN * ROWB;        // K tile   [key][d]
constexpr int VT_BYTES = D * ROWB;         // V^T tile [dv][key position]
constexpr int TILE_BYTES = KT_BYTES + VT_BYTES;
constexpr int HALF_BYTES = 3 * TILE_BYTES; // three buffers of one key half
constexpr int LDS_BYTES = 2 * HALF_BYTES;  // 110592

struct FwdArgs {
  const uint16_t* q;   // (batch, sq, 64)
  const uint16_t* k;   // (batch, sk, 64)
  const uint16_t* v;
  uint16_t* out;       // (batch, sq, 64) or NULL
  float* lse;          // (batch, sq) or NULL
  float* out_acc;      // (batch, sq, 64) fp32, merged in place, or NULL
  float* lse_acc;      // (batch, sq) fp32, merged in place, or NULL
  int sq, sk;
  float scale;
};

__global__ __launch_bounds__(THREADS) void attn_fwd_mfma_kernel(FwdArgs p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int qb = wave & 3, ks = wave >> 2;
  const int th = tid & 255;  // thread index inside the key half
  const long long b = blockIdx.y;
  const int q0 = blockIdx.x * BM + qb * 32;
  const int khalf = p.sk >> 1;
  const int ntiles = khalf / BN;
  const float c2 = p.scale * 1.4426950408889634f;  // scores are handled in base 2

  unsigned char* lds = smem + ks * HALF_BYTES;
  const uint16_t* kbase = p.k + (b * p.sk + (long long)ks * khalf) * D;
  const uint16_t* vbase = p.v + (b * p.sk + (long long)ks * khalf) * D;

  // Q fragments of this wavefront's 32 queries (B operand of S^T = K Q^T)
  bf16x8 qf[4];
  {
    const uint16_t* qrow = p.q + (b * p.sq + q0 + ln) * D + 8 * kg;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      qf[c] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(qrow + 16 * c));
  }

  // ---- tile prefetch: K rows copied, V rows transposed to [dv][key position]
  u32x4 kst[2];
  uint32_t vst[8];
  const int k_row0 = th >> 3, k_c16 = th & 7;          // K chunk of the first pass (second pass: +32 rows)
  const int v_g8 = th >> 5, v_dvp = th & 31;           // V task: 8 keys x 2 dv
  auto issue_loads = [&](int t) {
    const uint16_t* kt = kbase + (long long)t * BN * D;
    const uint16_t* vt = vbase + (long long)t * BN * D;
    kst[0] = *reinterpret_cast<const u32x4*>(kt + k_row0 * D + k_c16 * 8);
    kst[1] = *reinterpret_cast<const u32x4*>(kt + (k_row0 + 32) * D + k_c16 * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      vst[i] = *reinterpret_cast<const uint32_t*>(vt + (v_g8 * 8 + i) * D + 2 * v_dvp);
  };
  auto store_tile = [&](int buf) {
    unsigned char* kt = lds + buf * TILE_BYTES;
    unsigned char* vt = kt + KT_BYTES;
    *reinterpret_cast<u32x4*>(kt + k_row0 * ROWB + k_c16 * 16) = kst[0];
    *reinterpret_cast<u32x4*>(kt + (k_row0 + 32) * ROWB + k_c16 * 16) = kst[1];
    // keys k0..k0+7 of this task, k0 = 8*v_g8. Position of key x inside its group of
    // 16: ((x%8)/4)*8 + (x/8)*4 + x%4  (the order an accumulator lane holds them).
    const int grp = v_g8 >> 1, h8 = v_g8 & 1;
    const int pos_lo = grp * 16 + h8 * 4;      // keys k0..k0+3
    const int pos_hi = pos_lo + 8;             // keys k0+4..k0+7
#pragma unroll
    for (int e = 0; e < 2; ++e) {              // dv = 2*v_dvp + e
      const uint32_t sel = e ? 0x07060302u : 0x05040100u;
      u32x2 lo, hi;
      lo.x = __builtin_amdgcn_perm(vst[1], vst[0], sel);
      lo.y = __builtin_amdgcn_perm(vst[3], vst[2], sel);
      hi.x = __builtin_amdgcn_perm(vst[5], vst[4], sel);
      hi.y = __builtin_amdgcn_perm(vst[7], vst[6], sel);
      // 16-byte chunks of a V^T row are XOR-swizzled with (row / 8) % 8: the 32 lanes
      // of a store, 288 bytes apart, would otherwise share 4 bank groups
      unsigned char* row = vt + (2 * v_dvp + e) * ROWB;
      const int sw = (v_dvp >> 2) & 7;
      *reinterpret_cast<u32x2*>(row + ((((pos_lo * 2) >> 4) ^ sw) << 4) + ((pos_lo * 2) & 15)) = lo;
      *reinterpret_cast<u32x2*>(row + ((((pos_hi * 2) >> 4) ^ sw) << 4) + ((pos_hi * 2) & 15)) = hi;
    }
  };

  f32x16 o[2];   // O^T: lane = query, register i of block nb = dv nb*32 + 8*(i/4) + 4*kg + i%4
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[nb][i] = 0.0f;
  float m = -INFINITY;  // running max of the raw scores of this query
  f32x16 lsum;          // running sum of the probabilities of this query (every register the same)
#pragma unroll
  for (int i = 0; i < 16; ++i) lsum[i] = 0.0f;
  bf16x8 ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = (__bf16)1.0f;

  // S^T of one 64-key tile: 2 blocks of 32 keys x 32 queries (prologue only)
  auto scores = [&](int buf, f32x16 (&s)[2]) {
    const unsigned char* kt = lds + buf * TILE_BYTES;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[sb][i] = 0.0f;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const bf16x8 a = __builtin_bit_cast(
            bf16x8, *reinterpret_cast<const u32x4*>(kt + (sb * 32 + ln) * ROWB + (16 * c + 8 * kg) * 2));
        s[sb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[c], s[sb], 0, 0, 0);
      }
    }
  };

  // Running max of a tile's scores; rescales the state when some lane of the wavefront
  // saw a larger score (the max settles after a few tiles, so this is a rarely taken,
  // wave-uniform branch). Returns the exponent offset of the tile.
  auto new_max = [&](const f32x16 (&s)[2]) {
    // tree over the 32 scores of the lane (short dependency chains), then the lane that
    // shares the query (lane ^ 32) through a register swap instead of an LDS round trip
    // (three-input maxima: v_max3_f32 halves the instruction count of the tree)
    auto max3 = [](float a, float b, float c) { return fmaxf(fmaxf(a, b), c); };
    float t[12];
#pragma unroll
    for (int i = 0; i < 5; ++i) {
      t[i] = max3(s[0][3 * i], s[0][3 * i + 1], s[0][3 * i + 2]);
      t[5 + i] = max3(s[1][3 * i], s[1][3 * i + 1], s[1][3 * i + 2]);
    }
    t[10] = s[0][15];
    t[11] = s[1][15];
    const float u0 = max3(t[0], t[1], t[2]), u1 = max3(t[3], t[4], t[5]);
    const float u2 = max3(t[6], t[7], t[8]), u3 = max3(t[9], t[10], t[11]);
    float mx = fmaxf(max3(u0, u1, u2), u3);
    float mn;
    {
      const uint32_t bits = __float_as_uint(mx);
      const auto sw = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
      mn = max3(__uint_as_float(sw[0]), __uint_as_float(sw[1]), m);
    }
    if (__builtin_amdgcn_ballot_w64(mn > m) != 0) {
      const float alpha = __builtin_amdgcn_exp2f((m - mn) * c2);
#pragma unroll
      for (int i = 0; i < 16; ++i) lsum[i] *= alpha;
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[nb][i] *= alpha;
      m = mn;
    }
    return m * c2;
  };

  // ---- software pipeline over the tiles, three LDS buffers per key half. In iteration t
  // the scores of tile t+1 and the P V products of tile t go to the matrix core one
  // instruction at a time, each followed by about its run time of vector work (the
  // exponentials of tile t); tile t+2 moves from registers to LDS and the global loads
  // of tile t+3 are issued. Past the last tile the same instructions run on clamped tile
  // indices and their results are dropped, which keeps the loop body free of branches
  // apart from the rare rescale. The fences pin the hand-made instruction order.
  const int last = ntiles - 1;
  issue_loads(0);
  store_tile(0);
  issue_loads(last < 1 ? last : 1);
  store_tile(1);
  issue_loads(last < 2 ? last : 2);
  __syncthreads();
  f32x16 s_a[2], s_b[2];
  scores(0, s_a);
  int b0 = 0, b1 = 1, b2 = 2;  // buffers of tiles t, t+1, t+2
#define JG_FENCE() __builtin_amdgcn_sched_barrier(0)
  auto iteration = [&](int t, const f32x16 (&s_in)[2], f32x16 (&s_out)[2]) {
    const unsigned char* kt = lds + b1 * TILE_BYTES;              // K of tile t+1
    const unsigned char* vt = lds + b0 * TILE_BYTES + KT_BYTES;   // V^T of tile t
    // K fragments of the next tile: requested first, they land under the max
    u32x4 kf[2][4];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int c = 0; c < 4; ++c)
        kf[sb][c] = *reinterpret_cast<const u32x4*>(kt + (sb * 32 + ln) * ROWB + (16 * c + 8 * kg) * 2);
    JG_FENCE();
    const float mc = new_max(s_in);
    JG_FENCE();
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int i = 0; i < 16; ++i) s_out[sb][i] = 0.0f;
    bf16x8 pk_prev;
    u32x4 vf_prev[2];
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      const int sb = f >> 1, tt = f & 1;
      // V^T fragments of this P fragment (used one stage later)
      u32x4 vf[2];
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
        vf[nb] = *reinterpret_cast<const u32x4*>(vt + (nb * 32 + ln) * ROWB +
                                                 (((sb * 4 + 2 * tt + kg) ^ ((nb * 4 + (ln >> 3)) & 7)) << 4));
      float x[8], e[8];
      // two score instructions of the next tile, vector work behind each
      s_out[sb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[sb][2 * tt]), qf[2 * tt],
                                                          s_out[sb], 0, 0, 0);
      JG_FENCE();
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = s_in[sb][8 * tt + i] * c2 - mc;
      JG_FENCE();
      s_out[sb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[sb][2 * tt + 1]),
                                                          qf[2 * tt + 1], s_out[sb], 0, 0, 0);
      JG_FENCE();
      e[0] = __builtin_amdgcn_exp2f(x[0]);
      e[1] = __builtin_amdgcn_exp2f(x[1]);
      JG_FENCE();
      // the three P V instructions of the previous fragment
      if (f > 0) lsum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pk_prev, lsum, 0, 0, 0);
      JG_FENCE();
      e[2] = __builtin_amdgcn_exp2f(x[2]);
      e[3] = __builtin_amdgcn_exp2f(x[3]);
      JG_FENCE();
      if (f > 0)
        o[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf_prev[0]), pk_prev, o[0], 0, 0, 0);
      JG_FENCE();
      e[4] = __builtin_amdgcn_exp2f(x[4]);
      e[5] = __builtin_amdgcn_exp2f(x[5]);
      JG_FENCE();
      if (f > 0)
        o[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf_prev[1]), pk_prev, o[1], 0, 0, 0);
      JG_FENCE();
      e[6] = __builtin_amdgcn_exp2f(x[6]);
      e[7] = __builtin_amdgcn_exp2f(x[7]);
      bf16x8 pk;
#pragma unroll
      for (int i = 0; i < 8; i += 2) {
        f32x2 v2 = {e[i], e[i + 1]};
        const bf16x2 h2 = __builtin_convertvector(v2, bf16x2);
        pk[i] = h2.x;
        pk[i + 1] = h2.y;
      }
      JG_FENCE();
      pk_prev = pk;
      vf_prev[0] = vf[0];
      vf_prev[1] = vf[1];
    }
    // last fragment's P V under the tile hand-over
    lsum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pk_prev, lsum, 0, 0, 0);
    JG_FENCE();
    store_tile(b2);
    JG_FENCE();
    o[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf_prev[0]), pk_prev, o[0], 0, 0, 0);
    JG_FENCE();
    issue_loads(t + 3 < last ? t + 3 : last);
    JG_FENCE();
    o[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf_prev[1]), pk_prev, o[1], 0, 0, 0);
    __syncthreads();
    const int tmp = b0;
    b0 = b1;
    b1 = b2;
    b2 = tmp;
  };
#undef JG_FENCE
  int t = 0;
  for (; t + 1 < ntiles; t += 2) {
    iteration(t, s_a, s_b);
    iteration(t + 1, s_b, s_a);
  }
  if (t < ntiles) iteration(t, s_a, s_b);

  // ---- the two key halves combine via LDS
  float l = lsum[0];
  float* xo = reinterpret_cast<float*>(smem) + qb * (32 * 64 + 128);  // [32 regs][64 lanes] + m,l
  if (ks == 1) {
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) xo[(nb * 16 + i) * 64 + lane] = o[nb][i];
    xo[32 * 64 + lane] = m;
    xo[32 * 64 + 64 + lane] = l;
  }
  __syncthreads();
  if (ks == 1) return;
  {
    const float m1 = xo[32 * 64 + lane], l1 = xo[32 * 64 + 64 + lane];
    const float mn = fmaxf(m, m1);
    const float a0 = __builtin_amdgcn_exp2f((m - mn) * c2), a1 = __builtin_amdgcn_exp2f((m1 - mn) * c2);
    l = l * a0 + l1 * a1;
    m = mn;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[nb][i] = o[nb][i] * a0 + xo[(nb * 16 + i) * 64 + lane] * a1;
  }

  // ---- epilogue: normalise, write and / or merge
  const float inv = 1.0f / l;
  const float lse_j = (m * c2 + log2f(l)) * 0.6931471805599453f;  // natural log
  const long long qi = b * p.sq + q0 + ln;
  float w = 0.0f;
  if (p.out_acc != nullptr) {
    const float l_old = p.lse_acc[qi];
    w = 1.0f / (1.0f + __expf(l_old - lse_j));  // sigmoid(lse_j - l_old); l_old = -inf -> 1
    if (kg == 0) {
      const float mxl = fmaxf(l_old, lse_j);
      p.lse_acc[qi] = mxl + log1pf(__expf(-fabsf(l_old - lse_j)));
    }
  }
  if (p.lse != nullptr && kg == 0) p.lse[qi] = lse_j;
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int dv = nb * 32 + 8 * j + 4 * kg;
      f32x4 val = {o[nb][4 * j] * inv, o[nb][4 * j + 1] * inv, o[nb][4 * j + 2] * inv,
                   o[nb][4 * j + 3] * inv};
      const bf16x4 h = __builtin_convertvector(val, bf16x4);  // the core's output dtype
      if (p.out != nullptr) *reinterpret_cast<bf16x4*>(p.out + qi * D + dv) = h;
      if (p.out_acc != nullptr) {
        f32x4* dst = reinterpret_cast<f32x4*>(p.out_acc + qi * D + dv);
        f32x4 a = *dst;
        const f32x4 hv = __builtin_convertvector(h, f32x4);
        a.x += w * (hv.x - a.x);
        a.y += w * (hv.y - a.y);
        a.z += w * (hv.z - a.z);
        a.w += w * (hv.w - a.w);
        *dst = a;
      }
    }
}

}  // namespace

namespace jg {

bool attn_mfma_fwd_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias) {
  return dtype == JG_BF16 && !has_bias && d == D && sq > 0 && sk > 0 && sq % BM == 0 &&
         sk % (2 * BN) == 0 && batch > 0 && batch <= 65535;
}

int attn_mfma_fwd(void* out, float* lse, const void* q, const void* k, const void* v,
                  long long batch, int sq, int sk, float scale, float* out_acc, float* lse_acc,
                  hipStream_t s) {
  FwdArgs a;
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k);
  a.v = static_cast<const uint16_t*>(v);
  a.out = static_cast<uint16_t*>(out);
  a.lse = lse;
  a.out_acc = out_acc;
  a.lse_acc = lse_acc;
  a.sq = sq;
  a.sk = sk;
  a.scale = scale;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_fwd_mfma_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (e != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "jg_attn_fwd: cannot reserve %d bytes of LDS", LDS_BYTES);
    attr_set = true;
  }
  dim3 grid((unsigned)(sq / BM), (unsigned)batch, 1);
  attn_fwd_mfma_kernel<<<grid, THREADS, LDS_BYTES, s>>>(a);
  JG_CHECK_LAUNCH("jg_attn_fwd(mfma)");
  return JG_OK;
}

}  // namespace jg

// The backward MFMA kernels live in attn_bwd_mfma.hip.
