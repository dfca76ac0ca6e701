// Backward of the blockwise attention core on the bf16 matrix cores, head size
// 64, from the ring's GLOBAL out / lse (p = exp(s - lse) is already globally
// normalised). Two kernels, no atomics, deterministic:
//
//   dQ kernel      lane = query (as in the forward kernel). Per 64-key tile:
//                    S^T  = K Q^T                 A = K rows,    B = Q (registers)
//                    dP^T = V dO^T                A = V rows,    B = dO (registers)
//                    dS^T = P^T o (dP^T - delta) * scale      (lane-local)
//                    dQ^T += K^T dS^T             A = K^T (transposed LDS copy),
//                                                 B = dS^T straight from registers
//                  It also computes delta = rowsum(dO o O) and leaves it in the
//                  workspace for the second kernel.
//   dK/dV kernel   lane = key. Per 64-query tile:
//                    S  = Q K^T                   A = Q rows,    B = K (registers)
//                    dP = dO V^T                  A = dO rows,   B = V (registers)
//                    P, dS from lse / delta of the tile (broadcast LDS reads)
//                    dV^T += dO^T P               A = dO^T (transposed LDS copy)
//                    dK^T += Q^T dS               A = Q^T  (transposed LDS copy)
//   The score tile is recomputed in each kernel (7 matrix products instead of the
//   5 of a one-kernel formulation) so that P / dS are always produced in the
//   register layout the next MFMA consumes and never travel through LDS.
//
//   Workgroup: 512 threads = 8 wavefronts = 4 blocks of 32 rows (queries for dQ,
//   keys for dK/dV) x 2 halves of the streamed side, combined through LDS.
//   Streamed tiles are fetched as 8-row x 2-column dword tasks, which one thread
//   can write both untransposed and transposed (8 channels-per-slot trick).
//
// Reference behaviour restated here:
//   jigsaw/modules/attention/_functional/cores/math.py:125-149
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
constexpr int BR = 128;           // resident rows per workgroup (4 blocks of 32)
constexpr int BT = 64;            // streamed rows per tile
constexpr int THREADS = 512;
constexpr int ROWB = 144;         // LDS row pitch in bytes
constexpr int TILE = BT * ROWB;   // 9216: one 64 x 64 bf16 tile, natural or transposed
constexpr float LOG2E = 1.4426950408889634f;

// Transposed tiles hold streamed row x (0..63) at position
//   (x & ~15) | ((x % 8) / 4) * 8 | ((x % 16) / 8) * 4 | (x % 4):
// inside each group of 16 the order is the one an accumulator lane holds its rows in.

// A task = 8 consecutive streamed rows x 2 consecutive columns, held as 8 dwords.
struct Task {
  uint32_t w[8];
};

__device__ __forceinline__ void task_load(Task& t, const uint16_t* tile, int g8, int cp) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
    t.w[i] = *reinterpret_cast<const uint32_t*>(tile + (g8 * 8 + i) * D + 2 * cp);
}

__device__ __forceinline__ void task_store_nat(const Task& t, unsigned char* nat, int g8, int cp) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
    *reinterpret_cast<uint32_t*>(nat + (g8 * 8 + i) * ROWB + 4 * cp) = t.w[i];
}

__device__ __forceinline__ void task_store_tr(const Task& t, unsigned char* tr, int g8, int cp) {
  const int pos_lo = (g8 >> 1) * 16 + (g8 & 1) * 4;  // rows 8*g8 .. +3
  const int pos_hi = pos_lo + 8;                     // rows 8*g8+4 .. +7
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const uint32_t sel = e ? 0x07060302u : 0x05040100u;
    u32x2 lo, hi;
    lo.x = __builtin_amdgcn_perm(t.w[1], t.w[0], sel);
    lo.y = __builtin_amdgcn_perm(t.w[3], t.w[2], sel);
    hi.x = __builtin_amdgcn_perm(t.w[5], t.w[4], sel);
    hi.y = __builtin_amdgcn_perm(t.w[7], t.w[6], sel);
    unsigned char* row = tr + (2 * cp + e) * ROWB;
    *reinterpret_cast<u32x2*>(row + pos_lo * 2) = lo;
    *reinterpret_cast<u32x2*>(row + pos_hi * 2) = hi;
  }
}

__device__ __forceinline__ bf16x8 lds_frag(const unsigned char* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(p));
}

// Natural (untransposed) 64 x 64 tiles travel from memory straight into LDS (no registers,
// no ds_write): a wavefront instruction lands 64 x 16 bytes contiguously, lane order. Rows
// are 128 bytes, and the 16-byte chunks of a row are XOR-swizzled with (row / 2) % 8 so that
// the 16 lanes a fragment read serves per cycle hit 16 distinct chunks of the banks.
constexpr int NAT = BT * D * 2;  // 8192 bytes

// Four of the 8 instructions of a tile: the 256 threads of a half fetch 4 KB per call.
__device__ __forceinline__ void nat_dma(const uint16_t* tile, unsigned char* lds_tile, int th, int part) {
  const int w = (th >> 6) + 4 * part;          // instruction 0..7 -> rows 8w .. 8w+7
  const int i = th & 63;
  const int row = 8 * w + (i >> 3);
  const int chunk = (i & 7) ^ ((row >> 1) & 7);
  __builtin_amdgcn_global_load_lds(reinterpret_cast<const char*>(tile) + row * (D * 2) + chunk * 16,
                                   (__attribute__((address_space(3))) void*)(lds_tile + w * 1024), 16, 0, 0);
}

// fragment of a natural tile: row r (0..63), 16-byte chunk c (0..7)
__device__ __forceinline__ bf16x8 nat_frag(const unsigned char* nat, int r, int c) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(nat + r * (D * 2) + ((c ^ ((r >> 1) & 7)) << 4)));
}

__device__ __forceinline__ bf16x8 pack8(const float* e) {
  bf16x8 pk;
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    f32x2 v2 = {e[i], e[i + 1]};
    const bf16x2 h2 = __builtin_convertvector(v2, bf16x2);
    pk[i] = h2.x;
    pk[i + 1] = h2.y;
  }
  return pk;
}

struct BwdArgs {
  const uint16_t* dout;
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  const uint16_t* out;
  const float* lse;
  float* delta;     // (batch, sq) workspace
  uint16_t* dq;
  uint16_t* dk;
  uint16_t* dv;
  int sq, sk;
  float scale;
};

// ------------------------------------------------------------------ dQ kernel
constexpr int DQ_BUF = 2 * NAT + TILE;       // K natural, V natural, K transposed
constexpr int DQ_HALF = 2 * DQ_BUF;         // double buffered
constexpr int DQ_LDS = 2 * DQ_HALF;         // 102400

__global__ __launch_bounds__(THREADS) void attn_bwd_dq_kernel(BwdArgs p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int qb = wave & 3, ks = wave >> 2;
  const int th = tid & 255;
  const int g8 = th >> 5, cp = th & 31;
  const long long b = blockIdx.y;
  const int q0 = blockIdx.x * BR + qb * 32;
  const int khalf = p.sk >> 1;
  const int ntiles = khalf / BT;
  const float c2 = p.scale * LOG2E;
  const long long qi = b * p.sq + q0 + ln;

  unsigned char* lds = smem + ks * DQ_HALF;
  const uint16_t* kbase = p.k + (b * p.sk + (long long)ks * khalf) * D;
  const uint16_t* vbase = p.v + (b * p.sk + (long long)ks * khalf) * D;

  bf16x8 qf[4], dof[4];
  float delta;
  {
    const uint16_t* qrow = p.q + qi * D + 8 * kg;
    const uint16_t* drow = p.dout + qi * D + 8 * kg;
    const uint16_t* orow = p.out + qi * D + 8 * kg;
    float dl = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      qf[c] = lds_frag(reinterpret_cast<const unsigned char*>(qrow + 16 * c));
      dof[c] = lds_frag(reinterpret_cast<const unsigned char*>(drow + 16 * c));
      const bf16x8 of = lds_frag(reinterpret_cast<const unsigned char*>(orow + 16 * c));
#pragma unroll
      for (int i = 0; i < 8; ++i) dl += (float)dof[c][i] * (float)of[i];
    }
    delta = dl + __shfl_xor(dl, 32, 64);
    if (ks == 0 && kg == 0) p.delta[qi] = delta;
  }
  const float lse2 = p.lse[qi] * LOG2E;

  Task tk;
  // K and V of tile t straight into buffer `buf` (it must be free: the barrier that ended
  // the iteration before), K once more through registers for the transposed copy
  auto issue_loads = [&](int t, int buf) {
    unsigned char* base = lds + buf * DQ_BUF;
    const uint16_t* kt_g = kbase + (long long)t * BT * D;
    const uint16_t* vt_g = vbase + (long long)t * BT * D;
    nat_dma(kt_g, base, th, 0);
    nat_dma(kt_g, base, th, 1);
    nat_dma(vt_g, base + NAT, th, 0);
    nat_dma(vt_g, base + NAT, th, 1);
    task_load(tk, kt_g, g8, cp);
  };
  auto store_tile = [&](int buf) {
    task_store_tr(tk, lds + buf * DQ_BUF + 2 * NAT, g8, cp);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the direct-to-LDS loads of this buffer have landed
  };

  f32x16 dq[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[nb][i] = 0.0f;

  // One 64-key tile. The two 32-key blocks are software pipelined: the score / dP
  // products of block 1 go to the matrix core one instruction at a time with the
  // exponentials of block 0 behind them, and the dQ products of a fragment run under
  // the vector work of the next one. The fences pin that order. dS is kept without the
  // softmax scale, which multiplies dQ once at the end.
#define JG_FENCE() __builtin_amdgcn_sched_barrier(0)
  auto compute_tile = [&](int buf) {
    const unsigned char* kn = lds + buf * DQ_BUF;
    const unsigned char* vn = kn + NAT;
    const unsigned char* kt = kn + 2 * NAT;
    f32x16 s[2], dp[2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s[sb][i] = 0.0f;
        dp[sb][i] = 0.0f;
      }
    // fragment (sb, t): 8 probabilities -> dS, packed for the dQ product
    auto ds_frag = [&](int sb, int t) {
      float e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float pr = __builtin_amdgcn_exp2f(s[sb][8 * t + i] * c2 - lse2);
        e[i] = pr * (dp[sb][8 * t + i] - delta);
      }
      return pack8(e);
    };
    auto dq_mfma = [&](int sb, int t, int nb, const bf16x8& f) {
      dq[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
          lds_frag(kt + (nb * 32 + ln) * ROWB + (sb * 32 + 16 * t + 8 * kg) * 2), f, dq[nb], 0, 0, 0);
    };
    // block 0: scores and dP
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      s[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nat_frag(kn, ln, 2 * c + kg), qf[c], s[0], 0, 0, 0);
      dp[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nat_frag(vn, ln, 2 * c + kg), dof[c], dp[0], 0, 0, 0);
    }
    JG_FENCE();
    // block 1 products with the vector work of block 0 behind them
    bf16x8 f00, f01;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      s[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nat_frag(kn, 32 + ln, 2 * c + kg), qf[c], s[1], 0, 0, 0);
      dp[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nat_frag(vn, 32 + ln, 2 * c + kg), dof[c], dp[1], 0, 0, 0);
      if (c == 1) f00 = ds_frag(0, 0);
      if (c == 3) f01 = ds_frag(0, 1);
      JG_FENCE();
    }
    // dQ products of block 0 under the vector work of block 1
    dq_mfma(0, 0, 0, f00);
    dq_mfma(0, 0, 1, f00);
    JG_FENCE();
    const bf16x8 f10 = ds_frag(1, 0);
    JG_FENCE();
    dq_mfma(0, 1, 0, f01);
    dq_mfma(0, 1, 1, f01);
    JG_FENCE();
    const bf16x8 f11 = ds_frag(1, 1);
    JG_FENCE();
    dq_mfma(1, 0, 0, f10);
    dq_mfma(1, 0, 1, f10);
    dq_mfma(1, 1, 0, f11);
    dq_mfma(1, 1, 1, f11);
  };
#undef JG_FENCE

  int buf = 0;
  issue_loads(0, 0);
  store_tile(0);
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const bool has_next = t + 1 < ntiles;
    if (has_next) issue_loads(t + 1, buf ^ 1);
    compute_tile(buf);
    if (has_next) store_tile(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  // combine the two key halves, then write dQ (lane = query, 4 consecutive d per store)
  float* xo = reinterpret_cast<float*>(smem) + qb * (32 * 64);
  if (ks == 1) {
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) xo[(nb * 16 + i) * 64 + lane] = dq[nb][i];
  }
  __syncthreads();
  if (ks == 1) return;
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f32x4 val;
      val.x = (dq[nb][4 * j + 0] + xo[(nb * 16 + 4 * j + 0) * 64 + lane]) * p.scale;
      val.y = (dq[nb][4 * j + 1] + xo[(nb * 16 + 4 * j + 1) * 64 + lane]) * p.scale;
      val.z = (dq[nb][4 * j + 2] + xo[(nb * 16 + 4 * j + 2) * 64 + lane]) * p.scale;
      val.w = (dq[nb][4 * j + 3] + xo[(nb * 16 + 4 * j + 3) * 64 + lane]) * p.scale;
      *reinterpret_cast<bf16x4*>(p.dq + qi * D + nb * 32 + 8 * j + 4 * kg) =
          __builtin_convertvector(val, bf16x4);
    }
}

// -------------------------------------------------------------- dK/dV kernel
constexpr int DKV_STATS = 2 * BT * 4;                 // lse2[64], delta[64] as floats
constexpr int DKV_HALF = 4 * TILE + DKV_STATS;        // Q nat, Q tr, dO nat, dO tr + stats
constexpr int DKV_LDS = 4 * DKV_HALF;                 // 149504: two query halves, double buffered

__global__ __launch_bounds__(THREADS) void attn_bwd_dkv_kernel(BwdArgs p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int kb = wave & 3, qs = wave >> 2;
  const int th = tid & 255;
  const int g8 = th >> 5, cp = th & 31;
  const long long b = blockIdx.y;
  const int k0 = blockIdx.x * BR + kb * 32;
  const int qhalf = p.sq >> 1;
  const int ntiles = qhalf / BT;
  const float c2 = p.scale * LOG2E;
  const long long ki = b * p.sk + k0 + ln;

  unsigned char* lds = smem + qs * (2 * DKV_HALF);  // two buffers: Q nat, Q tr, dO nat, dO tr, stats
  const long long qrow0 = b * p.sq + (long long)qs * qhalf;
  const uint16_t* qbase = p.q + qrow0 * D;
  const uint16_t* dbase = p.dout + qrow0 * D;

  bf16x8 kf[4], vf[4];
  {
    const uint16_t* krow = p.k + ki * D + 8 * kg;
    const uint16_t* vrow = p.v + ki * D + 8 * kg;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      kf[c] = lds_frag(reinterpret_cast<const unsigned char*>(krow + 16 * c));
      vf[c] = lds_frag(reinterpret_cast<const unsigned char*>(vrow + 16 * c));
    }
  }

  Task tq, tdo;
  float st_reg = 0.0f;
  auto issue_loads = [&](int t) {
    task_load(tq, qbase + (long long)t * BT * D, g8, cp);
    task_load(tdo, dbase + (long long)t * BT * D, g8, cp);
    // One plain load for every lane, used only when the tile goes to LDS: a load under a
    // per-lane condition, or arithmetic on its result here, would make the wavefront wait
    // for it (and for the tile loads issued before it) on the spot.
    const float* src = th < BT ? p.lse : p.delta;
    st_reg = src[qrow0 + (long long)t * BT + (th & (BT - 1))];
  };
  auto store_tile = [&](int buf) {
    unsigned char* base = lds + buf * DKV_HALF;
    task_store_nat(tq, base, g8, cp);
    task_store_tr(tq, base + TILE, g8, cp);
    task_store_nat(tdo, base + 2 * TILE, g8, cp);
    task_store_tr(tdo, base + 3 * TILE, g8, cp);
    if (th < 2 * BT) reinterpret_cast<float*>(base + 4 * TILE)[th] = th < BT ? st_reg * LOG2E : st_reg;
  };

  f32x16 dk[2], dv[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      dk[nb][i] = 0.0f;
      dv[nb][i] = 0.0f;
    }

  // dS is kept without the softmax scale, which multiplies dK once at the end
  auto compute_tile = [&](int buf) {
    const unsigned char* qn = lds + buf * DKV_HALF;
    const unsigned char* qt = qn + TILE;
    const unsigned char* dn = qn + 2 * TILE;
    const unsigned char* dt = qn + 3 * TILE;
    const float* st = reinterpret_cast<const float*>(qn + 4 * TILE);  // lse2[64] then delta[64]
    bf16x8 pf[2][2], dsf[2][2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      f32x16 s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s[i] = 0.0f;
        dp[i] = 0.0f;
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int off = (sb * 32 + ln) * ROWB + (16 * c + 8 * kg) * 2;
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(qn + off), kf[c], s, 0, 0, 0);
        dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(dn + off), vf[c], dp, 0, 0, 0);
      }
      // register i of this lane: query sb*32 + 8*(i/4) + 4*kg + i%4, key ln
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float pe[8], de[8];
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const int j = 2 * t + jj;
          const f32x4 l4 = *reinterpret_cast<const f32x4*>(st + sb * 32 + 8 * j + 4 * kg);
          const f32x4 d4 = *reinterpret_cast<const f32x4*>(st + BT + sb * 32 + 8 * j + 4 * kg);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float pr = __builtin_amdgcn_exp2f(s[4 * j + e] * c2 - l4[e]);
            pe[4 * jj + e] = pr;
            de[4 * jj + e] = pr * (dp[4 * j + e] - d4[e]);
          }
        }
        pf[sb][t] = pack8(pe);
        dsf[sb][t] = pack8(de);
      }
    }
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          const int off = (nb * 32 + ln) * ROWB + (sb * 32 + 16 * t + 8 * kg) * 2;
          dv[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(dt + off), pf[sb][t], dv[nb], 0, 0, 0);
          dk[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(qt + off), dsf[sb][t], dk[nb], 0, 0, 0);
        }
  };

  int buf = 0;
  issue_loads(0);
  store_tile(0);
  // The K / V fragments came straight from memory: they are waited for here, once. Left
  // to the first MFMA that reads them, the wait would sit inside the loop, behind the
  // tile loads that every iteration has just issued.
#pragma unroll
  for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(kf[c]), "+v"(vf[c]));
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const bool has_next = t + 1 < ntiles;
    if (has_next) issue_loads(t + 1);
    compute_tile(buf);
    if (has_next) store_tile(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  // combine the two query halves, then write dK / dV (lane = key)
  float* xo = reinterpret_cast<float*>(smem) + kb * (64 * 64);
  if (qs == 1) {
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        xo[(nb * 16 + i) * 64 + lane] = dk[nb][i];
        xo[(32 + nb * 16 + i) * 64 + lane] = dv[nb][i];
      }
  }
  __syncthreads();
  if (qs == 1) return;
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f32x4 a, c;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        a[e] = (dk[nb][4 * j + e] + xo[(nb * 16 + 4 * j + e) * 64 + lane]) * p.scale;
        c[e] = dv[nb][4 * j + e] + xo[(32 + nb * 16 + 4 * j + e) * 64 + lane];
      }
      const int col = nb * 32 + 8 * j + 4 * kg;
      *reinterpret_cast<bf16x4*>(p.dk + ki * D + col) = __builtin_convertvector(a, bf16x4);
      *reinterpret_cast<bf16x4*>(p.dv + ki * D + col) = __builtin_convertvector(c, bf16x4);
    }
}

}  // namespace

namespace jg {

bool attn_mfma_bwd_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias) {
  return dtype == JG_BF16 && !has_bias && d == D && sq > 0 && sk > 0 && sq % BR == 0 &&
         sk % BR == 0 && batch > 0 && batch <= 65535;
}

size_t attn_mfma_bwd_workspace(long long batch, int sq, int) {
  return (size_t)batch * sq * sizeof(float);
}

int attn_mfma_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q, const void* k,
                  const void* v, const void* out, const float* lse, long long batch, int sq,
                  int sk, float scale, void* ws, hipStream_t s) {
  BwdArgs a;
  a.dout = static_cast<const uint16_t*>(dout);
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k);
  a.v = static_cast<const uint16_t*>(v);
  a.out = static_cast<const uint16_t*>(out);
  a.lse = lse;
  a.delta = static_cast<float*>(ws);
  a.dq = static_cast<uint16_t*>(dq);
  a.dk = static_cast<uint16_t*>(dk);
  a.dv = static_cast<uint16_t*>(dv);
  a.sq = sq;
  a.sk = sk;
  a.scale = scale;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_bwd_dq_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, DQ_LDS);
    hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_bwd_dkv_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, DKV_LDS);
    if (e1 != hipSuccess || e2 != hipSuccess)
      JG_FAIL(JG_ERR_LAUNCH, "jg_attn_bwd: cannot reserve LDS");
    attr_set = true;
  }
  attn_bwd_dq_kernel<<<dim3((unsigned)(sq / BR), (unsigned)batch, 1), THREADS, DQ_LDS, s>>>(a);
  JG_CHECK_LAUNCH("jg_attn_bwd(dq)");
  attn_bwd_dkv_kernel<<<dim3((unsigned)(sk / BR), (unsigned)batch, 1), THREADS, DKV_LDS, s>>>(a);
  JG_CHECK_LAUNCH("jg_attn_bwd(dkv)");
  return JG_OK;
}

}  // namespace jg
