// Blockwise (flash-style) attention of one K/V chunk on the bf16 / fp16 matrix cores for head
// sizes 96 and 128, non-causal, no bias: forward (output + natural-log LSE) and backward
// from a given (global) output and LSE. Same arithmetic as the head-size-64 kernels,
// written for clarity rather than hand-scheduled: tiles of 32 keys (forward, dQ) or 32
// queries (dK/dV) pass through a double-buffered LDS stage, fetched to registers one tile
// ahead.
//
//   forward / dQ   lane = query. S^T = K Q^T (A = K rows from LDS, B = Q rows kept in
//                  registers), so the running max / sum, lse and delta of a query are
//                  scalars of the two lanes that share it. P^T (or dS^T) leaves the
//                  accumulator already in B-fragment position for O^T += V^T P^T
//                  (dQ^T += K^T dS^T): the A operand is a transposed copy of the tile in
//                  LDS whose 32 columns are stored in the order the accumulator holds its
//                  rows.
//   dK / dV        lane = key. S = Q K^T and dP = dO V^T with K, V rows in registers;
//                  lse and delta of the tile's queries are read from LDS per accumulator
//                  row; dV^T += dO^T P and dK^T += Q^T dS use transposed copies of the dO
//                  and Q tiles.
//
// Reference behaviour restated here:
//   jigsaw/modules/attention/_functional/cores/math.py:69-78   (forward)
//   jigsaw/modules/attention/_functional/cores/math.py:125-149 (backward)
#include "jg_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int WAVES = 4, THREADS = WAVES * 64;
constexpr int BQ = 32 * WAVES;  // rows (queries or keys) of a workgroup, 32 per wavefront
constexpr int BT = 32;          // rows of a streamed tile
constexpr float LOG2E = 1.4426950408889634f;

template <int D>
struct Geo {
  static constexpr int C16 = D / 16, NB = D / 32;
  static constexpr int RP = D * 2 + 16;   // bytes per row of a row-major tile (32 rows of D): an odd number of 16-byte units
  static constexpr int TP = BT * 2 + 16;  // bytes per row of a transposed tile (D rows of 32)
  static constexpr int ROWMAJ = BT * RP, TRANS = D * TP;
  static constexpr int CHUNKS = BT * D / 8;  // 16-byte pieces of a tile
  static constexpr int PER = (CHUNKS + THREADS - 1) / THREADS;
};

// Column of a transposed tile that holds tile row x: inside a group of 16 rows the order is the
// one in which an MFMA accumulator lane holds its rows, so that probabilities need no shuffle on
// their way from accumulator to B operand: 16*(x/16) + ((x%8)/4)*8 + ((x%16)/8)*4 + x%4.

template <int D>
struct TileRegs {
  u32x4 v[Geo<D>::PER];
};

// 32 rows x D of a row-major (row stride D) bf16 matrix to registers
template <int D>
__device__ __forceinline__ void tile_fetch(TileRegs<D>& r, const uint16_t* src) {
#pragma unroll
  for (int i = 0; i < Geo<D>::PER; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c < Geo<D>::CHUNKS) r.v[i] = *reinterpret_cast<const u32x4*>(src + c * 8);  // rows are contiguous: chunk c = 8 elements at c*8
  }
}
template <int D>
__device__ __forceinline__ void tile_store_rows(const TileRegs<D>& r, unsigned char* dst) {
#pragma unroll
  for (int i = 0; i < Geo<D>::PER; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c < Geo<D>::CHUNKS) {
      const int row = c / (D / 8), col8 = c % (D / 8);
      *reinterpret_cast<u32x4*>(dst + row * Geo<D>::RP + col8 * 16) = r.v[i];
    }
  }
}
// Transposed staging: a thread takes 8 rows x 2 columns of the tile (8 dwords) and writes, for each
// of its two columns, the 8 values as two 8-byte pieces of the transposed tile's row.
template <int D>
struct TransRegs {
  uint32_t w[8];
};
template <int D>
__device__ __forceinline__ void trans_fetch(TransRegs<D>& r, const uint16_t* src) {
  if (threadIdx.x < 4 * (D / 2)) {
    const int g8 = threadIdx.x / (D / 2), cp = threadIdx.x % (D / 2);
#pragma unroll
    for (int i = 0; i < 8; ++i) r.w[i] = *reinterpret_cast<const uint32_t*>(src + (g8 * 8 + i) * D + 2 * cp);
  }
}
template <int D>
__device__ __forceinline__ void trans_store(const TransRegs<D>& r, unsigned char* dst) {
  if (threadIdx.x < 4 * (D / 2)) {
    const int g8 = threadIdx.x / (D / 2), cp = threadIdx.x % (D / 2);
    // rows 8*g8 .. 8*g8+7 of the tile: the first four land at the place of row 8*g8, the last four 8 places on
    const int pos_lo = (g8 >> 1) * 16 + (g8 & 1) * 4, pos_hi = pos_lo + 8;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const uint32_t sel = e ? 0x07060302u : 0x05040100u;
      u32x2 lo, hi;
      lo.x = __builtin_amdgcn_perm(r.w[1], r.w[0], sel);
      lo.y = __builtin_amdgcn_perm(r.w[3], r.w[2], sel);
      hi.x = __builtin_amdgcn_perm(r.w[5], r.w[4], sel);
      hi.y = __builtin_amdgcn_perm(r.w[7], r.w[6], sel);
      unsigned char* row = dst + (2 * cp + e) * Geo<D>::TP;
      *reinterpret_cast<u32x2*>(row + pos_lo * 2) = lo;
      *reinterpret_cast<u32x2*>(row + pos_hi * 2) = hi;
    }
  }
}

__device__ __forceinline__ f32x16 zero16() {
  f32x16 z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.0f;
  return z;
}
// The 16-bit element type of q, k, v: bf16 or fp16. Both have a 32x32x16 MFMA with the same operand
// layout; they differ in the conversions from and to fp32.
template <bool F16>
struct Half;
template <>
struct Half<false> {
  typedef bf16x8 x8;
  __device__ static __forceinline__ f32x16 mma(x8 a, x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ uint32_t pair(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  }
  __device__ static __forceinline__ void unpair(uint32_t w, float& a, float& b) {
    a = __uint_as_float(w << 16);
    b = __uint_as_float(w & 0xffff0000u);
  }
};
template <>
struct Half<true> {
  typedef f16x8 x8;
  __device__ static __forceinline__ f32x16 mma(x8 a, x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ uint32_t pair(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
  }
  __device__ static __forceinline__ void unpair(uint32_t w, float& a, float& b) {
    const f32x2 v = __builtin_convertvector(__builtin_bit_cast(f16x2, w), f32x2);
    a = v.x;
    b = v.y;
  }
};
template <bool F16>
__device__ __forceinline__ typename Half<F16>::x8 frag(const unsigned char* at) {
  return __builtin_bit_cast(typename Half<F16>::x8, *reinterpret_cast<const u32x4*>(at));
}
template <bool F16>
__device__ __forceinline__ typename Half<F16>::x8 pack8(const float* v) {
  u32x4 r;
  r.x = Half<F16>::pair(v[0], v[1]);
  r.y = Half<F16>::pair(v[2], v[3]);
  r.z = Half<F16>::pair(v[4], v[5]);
  r.w = Half<F16>::pair(v[6], v[7]);
  return __builtin_bit_cast(typename Half<F16>::x8, r);
}
template <bool F16>
__device__ __forceinline__ u32x2 pack4(float a, float b, float c, float d) {
  u32x2 r;
  r.x = Half<F16>::pair(a, b);
  r.y = Half<F16>::pair(c, d);
  return r;
}

// Workgroup -> (batch entry, row block). Consecutive workgroup ids go to the 8 XCDs in turn; each
// XCD is given a contiguous range of (batch entry, block) pairs, so the workgroups that stream the
// same K / V (or Q / dO) share one L2. Falls back to the plain order when the count does not divide.
struct BlockOf {
  long long bh;
  int blk;
};
__device__ __forceinline__ BlockOf block_of() {
  const unsigned nblk = gridDim.x, total = gridDim.x * gridDim.y;
  unsigned id = blockIdx.y * gridDim.x + blockIdx.x;
  if ((total & 7u) == 0) id = (id & 7u) * (total >> 3) + (id >> 3);
  BlockOf b;
  b.bh = id / nblk;
  b.blk = (int)(id % nblk);
  return b;
}

struct Args {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  const uint16_t* out;   // backward: the global output
  const uint16_t* dout;  // backward
  const float* lse_in;   // backward: the global lse
  float* delta;          // backward workspace (batch, sq): written by the dQ kernel, read by the dK/dV kernel
  uint16_t* o;           // forward output, or NULL when only the merge is wanted
  float* lse;            // forward output, or NULL
  float* out_acc;        // forward: fp32 (batch, sq, d) accumulator of the ring, merged in place, or NULL
  float* lse_acc;        // forward: fp32 (batch, sq), merged in place, or NULL
  uint16_t* dq;
  uint16_t* dk;
  uint16_t* dv;
  int sq, sk;
  float scale;
};

// ------------------------------------------------------------------- forward
template <int D, bool F16>
__global__ __launch_bounds__(THREADS) void attn_wide_fwd_kernel(Args p) {
  typedef Geo<D> G;
  typedef typename Half<F16>::x8 X8;
  constexpr int BUF = G::ROWMAJ + G::TRANS;  // K rows, then V^T
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * BUF];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const BlockOf wg = block_of();
  const long long bh = wg.bh;
  const int qi = wg.blk * BQ + wave * 32 + ln;
  const uint16_t* qrow = p.q + (bh * p.sq + qi) * D;
  const uint16_t* kb = p.k + bh * p.sk * D;
  const uint16_t* vb = p.v + bh * p.sk * D;
  const float c2 = p.scale * LOG2E;

  X8 qf[G::C16];
#pragma unroll
  for (int c = 0; c < G::C16; ++c) qf[c] = frag<F16>(reinterpret_cast<const unsigned char*>(qrow + 16 * c + 8 * kg));

  f32x16 o[G::NB];
#pragma unroll
  for (int nb = 0; nb < G::NB; ++nb) o[nb] = zero16();
  float m = -INFINITY, l = 0.0f;

  TileRegs<D> rk;
  TransRegs<D> rv;
  const int ntiles = p.sk / BT;
  tile_fetch<D>(rk, kb);
  trans_fetch<D>(rv, vb);
  tile_store_rows<D>(rk, smem);
  trans_store<D>(rv, smem + G::ROWMAJ);
  // The fragments that came straight from memory are waited for here, once. Left to the first matrix
  // instruction that reads them, the wait sits inside the loop, behind the tile loads every iteration has
  // just issued, and counts those too: each iteration then waited for its own prefetch.
#pragma unroll
  for (int c = 0; c < G::C16; ++c) asm volatile("" : "+v"(qf[c]));
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const unsigned char* kt = smem + (t & 1) * BUF;
    const unsigned char* vt = kt + G::ROWMAJ;
    if (t + 1 < ntiles) {
      tile_fetch<D>(rk, kb + (long long)(t + 1) * BT * D);
      trans_fetch<D>(rv, vb + (long long)(t + 1) * BT * D);
    }
    // S^T: lane = query ln, register i = key 8*(i/4) + 4*kg + i%4 of the tile
    f32x16 s = zero16();
#pragma unroll
    for (int c = 0; c < G::C16; ++c)
      s = Half<F16>::mma(frag<F16>(kt + ln * G::RP + (16 * c + 8 * kg) * 2), qf[c], s);
    float mx = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m, mx);
    // the maximum settles after a few tiles: rescale only when some query of the wavefront saw a larger score
    if (__builtin_amdgcn_ballot_w64(mn > m) != 0) {
      const float alpha = __builtin_amdgcn_exp2f((m - mn) * c2);  // first tile: exp2(-inf) = 0
      l *= alpha;
#pragma unroll
      for (int nb = 0; nb < G::NB; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[nb][i] *= alpha;
      m = mn;
    }
    const float off = m * c2;
    float pr[16], sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      pr[i] = __builtin_amdgcn_exp2f(s[i] * c2 - off);
      sum += pr[i];
    }
    l += sum;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const X8 pf = pack8<F16>(pr + 8 * ks);
#pragma unroll
      for (int nb = 0; nb < G::NB; ++nb)
        o[nb] = Half<F16>::mma(frag<F16>(vt + (nb * 32 + ln) * G::TP + (16 * ks + 8 * kg) * 2), pf,
                                                        o[nb]);
    }
    if (t + 1 < ntiles) {
      unsigned char* nk = smem + ((t + 1) & 1) * BUF;
      tile_store_rows<D>(rk, nk);
      trans_store<D>(rv, nk + G::ROWMAJ);
    }
    __syncthreads();
  }
  // the two lanes of a query saw the same maxima; their sums cover disjoint keys
  l += __shfl_xor(l, 32, 64);
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
  const float lse_j = l > 0.0f ? m * p.scale + __logf(l) : -INFINITY;
  const long long row = bh * p.sq + qi;
  // Ring merge (the reference's _online_softmax_merge_): w = sigmoid(lse_j - lse), out += w (out_j - out),
  // lse = logaddexp(lse, lse_j), with out_j rounded to the core's output dtype first as the unfused path has it.
  float w = 0.0f;
  if (p.out_acc != nullptr) {
    const float l_old = p.lse_acc[row];  // both lanes of the query read it before lane kg = 0 writes
    w = 1.0f / (1.0f + __expf(l_old - lse_j));  // l_old = -inf -> 1
    if (kg == 0) p.lse_acc[row] = fmaxf(l_old, lse_j) + log1pf(__expf(-fabsf(l_old - lse_j)));
  }
  if (p.lse != nullptr && kg == 0) p.lse[row] = lse_j;
  // register i of block nb: output column nb*32 + 8*(i/4) + 4*kg + i%4
#pragma unroll
  for (int nb = 0; nb < G::NB; ++nb)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int dv = nb * 32 + 8 * j + 4 * kg;
      const u32x2 h = pack4<F16>(o[nb][4 * j] * inv, o[nb][4 * j + 1] * inv, o[nb][4 * j + 2] * inv, o[nb][4 * j + 3] * inv);
      if (p.o != nullptr) *reinterpret_cast<u32x2*>(p.o + row * D + dv) = h;
      if (p.out_acc != nullptr) {
        f32x4* dst = reinterpret_cast<f32x4*>(p.out_acc + row * D + dv);
        f32x4 a = *dst;
        float h0, h1, h2, h3;
        Half<F16>::unpair(h.x, h0, h1);
        Half<F16>::unpair(h.y, h2, h3);
        a.x += w * (h0 - a.x);
        a.y += w * (h1 - a.y);
        a.z += w * (h2 - a.z);
        a.w += w * (h3 - a.w);
        *dst = a;
      }
    }
}

// ------------------------------------------------------------------- dQ (and delta)
template <int D, bool F16>
__global__ __launch_bounds__(THREADS) void attn_wide_dq_kernel(Args p) {
  typedef Geo<D> G;
  typedef typename Half<F16>::x8 X8;
  constexpr int BUF = 2 * G::ROWMAJ + G::TRANS;  // K rows, V rows, K^T
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const BlockOf wg = block_of();
  const long long bh = wg.bh;
  const int qi = wg.blk * BQ + wave * 32 + ln;
  const long long qoff = (bh * p.sq + qi) * D;
  const uint16_t* kb = p.k + bh * p.sk * D;
  const uint16_t* vb = p.v + bh * p.sk * D;
  const float c2 = p.scale * LOG2E;

  X8 qf[G::C16], dof[G::C16];
  float dl = 0.0f;
#pragma unroll
  for (int c = 0; c < G::C16; ++c) {
    qf[c] = frag<F16>(reinterpret_cast<const unsigned char*>(p.q + qoff + 16 * c + 8 * kg));
    dof[c] = frag<F16>(reinterpret_cast<const unsigned char*>(p.dout + qoff + 16 * c + 8 * kg));
    const X8 of = frag<F16>(reinterpret_cast<const unsigned char*>(p.out + qoff + 16 * c + 8 * kg));
#pragma unroll
    for (int j = 0; j < 8; ++j) dl += (float)dof[c][j] * (float)of[j];
  }
  // delta = rowsum(dO o O): the two lanes of a query hold disjoint halves of the row
  const float delta = dl + __shfl_xor(dl, 32, 64);
  if (kg == 0) p.delta[bh * p.sq + qi] = delta;
  const float lse2 = p.lse_in[bh * p.sq + qi] * LOG2E;

  f32x16 dq[G::NB];
#pragma unroll
  for (int nb = 0; nb < G::NB; ++nb) dq[nb] = zero16();

  TileRegs<D> rk, rv;
  TransRegs<D> rkt;
  const int ntiles = p.sk / BT;
  tile_fetch<D>(rk, kb);
  tile_fetch<D>(rv, vb);
  trans_fetch<D>(rkt, kb);
  tile_store_rows<D>(rk, smem);
  tile_store_rows<D>(rv, smem + G::ROWMAJ);
  trans_store<D>(rkt, smem + 2 * G::ROWMAJ);
  // The fragments that came straight from memory are waited for here, once. Left to the first matrix
  // instruction that reads them, the wait sits inside the loop, behind the tile loads every iteration has
  // just issued, and counts those too: each iteration then waited for its own prefetch.
#pragma unroll
  for (int c = 0; c < G::C16; ++c) asm volatile("" : "+v"(qf[c]), "+v"(dof[c]));
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const unsigned char* kt = smem + (t & 1) * BUF;
    const unsigned char* vt = kt + G::ROWMAJ;
    const unsigned char* ktt = kt + 2 * G::ROWMAJ;
    if (t + 1 < ntiles) {
      tile_fetch<D>(rk, kb + (long long)(t + 1) * BT * D);
      tile_fetch<D>(rv, vb + (long long)(t + 1) * BT * D);
      trans_fetch<D>(rkt, kb + (long long)(t + 1) * BT * D);
    }
    f32x16 s = zero16(), dp = zero16();
#pragma unroll
    for (int c = 0; c < G::C16; ++c) {
      s = Half<F16>::mma(frag<F16>(kt + ln * G::RP + (16 * c + 8 * kg) * 2), qf[c], s);
      dp = Half<F16>::mma(frag<F16>(vt + ln * G::RP + (16 * c + 8 * kg) * 2), dof[c], dp);
    }
    float ds[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) ds[i] = __builtin_amdgcn_exp2f(s[i] * c2 - lse2) * (dp[i] - delta);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const X8 dsf = pack8<F16>(ds + 8 * ks);
#pragma unroll
      for (int nb = 0; nb < G::NB; ++nb)
        dq[nb] = Half<F16>::mma(frag<F16>(ktt + (nb * 32 + ln) * G::TP + (16 * ks + 8 * kg) * 2),
                                                         dsf, dq[nb]);
    }
    if (t + 1 < ntiles) {
      unsigned char* nk = smem + ((t + 1) & 1) * BUF;
      tile_store_rows<D>(rk, nk);
      tile_store_rows<D>(rv, nk + G::ROWMAJ);
      trans_store<D>(rkt, nk + 2 * G::ROWMAJ);
    }
    __syncthreads();
  }
  uint16_t* row = p.dq + qoff;
#pragma unroll
  for (int nb = 0; nb < G::NB; ++nb)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      *reinterpret_cast<u32x2*>(row + nb * 32 + 8 * j + 4 * kg) =
          pack4<F16>(dq[nb][4 * j] * p.scale, dq[nb][4 * j + 1] * p.scale, dq[nb][4 * j + 2] * p.scale,
                dq[nb][4 * j + 3] * p.scale);
}

// ------------------------------------------------------------------- dK, dV
// MODE 0 forms dK and dV in one pass (two d x 32 accumulators a wavefront). That fits two workgroups
// per CU in 256 registers a lane at head size 96 but not at 128 (it would spill, and ran 1.3x slower
// that way), so head size 128 runs the kernel twice: MODE 1 forms dV only (from P), MODE 2 dK only
// (from dS), each with one accumulator and two workgroups per CU; the scores are computed in both.
// A launch with no more workgroups than CUs gains nothing from that and keeps the single pass.
template <int D, bool F16, int MODE>
__global__ __launch_bounds__(THREADS, (D <= 96 || MODE != 0) ? 2 : 1) void attn_wide_dkv_kernel(Args p) {
  typedef Geo<D> G;
  typedef typename Half<F16>::x8 X8;
  constexpr bool DV = MODE != 2, DK = MODE != 1;
  constexpr int STATS = 2 * BT * 4;                           // lse * log2(e) and delta of the tile's queries
  constexpr int BUF = 2 * G::ROWMAJ + 2 * G::TRANS + STATS;   // Q rows, dO rows, Q^T, dO^T, stats
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const BlockOf wg = block_of();
  const long long bh = wg.bh;
  const int ki = wg.blk * BQ + wave * 32 + ln;
  const long long koff = (bh * p.sk + ki) * D;
  const uint16_t* qb = p.q + bh * p.sq * D;
  const uint16_t* gb = p.dout + bh * p.sq * D;
  const float* lb = p.lse_in + bh * p.sq;
  const float* db = p.delta + bh * p.sq;
  const float c2 = p.scale * LOG2E;

  X8 kf[G::C16], vf[DK ? G::C16 : 1];
#pragma unroll
  for (int c = 0; c < G::C16; ++c) {
    kf[c] = frag<F16>(reinterpret_cast<const unsigned char*>(p.k + koff + 16 * c + 8 * kg));
    if (DK) vf[c] = frag<F16>(reinterpret_cast<const unsigned char*>(p.v + koff + 16 * c + 8 * kg));
  }
  f32x16 dk[DK ? G::NB : 1], dv[DV ? G::NB : 1];
#pragma unroll
  for (int nb = 0; nb < G::NB; ++nb) {
    if (DK) dk[nb] = zero16();
    if (DV) dv[nb] = zero16();
  }

  TileRegs<D> rq, rg;        // Q rows (scores); dO rows (dP: dK only)
  TransRegs<D> rqt, rgt;     // Q^T (dK only); dO^T (dV only)
  float st = 0.0f;  // one statistic per thread of the first wavefront: lse2 (lanes 0-31) or delta (32-63)
  const int ntiles = p.sq / BT;
  auto fetch = [&](int t) {
    tile_fetch<D>(rq, qb + (long long)t * BT * D);
    if (DK) tile_fetch<D>(rg, gb + (long long)t * BT * D);
    if (DK) trans_fetch<D>(rqt, qb + (long long)t * BT * D);
    if (DV) trans_fetch<D>(rgt, gb + (long long)t * BT * D);
    if (threadIdx.x < 2 * BT) {
      const float* src = threadIdx.x < BT ? lb : db;  // every lane loads; the factor is applied when stored
      st = src[t * BT + (threadIdx.x & (BT - 1))];
    }
  };
  auto store = [&](int buf) {
    unsigned char* base = smem + buf * BUF;
    tile_store_rows<D>(rq, base);
    if (DK) tile_store_rows<D>(rg, base + G::ROWMAJ);
    if (DK) trans_store<D>(rqt, base + 2 * G::ROWMAJ);
    if (DV) trans_store<D>(rgt, base + 2 * G::ROWMAJ + G::TRANS);
    if (threadIdx.x < 2 * BT)
      reinterpret_cast<float*>(base + 2 * G::ROWMAJ + 2 * G::TRANS)[threadIdx.x] = threadIdx.x < BT ? st * LOG2E : st;
  };
  fetch(0);
  store(0);
  // The fragments that came straight from memory are waited for here, once. Left to the first matrix
  // instruction that reads them, the wait sits inside the loop, behind the tile loads every iteration has
  // just issued, and counts those too: each iteration then waited for its own prefetch.
#pragma unroll
  for (int c = 0; c < G::C16; ++c) {
    asm volatile("" : "+v"(kf[c]));
    if (DK) asm volatile("" : "+v"(vf[c]));
  }
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const unsigned char* qt = smem + (t & 1) * BUF;
    const unsigned char* gt = qt + G::ROWMAJ;
    const unsigned char* qtt = qt + 2 * G::ROWMAJ;
    const unsigned char* gtt = qtt + G::TRANS;
    const float* stats = reinterpret_cast<const float*>(gtt + G::TRANS);
    if (t + 1 < ntiles) fetch(t + 1);
    // S and dP: lane = key ln, register i = query 8*(i/4) + 4*kg + i%4 of the tile
    f32x16 s = zero16(), dp = zero16();
#pragma unroll
    for (int c = 0; c < G::C16; ++c) {
      s = Half<F16>::mma(frag<F16>(qt + ln * G::RP + (16 * c + 8 * kg) * 2), kf[c], s);
      if (DK) dp = Half<F16>::mma(frag<F16>(gt + ln * G::RP + (16 * c + 8 * kg) * 2), vf[c], dp);
    }
    float pr[16], ds[16];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const f32x4 l4 = *reinterpret_cast<const f32x4*>(stats + 8 * j + 4 * kg);
      f32x4 d4 = {0.0f, 0.0f, 0.0f, 0.0f};
      if (DK) d4 = *reinterpret_cast<const f32x4*>(stats + BT + 8 * j + 4 * kg);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 4 * j + e;
        pr[i] = __builtin_amdgcn_exp2f(s[i] * c2 - l4[e]);
        ds[i] = pr[i] * (dp[i] - d4[e]);
      }
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      if (DV) {
        const X8 pf = pack8<F16>(pr + 8 * ks);
#pragma unroll
        for (int nb = 0; nb < G::NB; ++nb)
          dv[nb] = Half<F16>::mma(frag<F16>(gtt + (nb * 32 + ln) * G::TP + (16 * ks + 8 * kg) * 2), pf, dv[nb]);
      }
      if (DK) {
        const X8 dsf = pack8<F16>(ds + 8 * ks);
#pragma unroll
        for (int nb = 0; nb < G::NB; ++nb)
          dk[nb] = Half<F16>::mma(frag<F16>(qtt + (nb * 32 + ln) * G::TP + (16 * ks + 8 * kg) * 2), dsf, dk[nb]);
      }
    }
    if (t + 1 < ntiles) store((t + 1) & 1);
    __syncthreads();
  }
  uint16_t* krow = p.dk + koff;
  uint16_t* vrow = p.dv + koff;
#pragma unroll
  for (int nb = 0; nb < G::NB; ++nb)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (DK)
        *reinterpret_cast<u32x2*>(krow + nb * 32 + 8 * j + 4 * kg) =
            pack4<F16>(dk[nb][4 * j] * p.scale, dk[nb][4 * j + 1] * p.scale, dk[nb][4 * j + 2] * p.scale,
                       dk[nb][4 * j + 3] * p.scale);
      if (DV)
        *reinterpret_cast<u32x2*>(vrow + nb * 32 + 8 * j + 4 * kg) =
            pack4<F16>(dv[nb][4 * j], dv[nb][4 * j + 1], dv[nb][4 * j + 2], dv[nb][4 * j + 3]);
    }
}

int cu_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;
  }
  return cus;
}

template <int D, bool F16>
int launch_fwd(const Args& a, long long batch, hipStream_t s) {
  attn_wide_fwd_kernel<D, F16><<<dim3((unsigned)(a.sq / BQ), (unsigned)batch, 1), THREADS, 0, s>>>(a);
  JG_CHECK_LAUNCH("jg_attn_fwd(wide)");
  return JG_OK;
}

template <int D, bool F16>
int launch_bwd(const Args& a, long long batch, hipStream_t s) {
  typedef Geo<D> G;
  constexpr int DQ_LDS = 2 * (2 * G::ROWMAJ + G::TRANS);
  constexpr int DKV_LDS = 2 * (2 * G::ROWMAJ + 2 * G::TRANS + 2 * BT * 4);
  void (*dqk)(Args) = &attn_wide_dq_kernel<D, F16>;
  hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(dqk), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      DQ_LDS);
  if (e1 != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "jg_attn_bwd(wide): cannot reserve LDS");
  dqk<<<dim3((unsigned)(a.sq / BQ), (unsigned)batch, 1), THREADS, DQ_LDS, s>>>(a);
  JG_CHECK_LAUNCH("jg_attn_bwd(wide, dq)");
  // head size 96: dK and dV in one pass; head size 128: one pass each when the launch has more
  // workgroups than the chip has CUs (register budget, see the kernel)
  void (*passes[2])(Args) = {&attn_wide_dkv_kernel<D, F16, 0>, nullptr};
  if constexpr (D > 96) {
    if ((long long)(a.sk / BQ) * batch > cu_count()) {
      passes[0] = &attn_wide_dkv_kernel<D, F16, 1>;
      passes[1] = &attn_wide_dkv_kernel<D, F16, 2>;
    }
  }
  for (int i = 0; i < 2 && passes[i] != nullptr; ++i) {
    hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(passes[i]),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, DKV_LDS);
    if (e2 != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "jg_attn_bwd(wide): cannot reserve LDS");
    passes[i]<<<dim3((unsigned)(a.sk / BQ), (unsigned)batch, 1), THREADS, DKV_LDS, s>>>(a);
    JG_CHECK_LAUNCH("jg_attn_bwd(wide, dkv)");
  }
  return JG_OK;
}

}  // namespace

namespace jg {

bool attn_wide_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias) {
  return (dtype == JG_BF16 || dtype == JG_F16) && !has_bias && (d == 96 || d == 128) && sq > 0 && sk > 0 && sq % BQ == 0 &&
         sk % BQ == 0 && batch > 0 && batch <= 65535;
}

int attn_wide_fwd(void* out, float* lse, const void* q, const void* k, const void* v, long long batch, int sq,
                  int sk, int d, int dtype, float scale, float* out_acc, float* lse_acc, hipStream_t s) {
  Args a{};
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k);
  a.v = static_cast<const uint16_t*>(v);
  a.o = static_cast<uint16_t*>(out);
  a.lse = lse;
  a.out_acc = out_acc;
  a.lse_acc = lse_acc;
  a.sq = sq; a.sk = sk; a.scale = scale;
  if (dtype == JG_F16) return d == 128 ? launch_fwd<128, true>(a, batch, s) : launch_fwd<96, true>(a, batch, s);
  return d == 128 ? launch_fwd<128, false>(a, batch, s) : launch_fwd<96, false>(a, batch, s);
}

int attn_wide_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q, const void* k, const void* v,
                  const void* out, const float* lse, long long batch, int sq, int sk, int d, int dtype,
                  float scale, void* ws, hipStream_t s) {
  Args a{};
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k);
  a.v = static_cast<const uint16_t*>(v);
  a.out = static_cast<const uint16_t*>(out);
  a.dout = static_cast<const uint16_t*>(dout);
  a.lse_in = lse;
  a.delta = static_cast<float*>(ws);
  a.dq = static_cast<uint16_t*>(dq);
  a.dk = static_cast<uint16_t*>(dk);
  a.dv = static_cast<uint16_t*>(dv);
  a.sq = sq; a.sk = sk; a.scale = scale;
  if (dtype == JG_F16) return d == 128 ? launch_bwd<128, true>(a, batch, s) : launch_bwd<96, true>(a, batch, s);
  return d == 128 ? launch_bwd<128, false>(a, batch, s) : launch_bwd<96, false>(a, batch, s);
}

}  // namespace jg
