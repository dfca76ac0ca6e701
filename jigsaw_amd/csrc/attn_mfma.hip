// Blockwise (flash-style) attention of one K/V chunk on the bf16 matrix cores,
// head size 64, non-causal, with the ring's log-sum-exp merge fused into the
// epilogue. Forward kernel.
//
//   S^T = K Q^T      MFMA 32x32x16: A = K rows (32 keys x 16 d, from LDS), B = Q rows
//                    (16 d x 32 queries, in registers for the whole kernel). An
//                    accumulator lane owns ONE query and 16 of the 32 keys, so the
//                    running max / sum of the online softmax are per-lane scalars (one
//                    exchange per step between the two lanes that share a query).
//   O^T = V^T P^T    A = V^T (32 dv x 16 keys), B = P^T: the probabilities of a lane are
//                    already in B-fragment position (the 16 keys of a K-step are taken
//                    in the order the accumulator holds them), so P never leaves
//                    registers. V stays row-major in LDS; its transposed fragments come
//                    from the LDS transpose read (ds_read_b64_tr_b16: within 16 lanes,
//                    lane i receives element i % 4 of the 8 bytes lanes i / 4 + 4 j
//                    point at, j = 0..3), two reads of 4 consecutive keys per fragment.
//   Tiles            K and V tiles (32 keys x 128 bytes) travel from memory straight into
//                    LDS (global_load_lds, 16 bytes per lane, no registers, no vector
//                    instructions); the 16-byte chunks of a row are XOR-swizzled with
//                    row % 8 by choosing which chunk a lane fetches. Four buffers per key
//                    quarter, filled three tiles ahead. The fragment addresses are per-lane
//                    constants: the loop spends its vector instructions on the softmax.
//   Operand reuse    every MFMA takes one fragment from LDS (1 KB per wavefront), so a
//                    wavefront with one query block asks LDS for 128 bytes per cycle
//                    and compute unit at full matrix-core rate. Each wavefront therefore
//                    owns TWO query blocks (64 queries): a K or V^T fragment is read once
//                    and feeds two MFMAs.
//   Workgroup        512 threads = 8 wavefronts = 2 query groups (64 queries) x 4 key
//                    quarters; the quarters are combined through LDS at the end. The two
//                    query blocks of a wavefront are half a step apart: while the softmax
//                    of one runs on the vector unit, the scores of the other and the P V
//                    products of the previous one run on the matrix core. The kernel is
//                    bound by the vector unit (about 90 instruction slots per query block
//                    and step against 64 for its 8 MFMAs).
//   Epilogue         out_j = O / l (bf16), lse_j = m*scale + ln l; optionally merged
//                    in place into the ring's fp32 accumulator:
//                    w = sigmoid(lse_j - lse), out += w (out_j - out), lse = logaddexp.
//                    The result tile goes through LDS so that all 512 threads move the
//                    workgroup's contiguous 32 KB of the accumulator in 16-byte pieces.
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
constexpr int BN = 32;            // keys per tile
constexpr int NQ = 4;             // key quarters
constexpr int NBUF = 4;           // tile buffers per quarter
constexpr int THREADS = 512;
constexpr int ROWB = 128;         // bytes per K / V row: 64 bf16, chunks XOR-swizzled, no padding
constexpr int KV_BYTES = BN * ROWB;            // 4096: one K or V tile
constexpr int TILE_BYTES = 2 * KV_BYTES;       // K tile, then V tile
constexpr int QUARTER_BYTES = NBUF * TILE_BYTES;
constexpr int LDS_BYTES = NQ * QUARTER_BYTES;  // 131072
// The reference score of a query follows its running max lazily: it moves only when a tile's
// max lies more than this many powers of two (after scaling) above it. Probabilities then reach 2^8 at most
// (fp32 sums and accumulators, bf16 keeps its relative precision), and the rescale of the
// state, which a per-tile max would trigger in almost every tile of a 64-lane wavefront
// (some query of 32 sees a new max), becomes the rare branch it is meant to be.
constexpr float RESCALE_ABOVE = 8.0f;
constexpr int XO_FLOATS = 68 * 64;             // hand-over of one wavefront: 64 O registers + m, l per query block
constexpr int STAGE_PITCH = 68;                // floats per query row of the staged result (64 + 4: 16-byte rows 4 banks apart)
static_assert(4 * XO_FLOATS * 4 <= LDS_BYTES, "the hand-over slots reuse the tile buffers");
static_assert((BM * STAGE_PITCH + BM) * 4 <= LDS_BYTES, "the staged result reuses the tile buffers");

typedef short i16x4 __attribute__((ext_vector_type(4)));

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

// The values of a lane and of lane ^ 32 (in an order that depends on the lane's half): a
// register swap instead of an LDS round trip. Callers combine the two symmetrically.
__device__ __forceinline__ void pair32(float v, float& a, float& b) {
  const uint32_t bits = __float_as_uint(v);
  const auto sw = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
  a = __uint_as_float(sw[0]);
  b = __uint_as_float(sw[1]);
}

// Workgroup -> (batch entry, row block). Consecutive workgroup ids go to the 8 XCDs in turn; each
// XCD is given a contiguous range of (batch entry, block) pairs, so the workgroups that stream the
// same K / V (or Q / dO) share one L2 instead of every L2 holding every head. Falls back to the
// plain order when the count does not divide.
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

__global__ __launch_bounds__(THREADS) void attn_fwd_mfma_kernel(FwdArgs p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int qg = wave & 1, kq = wave >> 1;
  const BlockOf where = block_of();
  const long long b = where.bh;
  const int q0 = where.blk * BM + qg * 64;
  const int kquarter = p.sk >> 2;
  const int ntiles = kquarter / BN;
  const float c2 = p.scale * 1.4426950408889634f;  // scores are handled in base 2

  unsigned char* lds = smem + kq * QUARTER_BYTES;

  // Q fragments of this wavefront's 2 x 32 queries (B operand of S^T = K Q^T)
  bf16x8 qf[2][4];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const uint16_t* qrow = p.q + (b * p.sq + q0 + qb * 32 + ln) * D + 8 * kg;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      qf[qb][c] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(qrow + 16 * c));
  }

  // ---- tiles: memory -> LDS directly. One instruction of a wavefront lands 64 x 16 bytes
  // contiguously in lane order = 8 rows; lane L sits at row L / 8, chunk position L % 8 and
  // fetches the chunk (L % 8) ^ (row % 8) of its row. A wavefront moves rows 16 qg .. 16 qg + 15
  // of the K tile and of the V tile (two instructions each).
  // The transfer is written in assembly: a wave-uniform 64-bit base in scalar registers (tile
  // and row block, advanced with scalar arithmetic), the lane's constant 32-bit offset, and the
  // LDS address of the 1 KB block in M0, so that issuing a tile costs no vector instruction.
  // (It also keeps the compiler from putting a wait for ALL outstanding transfers in front of
  // every LDS read, which is how it orders LDS reads against transfers it knows about. The
  // kernel orders them itself: a buffer is read only after the wait + barrier that follows its
  // transfer, and refilled only after the barrier that follows its last read.)
  const uint32_t dma_off = (uint32_t)((lane >> 3) * ROWB + (((lane & 7) ^ (lane >> 3)) << 4));
  const int qg_u = __builtin_amdgcn_readfirstlane(qg), kq_u = __builtin_amdgcn_readfirstlane(kq);
  const char* kdma = reinterpret_cast<const char*>(p.k + (b * p.sk + (long long)kq_u * kquarter) * D) + 16 * qg_u * ROWB;
  const char* vdma = reinterpret_cast<const char*>(p.v + (b * p.sk + (long long)kq_u * kquarter) * D) + 16 * qg_u * ROWB;
  typedef __attribute__((address_space(3))) unsigned char* lds_bytes;
  const uint32_t lds_dma = (uint32_t)(uintptr_t)((lds_bytes)smem) + (uint32_t)(kq_u * QUARTER_BYTES + 16 * qg_u * ROWB);
  auto dma_1k = [&](const char* src, uint32_t dst) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(dma_off), "s"(src), "s"(dst) : "m0");
  };
  auto dma_tile = [&](int t, int buf) {
    const long long off = (long long)t * KV_BYTES;
    const uint32_t dst = lds_dma + (uint32_t)(buf * TILE_BYTES);
    dma_1k(kdma + off, dst);
    dma_1k(kdma + off + 8 * ROWB, dst + 8 * ROWB);
    dma_1k(vdma + off, dst + KV_BYTES);
    dma_1k(vdma + off + 8 * ROWB, dst + KV_BYTES + 8 * ROWB);
  };
  // per-lane constant parts of the fragment addresses
  //   K fragment c of key row ln: logical chunk 2 c + kg, stored at chunk (2 c + kg) ^ (ln % 8)
  int kaddr[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) kaddr[c] = ln * ROWB + (((2 * c + kg) ^ (ln & 7)) << 4);
  //   V^T fragment (dv block nb, K-step tt) = two transpose reads (r = 0, 1) of the 4 keys
  //   16 tt + 8 r + 4 kg + 0..3: lane p of a group of 16 points at key row +p / 4, dv 32 nb +
  //   16 (group % 2) + 4 (p % 4); the row's swizzle is (4 kg + p / 4), the same for every (tt, r)
  int vaddr[2];
  {
    const int pp = lane & 15, g1 = (lane >> 4) & 1;
    const int rsw = 4 * kg + (pp >> 2);
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
      vaddr[nb] = rsw * ROWB + (((4 * nb + 2 * g1 + ((pp & 3) >> 1)) ^ rsw) << 4) + 8 * (pp & 1);
  }

  f32x16 o[2][2];  // [query block][dv block] O^T: lane = query, register i = dv nb*32 + 8*(i/4) + 4*kg + i%4
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[qb][nb][i] = 0.0f;
  float m[2] = {-INFINITY, -INFINITY};  // reference score of the lane's query (both lanes of a query agree)
  float l[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};  // running sums (two chains) of the probabilities of the lane's OWN 16 keys per block

  f32x16 s[2];       // scores of the two query blocks (half a step apart)
  u32x4 kf[4];       // K fragments of the tile whose scores are being formed
  bf16x8 vf[2][2];   // V^T fragments [dv block][K-step] of the tile whose P V products are being formed
  bf16x8 pk[2][2];   // probabilities [query block][K-step], bf16, in B-fragment position

  auto load_kf = [&](int buf) {
    const unsigned char* kt = lds + buf * TILE_BYTES;
#pragma unroll
    for (int c = 0; c < 4; ++c) kf[c] = *reinterpret_cast<const u32x4*>(kt + kaddr[c]);
  };
  auto load_vf = [&](int buf) {
    const unsigned char* vt = lds + buf * TILE_BYTES + KV_BYTES;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        typedef __attribute__((address_space(3))) i16x4* tr_ptr;
        const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(vt + vaddr[nb] + (16 * tt) * ROWB));
        const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(vt + vaddr[nb] + (16 * tt + 8) * ROWB));
        u32x4 w;
        w.x = __builtin_bit_cast(u32x2, lo).x;
        w.y = __builtin_bit_cast(u32x2, lo).y;
        w.z = __builtin_bit_cast(u32x2, hi).x;
        w.w = __builtin_bit_cast(u32x2, hi).y;
        vf[nb][tt] = __builtin_bit_cast(bf16x8, w);
      }
  };
  // Online softmax of the 32 x 32 score block of one query block, in two parts. First the
  // reference: when some lane of the wavefront sees a score more than RESCALE_ABOVE powers of
  // two over its reference (a rarely taken, wave-uniform branch; the first tile always takes
  // it, its reference being -inf) the two lanes of each query agree on the tile's max, the
  // reference moves there and the state is rescaled. Then probabilities and partial row
  // sums: straight-line vector work that is interleaved with the matrix-core instructions
  // of the other query block.
  const float slack = RESCALE_ABOVE / c2;  // in score units
  auto new_max = [&](int qb) {
    // (written as instructions: fmaxf() would first quieten each operand, one more instruction each)
    auto max3 = [](float a, float b, float c) {
      float r;
      asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
      return r;
    };
    const f32x16& sc = s[qb];
    const float t0 = max3(sc[0], sc[1], sc[2]), t1 = max3(sc[3], sc[4], sc[5]), t2 = max3(sc[6], sc[7], sc[8]);
    const float t3 = max3(sc[9], sc[10], sc[11]), t4 = max3(sc[12], sc[13], sc[14]);
    const float mx = max3(max3(t0, t1, t2), max3(t3, t4, sc[15]), sc[15]);  // of the lane's own 16 keys
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx > m[qb] + slack) != 0, 0)) {
      float pa, pb;
      pair32(mx, pa, pb);
      const float mq = max3(pa, pb, pb);  // largest score of the query in this tile
      if (mq > m[qb] + slack) {           // the same decision in both lanes of the query
        const float alpha = __builtin_amdgcn_exp2f((m[qb] - mq) * c2);  // 0 for the first tile
        l[qb][0] *= alpha;
        l[qb][1] *= alpha;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[qb][nb][i] *= alpha;
        m[qb] = mq;
      }
    }
  };
  // Probabilities of score pair j (0..7) of a query block: two multiply-adds (scale, minus the
  // reference), two exponentials, two additions for
  // the row sum (two chains), one rounding of the pair to bf16. (The dot-product instructions
  // would add a pair in one instruction, but they do not run beside the matrix core's work.)
  auto prob_pair = [&](int qb, int j) {
    const float mc = m[qb] * c2;
    const f32x2 v2 = {__builtin_amdgcn_exp2f(s[qb][2 * j] * c2 - mc), __builtin_amdgcn_exp2f(s[qb][2 * j + 1] * c2 - mc)};
    l[qb][0] += v2.x;
    l[qb][1] += v2.y;
    const bf16x2 h2 = __builtin_convertvector(v2, bf16x2);
    pk[qb][j >> 2][2 * (j & 3)] = h2.x;
    pk[qb][j >> 2][2 * (j & 3) + 1] = h2.y;
  };
  auto pv_one = [&](int qb, int nb, int tt) {
    o[qb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[nb][tt], pk[qb][tt], o[qb][nb], 0, 0, 0);
  };
  // score instruction i (0..3) of a query block
  auto score_one = [&](int qb, int i) {
    if (i == 0) {
      f32x16 z;
#pragma unroll
      for (int r = 0; r < 16; ++r) z[r] = 0.0f;
      s[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[0]), qf[qb][0], z, 0, 0, 0);
    } else {
      s[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[i]), qf[qb][i], s[qb], 0, 0, 0);
    }
  };
  // The probabilities are wanted HERE (a use the optimiser cannot move): without it their
  // computation sinks to the block of the MFMAs that consume them, behind the next branch.
  auto pin = [](const bf16x8& a, const bf16x8& b2_) { asm volatile("" : : "v"(a), "v"(b2_)); };
  // ---- software pipeline over the 32-key tiles, four LDS buffers per key quarter. In
  // iteration t the scores of query block 1 (tile t) and the P V products of query block 1
  // (tile t-1) run under the softmax of query block 0 (tile t); the P V products of query
  // block 0 (tile t) and its scores of tile t+1 run under the softmax of query block 1.
  // The transfer of tile t+3 is issued first, into the buffer tile t-1 has left. Past the
  // last tile the same instructions run on clamped tile indices and their results are
  // dropped, which keeps the loop body free of branches apart from the rare rescale.
  const int last = ntiles - 1;
  dma_tile(0, 0);
  dma_tile(last < 1 ? last : 1, 1);
  dma_tile(last < 2 ? last : 2, 2);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  __syncthreads();
  load_kf(0);
#pragma unroll
  for (int i = 0; i < 4; ++i) score_one(0, i);
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pk[1][tt][i] = (__bf16)0.0f;  // the first "previous" P V adds nothing
      vf[0][tt][i] = (__bf16)0.0f;
      vf[1][tt][i] = (__bf16)0.0f;
    }

#define JG_FENCE() __builtin_amdgcn_sched_barrier(0)
  // One half of an iteration: query block `qa` has its scores ready and gets its softmax; the
  // matrix core meanwhile forms the next scores of the other query block `qo` and then finishes
  // that block's P V products of the tile before. One MFMA, then one pair of probabilities,
  // and so on; the fences pin that order. The scores go first so that they are complete long
  // before the next half reads them (an MFMA chain of one wavefront shares the matrix core
  // with the other wavefront of the SIMD, so its last result arrives late); the two MFMAs in
  // front of the max are work for the matrix core while the vector unit runs the max tree.
  auto half = [&](int qa, int qo, auto&& after_scores, auto&& after_pv) {
    score_one(qo, 0);
    score_one(qo, 1);
    JG_FENCE();
    new_max(qa);
    JG_FENCE();
#pragma unroll
    for (int i = 2; i < 4; ++i) {
      score_one(qo, i);
      JG_FENCE();
      prob_pair(qa, i - 2);
      JG_FENCE();
    }
    after_scores();  // the K fragments are free
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pv_one(qo, i & 1, i >> 1);
      JG_FENCE();
      prob_pair(qa, 2 + i);
      JG_FENCE();
    }
    after_pv();  // the V^T fragments are free
    prob_pair(qa, 6);
    prob_pair(qa, 7);
    pin(pk[qa][0], pk[qa][1]);
    JG_FENCE();
  };
  auto iteration = [&](int t, int cur, int nxt, int tgt) {
    dma_tile(t + 3 < last ? t + 3 : last, tgt);
    // softmax of query block 0 (tile t) under: scores of block 1 (tile t), P V of block 1 (tile t-1)
    half(0, 1, [&]() { load_kf(nxt); }, [&]() { load_vf(cur); });
    // softmax of query block 1 (tile t) under: scores of block 0 (tile t+1), P V of block 0 (tile t)
    half(1, 0, [&]() {}, [&]() {});
    __builtin_amdgcn_s_waitcnt(0x0F74);  // vmcnt(4): every transfer but this iteration's has landed
    __syncthreads();
  };
  // (unrolling over the four buffers would turn every LDS address into an immediate, but the
  // longer code ran no faster)
  for (int t = 0; t < ntiles; ++t) iteration(t, t & 3, (t + 1) & 3, (t + 3) & 3);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the clamped transfers of the last iterations still target LDS
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) pv_one(1, nb, tt);  // last tile, query block 1

  // ---- the two lanes of a query add their partial sums; the four key quarters combine via LDS
  // (quarters 1 and 3 hand over to 0 and 2, then 2 to 0)
  float lt[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    float pa, pb;
    pair32(l[qb][0] + l[qb][1], pa, pb);
    lt[qb] = pa + pb;
  }
  float* xo_base = reinterpret_cast<float*>(smem);
  auto hand_over = [&](int slot) {
    float* xo = xo_base + slot * XO_FLOATS;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) xo[((qb * 2 + nb) * 16 + i) * 64 + lane] = o[qb][nb][i];
      xo[(64 + qb) * 64 + lane] = m[qb];
      xo[(66 + qb) * 64 + lane] = lt[qb];
    }
  };
  auto take_over = [&](int slot) {
    const float* xo = xo_base + slot * XO_FLOATS;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const float m1 = xo[(64 + qb) * 64 + lane], l1 = xo[(66 + qb) * 64 + lane];
      const float mn = fmaxf(m[qb], m1);
      const float a0 = __builtin_amdgcn_exp2f((m[qb] - mn) * c2), a1 = __builtin_amdgcn_exp2f((m1 - mn) * c2);
      lt[qb] = lt[qb] * a0 + l1 * a1;
      m[qb] = mn;
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          o[qb][nb][i] = o[qb][nb][i] * a0 + xo[((qb * 2 + nb) * 16 + i) * 64 + lane] * a1;
    }
  };
  __syncthreads();  // every wavefront is past its last LDS read and its last transfer
  if (kq & 1) hand_over((kq >> 1) * 2 + qg);
  __syncthreads();
  if (!(kq & 1)) take_over((kq >> 1) * 2 + qg);
  __syncthreads();
  if (kq == 2) hand_over(qg);
  __syncthreads();
  if (kq == 0) take_over(qg);
  __syncthreads();

  // ---- epilogue: the two wavefronts that hold the result normalise it and stage it in LDS
  // as [query][dv] fp32 (already rounded to the core's output dtype) with the merge weight of
  // each query; then all 512 threads write and / or merge the workgroup's contiguous block
  float* stage = reinterpret_cast<float*>(smem);
  float* stage_w = stage + BM * STAGE_PITCH;
  if (kq == 0) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const float inv = 1.0f / lt[qb];
      const float lse_j = (m[qb] * c2 + log2f(lt[qb])) * 0.6931471805599453f;  // natural log
      const int ql = qg * 64 + qb * 32 + ln;  // query inside the workgroup
      const long long qi = b * p.sq + where.blk * BM + ql;
      if (kg == 0) {
        float w = 0.0f;
        if (p.out_acc != nullptr) {
          const float l_old = p.lse_acc[qi];
          w = 1.0f / (1.0f + __expf(l_old - lse_j));  // sigmoid(lse_j - l_old); l_old = -inf -> 1
          const float mxl = fmaxf(l_old, lse_j);
          p.lse_acc[qi] = mxl + log1pf(__expf(-fabsf(l_old - lse_j)));
        }
        stage_w[ql] = w;
        if (p.lse != nullptr) p.lse[qi] = lse_j;
      }
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int dv = nb * 32 + 8 * j + 4 * kg;
          f32x4 val = {o[qb][nb][4 * j] * inv, o[qb][nb][4 * j + 1] * inv, o[qb][nb][4 * j + 2] * inv,
                       o[qb][nb][4 * j + 3] * inv};
          const bf16x4 h = __builtin_convertvector(val, bf16x4);  // the core's output dtype
          *reinterpret_cast<f32x4*>(stage + ql * STAGE_PITCH + dv) = __builtin_convertvector(h, f32x4);
        }
    }
  }
  __syncthreads();
  {
    const long long row0 = b * p.sq + (long long)where.blk * BM;
    f32x4 hv[4], acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {  // piece e = tid + 512 i of the 128 x 16 pieces of 4 floats
      const int e = tid + THREADS * i;
      hv[i] = *reinterpret_cast<const f32x4*>(stage + (e >> 4) * STAGE_PITCH + 4 * (e & 15));
      if (p.out_acc != nullptr) acc[i] = *reinterpret_cast<const f32x4*>(p.out_acc + row0 * D + 4 * (long long)e);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + THREADS * i;
      if (p.out != nullptr)
        *reinterpret_cast<bf16x4*>(p.out + row0 * D + 4 * (long long)e) = __builtin_convertvector(hv[i], bf16x4);
      if (p.out_acc != nullptr) {
        const float w = stage_w[e >> 4];
        f32x4 a = acc[i];
        a.x += w * (hv[i].x - a.x);
        a.y += w * (hv[i].y - a.y);
        a.z += w * (hv[i].z - a.z);
        a.w += w * (hv[i].w - a.w);
        *reinterpret_cast<f32x4*>(p.out_acc + row0 * D + 4 * (long long)e) = a;
      }
    }
  }
}

}  // namespace

namespace jg {

bool attn_mfma_fwd_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias) {
  return dtype == JG_BF16 && !has_bias && d == D && sq > 0 && sk > 0 && sq % BM == 0 &&
         sk % (NQ * BN) == 0 && batch > 0 && batch <= 65535;
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
