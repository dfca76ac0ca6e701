// Backward of the blockwise attention core on the bf16 matrix cores, head size
// 64, from the ring's GLOBAL out / lse (p = exp(s - lse) is already globally
// normalised). Two kernels, no atomics, deterministic:
//
//   dQ kernel      lane = query (as in the forward kernel). Per 64-key tile:
//                    S^T  = K Q^T                 A = K rows,    B = Q (registers)
//                    dP^T = V dO^T                A = V rows,    B = dO (registers)
//                    dS^T = P^T o (dP^T - delta) * scale      (lane-local)
//                    dQ^T += K^T dS^T             A = K^T (LDS transpose reads),
//                                                 B = dS^T straight from registers
//                  It also computes delta = rowsum(dO o O) and leaves it in the
//                  workspace for the second kernel.
//   dK/dV kernel   lane = key. Per 64-query tile:
//                    S  = Q K^T                   A = Q rows,    B = K (registers)
//                    dP = dO V^T                  A = dO rows,   B = V (registers)
//                    P, dS from lse / delta of the tile (broadcast LDS reads)
//                    dV^T += dO^T P               A = dO^T (LDS transpose reads)
//                    dK^T += Q^T dS               A = Q^T  (LDS transpose reads)
//   The score tile is recomputed in each kernel (7 matrix products instead of the
//   5 of a one-kernel formulation) so that P / dS are always produced in the
//   register layout the next MFMA consumes and never travel through LDS.
//
//   Workgroup: 512 threads = 8 wavefronts = 4 blocks of 32 rows (queries for dQ,
//   keys for dK/dV) x 2 halves of the streamed side, combined through LDS.
//   Streamed tiles (64 rows x 128 bytes) travel from memory straight into LDS, row-major
//   with the 16-byte chunks of a row XOR-swizzled by row % 8 (no registers, no vector
//   instructions, no second, transposed copy): the transposed fragments come from
//   ds_read_b64_tr_b16 (within 16 lanes, lane i receives element i % 4 of the 8 bytes
//   that lanes i / 4 + 4 j point at, j = 0..3), two reads of 4 consecutive rows each.
//
//   Several resident chunks in one pass (the ring backward from saved chunks,
//   jigsaw/modules/attention/_functional/backward.py:176-277): the dQ kernel walks the key tiles of
//   every chunk in turn with dQ in its registers (one launch, one rounding), and the chunk is a
//   third grid dimension of the dK/dV kernel. The chunk pointers travel in the kernel-argument
//   segment (first parameter), where a wavefront reads entry c with scalar loads.
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
typedef short i16x4 __attribute__((ext_vector_type(4)));

constexpr int D = 64;
constexpr int BR = 128;           // resident rows per workgroup (4 blocks of 32)
constexpr int BT = 64;            // streamed rows per tile
constexpr int THREADS = 512;
constexpr int ROWB = D * 2;       // bytes per row of a tile in LDS (no padding)
constexpr int NAT = BT * ROWB;    // 8192: one 64 x 64 bf16 tile
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ bf16x8 lds_frag(const unsigned char* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(p));
}

// One wavefront instruction lands 64 x 16 bytes contiguously in LDS, lane order = 8 rows: lane L
// sits at row L / 8, chunk position L % 8 and fetches chunk (L % 8) ^ (row % 8) of its row.
// Written in assembly: wave-uniform 64-bit source in scalar registers, the lane's constant
// offset, the LDS address of the 1 KB block in M0. (With the compiler's own form of this load
// it orders every later LDS read behind ALL outstanding transfers, also those of the tile
// after next; the kernels order reads and transfers themselves, by their waits and barriers.)
__device__ __forceinline__ uint32_t dma_lane_offset(int lane) {
  return (uint32_t)((lane >> 3) * ROWB + (((lane & 7) ^ (lane >> 3)) << 4));
}
__device__ __forceinline__ void dma_1k(const char* src, uint32_t lane_off, uint32_t lds_dst) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_off), "s"(src), "s"(lds_dst) : "m0");
}
__device__ __forceinline__ uint32_t lds_address(const unsigned char* p) {
  typedef __attribute__((address_space(3))) unsigned char* lds_bytes;
  return (uint32_t)(uintptr_t)((lds_bytes)p);
}

// fragment of a row-major tile: row r (0..63), 16-byte chunk c (0..7)
__device__ __forceinline__ bf16x8 nat_frag(const unsigned char* nat, int r, int c) {
  return lds_frag(nat + r * ROWB + ((c ^ (r & 7)) << 4));
}

// Per-lane constant part of the address of a TRANSPOSED fragment (A operand: 32 columns of the
// tile x 16 of its rows): lane p of a group of 16 points at row +4 kg + p / 4, columns 32 nb +
// 16 (group % 2) + 4 (p % 4); the row's swizzle is 4 kg + p / 4 whatever multiple of 8 the
// fragment starts at.
__device__ __forceinline__ int tr_lane_offset(int lane, int nb) {
  const int pp = lane & 15, g1 = (lane >> 4) & 1, kg = lane >> 5;
  const int rsw = 4 * kg + (pp >> 2);
  return rsw * ROWB + (((4 * nb + 2 * g1 + ((pp & 3) >> 1)) ^ rsw) << 4) + 8 * (pp & 1);
}
// Transposed fragment whose 16 rows start at `row0` (a multiple of 16): slots 0..3 = rows
// row0 + 4 kg + 0..3, slots 4..7 = rows row0 + 8 + 4 kg + 0..3: the order an accumulator lane
// holds its rows in.
__device__ __forceinline__ bf16x8 tr_frag(const unsigned char* nat, int lane_off, int row0) {
  typedef __attribute__((address_space(3))) i16x4* tr_ptr;
  const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(nat + lane_off + row0 * ROWB));
  const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(nat + lane_off + (row0 + 8) * ROWB));
  u32x4 w;
  w.x = __builtin_bit_cast(u32x2, lo).x;
  w.y = __builtin_bit_cast(u32x2, lo).y;
  w.z = __builtin_bit_cast(u32x2, hi).x;
  w.w = __builtin_bit_cast(u32x2, hi).y;
  return __builtin_bit_cast(bf16x8, w);
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

// Workgroup -> (batch entry, row block). Consecutive workgroup ids go to the 8 XCDs in turn; each
// XCD is given a contiguous range of (batch entry, block) pairs, so the workgroups that stream the
// same K / V (or Q / dO) share one L2 instead of every L2 holding every head. Falls back to the
// plain order when the count does not divide.
struct BlockOf {
  long long bh;
  int blk;
  int chunk;
};
// gridDim = (row blocks, batch entries, chunks). The flat order is (batch entry, chunk, block), so the
// workgroups of one XCD's range stream the Q / dO (or K / V) of the same few batch entries.
__device__ __forceinline__ BlockOf block_of() {
  const unsigned nblk = gridDim.x, nch = gridDim.z, total = gridDim.x * gridDim.y * gridDim.z;
  unsigned id = (blockIdx.y * nch + blockIdx.z) * nblk + blockIdx.x;
  if ((total & 7u) == 0) id = (id & 7u) * (total >> 3) + (id >> 3);
  BlockOf b;
  b.blk = (int)(id % nblk);
  id /= nblk;
  b.chunk = (int)(id % nch);
  b.bh = id / nch;
  return b;
}

constexpr int MAX_CHUNKS = 16;
// Chunk c: k[c], v[c] (batch, sk, 64) and where its gradients go. FIRST kernel parameter: entry c is
// read from the kernel-argument segment by its offset (a by-value struct indexed with a run-time
// value would otherwise be copied to private memory lane by lane).
struct ChunkTable {
  const uint16_t* k[MAX_CHUNKS];
  const uint16_t* v[MAX_CHUNKS];
  uint16_t* dk[MAX_CHUNKS];
  uint16_t* dv[MAX_CHUNKS];
};
__device__ __forceinline__ const char* chunk_entry(int which, int c) {  // which: 0 k, 1 v, 2 dk, 3 dv; c wave-uniform
#if defined(__HIP_DEVICE_COMPILE__)
  const char* const* kt = (const char* const*)__builtin_amdgcn_kernarg_segment_ptr();
  return kt[which * MAX_CHUNKS + c];
#else
  (void)which; (void)c;
  return nullptr;
#endif
}

struct BwdArgs {
  const uint16_t* dout;
  const uint16_t* q;
  const uint16_t* out;
  const float* lse;
  float* delta;     // (batch, sq) workspace
  uint16_t* dq;
  int sq, sk;       // sk: keys per chunk
  int nchunks;
  long long batch;
  float scale;
};

// ------------------------------------------------------------------ dQ kernel
constexpr int NBUF = 4;                     // tiles in flight per half: read back, current, read ahead, landing
constexpr int DQ_BUF = 2 * NAT;             // K tile, V tile
constexpr int DQ_HALF = NBUF * DQ_BUF;
constexpr int DQ_LDS = 2 * DQ_HALF;         // 131072 (and at least 4 x 32 x 64 floats for the hand-over)

// Scheduling classes of __builtin_amdgcn_sched_group_barrier
#define JG_GROUP_VALU 0x002
#define JG_GROUP_MFMA 0x008
#define JG_GROUP_DS_READ 0x100

__global__ __launch_bounds__(THREADS) void attn_bwd_dq_kernel(ChunkTable chunks, BwdArgs p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int qb = wave & 3, ks = wave >> 2;
  const BlockOf where = block_of();
  const long long b = where.bh;
  const int q0 = where.blk * BR + qb * 32;
  // every chunk is cut in two key halves (one per wavefront group); a half's tiles of all chunks
  // form one stream of ntiles tiles
  const int khalf = p.sk >> 1;
  const int tiles_per_chunk = khalf / BT;
  const int ntiles = tiles_per_chunk * p.nchunks;
  const float c2 = p.scale * LOG2E;
  const long long qi = b * p.sq + q0 + ln;

  unsigned char* lds = smem + ks * DQ_HALF;
  // this wavefront moves rows 16 qb .. 16 qb + 15 of the K tile and of the V tile of its half
  const int ks_u = __builtin_amdgcn_readfirstlane(ks), qb_u = __builtin_amdgcn_readfirstlane(qb);
  const long long half_off = 2 * ((b * p.sk + (long long)ks_u * khalf) * D) + 16 * qb_u * ROWB;  // bytes into a chunk
  int ld_chunk = 0, ld_tile = 0;  // the load cursor: tiles are requested in stream order
  const char* kdma = chunk_entry(0, 0) + half_off;
  const char* vdma = chunk_entry(1, 0) + half_off;
  const uint32_t dma_off = dma_lane_offset(lane);
  const uint32_t lds_dma = lds_address(smem) + (uint32_t)(ks_u * DQ_HALF + 16 * qb_u * ROWB);
  const int tr_off[2] = {tr_lane_offset(lane, 0), tr_lane_offset(lane, 1)};
  // row fragments: row ln of a 32-row block, chunk 2 c + kg
  int row_off[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) row_off[c] = ln * ROWB + (((2 * c + kg) ^ (ln & 7)) << 4);

  // K and V of tile t straight into its buffer (free since the barrier that ended the tile before)
  auto issue_loads = [&](int t) {  // called with t = 0, 1, 2, ... in turn
    const long long off = (long long)ld_tile * NAT;
    const uint32_t dst = lds_dma + (uint32_t)((t & (NBUF - 1)) * DQ_BUF);
    dma_1k(kdma + off, dma_off, dst);
    dma_1k(kdma + off + 8 * ROWB, dma_off, dst + 8 * ROWB);
    dma_1k(vdma + off, dma_off, dst + NAT);
    dma_1k(vdma + off + 8 * ROWB, dma_off, dst + NAT + 8 * ROWB);
    if (++ld_tile == tiles_per_chunk && ld_chunk + 1 < p.nchunks) {
      ld_tile = 0;
      ++ld_chunk;
      kdma = chunk_entry(0, ld_chunk) + half_off;
      vdma = chunk_entry(1, ld_chunk) + half_off;
    }
  };
  auto tiles_landed = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's transfers have landed
  };

  // the first tiles are on their way while the wavefront fetches its own rows
  issue_loads(0);
  if (ntiles > 1) issue_loads(1);

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
  f32x16 minus_delta;
#pragma unroll
  for (int i = 0; i < 16; ++i) minus_delta[i] = -delta;

  f32x16 dq[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[nb][i] = 0.0f;

  // The stream of 32-key blocks is software pipelined three deep. While the vector unit turns the
  // scores and dP of block j into dS (B), the matrix core computes the scores and dP of block
  // j + 1 (A, 8 instructions) and adds block j - 1 to dQ (C, 4 instructions): the three are
  // independent, so every matrix instruction has about seven vector instructions to run
  // under it. dS is kept without the softmax scale, which multiplies dQ once at the end.
  f32x16 s_cur, dp_cur;
  bf16x8 ds_prev[2];
  auto scores = [&](const unsigned char* kn, int sb, f32x16& s, f32x16& dp) {
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.0f;
    // dP starts from -delta (a lane is one query): the product then leaves dP - delta behind
    dp = minus_delta;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(kn + sb * 32 * ROWB + row_off[c]), qf[c], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(kn + NAT + sb * 32 * ROWB + row_off[c]), dof[c], dp, 0, 0, 0);
    }
  };
  auto ds_frag = [&](int t) {
    float e[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float pr = __builtin_amdgcn_exp2f(s_cur[8 * t + i] * c2 - lse2);
      e[i] = pr * dp_cur[8 * t + i];
    }
    return pack8(e);
  };
  auto add_to_dq = [&](const unsigned char* kn, int sb) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
        dq[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(kn, tr_off[nb], sb * 32 + 16 * t), ds_prev[t], dq[nb], 0, 0, 0);
  };
  // one step of the pipeline: A of (k_next, sb_next), B of the current block, C of (k_prev, sb_prev)
  auto step = [&](const unsigned char* k_next, int sb_next, const unsigned char* k_prev, int sb_prev, bool ahead) {
    f32x16 s_n, dp_n;
    if (ahead) scores(k_next, sb_next, s_n, dp_n);
    bf16x8 ds_now[2];
    ds_now[0] = ds_frag(0);
    ds_now[1] = ds_frag(1);
    add_to_dq(k_prev, sb_prev);
    if (ahead) {
#define JG_SLOT(reads)                                               \
  __builtin_amdgcn_sched_group_barrier(JG_GROUP_MFMA, 1, 0);          \
  __builtin_amdgcn_sched_group_barrier(JG_GROUP_DS_READ, reads, 0);   \
  __builtin_amdgcn_sched_group_barrier(JG_GROUP_VALU, 7, 0);
      JG_SLOT(2) JG_SLOT(2) JG_SLOT(2) JG_SLOT(2) JG_SLOT(2) JG_SLOT(2) JG_SLOT(2) JG_SLOT(2)
      JG_SLOT(0) JG_SLOT(0) JG_SLOT(0) JG_SLOT(0)
#undef JG_SLOT
      s_cur = s_n;
      dp_cur = dp_n;
    }
    ds_prev[0] = ds_now[0];
    ds_prev[1] = ds_now[1];
  };

  tiles_landed();
  __syncthreads();
  scores(lds, 0, s_cur, dp_cur);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    ds_prev[0][i] = (__bf16)0.0f;  // block -1 adds nothing (times the finite K of block 0)
    ds_prev[1][i] = (__bf16)0.0f;
  }
  const unsigned char* k_back = lds;  // tile of the block before the current one
  int sb_back = 0;
  for (int t = 0; t + 1 < ntiles; ++t) {
    if (t + 2 < ntiles) issue_loads(t + 2);
    const unsigned char* kn = lds + (t & (NBUF - 1)) * DQ_BUF;
    const unsigned char* kn1 = lds + ((t + 1) & (NBUF - 1)) * DQ_BUF;
    step(kn, 1, k_back, sb_back, true);
    step(kn1, 0, kn, 0, true);
    k_back = kn;
    sb_back = 1;
    tiles_landed();
    __syncthreads();
  }
  {
    const unsigned char* kn = lds + ((ntiles - 1) & (NBUF - 1)) * DQ_BUF;
    step(kn, 1, k_back, sb_back, true);
    step(kn, 0, kn, 0, false);
    add_to_dq(kn, 1);
  }
  __syncthreads();  // the hand-over below reuses the tile buffers

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
constexpr int DKV_HALF = 2 * NAT + DKV_STATS;         // Q tile, dO tile + stats
constexpr int DKV_LDS = 4 * DKV_HALF;                 // 67584: two query halves, double buffered
// Key blocks per workgroup. With 2 (4 wavefronts, 64 keys) a launch has twice the workgroups, two of
// which share a CU: the two wavefronts of a SIMD then belong to different workgroups and do not
// march in step (the barrier per tile keeps the wavefronts of ONE workgroup in the same phase:
// all in their matrix instructions, then all in their exponentials).
#ifndef JG_DKV_KB
#define JG_DKV_KB 4
#endif
constexpr int DKV_KB = JG_DKV_KB;
constexpr int DKV_THREADS = 64 * 2 * DKV_KB;
constexpr int DKV_ROWS = 32 * DKV_KB;                 // keys per workgroup
constexpr int DKV_SHARE = BT / DKV_KB;                // rows of a streamed tile each wavefront of a half moves
static_assert(DKV_LDS >= DKV_KB * 64 * 64 * 4, "the hand-over of the partial dK / dV reuses the tile buffers");
static_assert(64 * DKV_KB >= 2 * BT, "one thread of a half per statistic");

__global__ __launch_bounds__(DKV_THREADS, 8 / (2 * DKV_KB) >= 2 ? 2 : 1) void attn_bwd_dkv_kernel(ChunkTable chunks, BwdArgs p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  const int kb = wave % DKV_KB, qs = wave / DKV_KB;
  const int th = tid % (64 * DKV_KB);
  const BlockOf where = block_of();
  const long long b = where.bh;
  const int k0 = where.blk * DKV_ROWS + kb * 32;
  const int qhalf = p.sq >> 1;
  const int ntiles = qhalf / BT;
  const float c2 = p.scale * LOG2E;
  const long long ki = b * p.sk + k0 + ln;

  unsigned char* lds = smem + qs * (2 * DKV_HALF);  // two buffers: Q tile, dO tile, stats
  const long long qrow0 = b * p.sq + (long long)qs * qhalf;
  // this wavefront moves its share of the rows of the Q tile and of the dO tile of its half
  const int qs_u = __builtin_amdgcn_readfirstlane(qs), kb_u = __builtin_amdgcn_readfirstlane(kb);
  const long long qrow0_u = b * p.sq + (long long)qs_u * qhalf;
  const char* qdma = reinterpret_cast<const char*>(p.q + qrow0_u * D) + DKV_SHARE * kb_u * ROWB;
  const char* ddma = reinterpret_cast<const char*>(p.dout + qrow0_u * D) + DKV_SHARE * kb_u * ROWB;
  const uint32_t dma_off = dma_lane_offset(lane);
  const uint32_t lds_dma = lds_address(smem) + (uint32_t)(qs_u * (2 * DKV_HALF) + DKV_SHARE * kb_u * ROWB);
  const int tr_off[2] = {tr_lane_offset(lane, 0), tr_lane_offset(lane, 1)};

  float st_reg = 0.0f;
  auto issue_loads = [&](int t, int buf) {
    const long long off = (long long)t * NAT;
    const uint32_t dst = lds_dma + (uint32_t)(buf * DKV_HALF);
#pragma unroll
    for (int r = 0; r < DKV_SHARE; r += 8) {
      dma_1k(qdma + off + r * ROWB, dma_off, dst + r * ROWB);
      dma_1k(ddma + off + r * ROWB, dma_off, dst + NAT + r * ROWB);
    }
    // One plain load for every lane, used only when the statistics go to LDS: a load under a
    // per-lane condition, or arithmetic on its result here, would make the wavefront wait
    // for it (and for the transfers issued before it) on the spot.
    const float* src = th < BT ? p.lse : p.delta;
    st_reg = src[qrow0 + (long long)t * BT + (th & (BT - 1))];
  };
  auto store_stats = [&](int buf) {
    unsigned char* base = lds + buf * DKV_HALF;
    if (th < 2 * BT) reinterpret_cast<float*>(base + 2 * NAT)[th] = th < BT ? st_reg * LOG2E : -st_reg;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the transfers into this buffer have landed
  };

  // the first tile is on its way while the wavefront fetches its own rows
  issue_loads(0, 0);

  bf16x8 kf[4], vf[4];
  {
    const uint16_t* krow = reinterpret_cast<const uint16_t*>(chunk_entry(0, where.chunk)) + ki * D + 8 * kg;
    const uint16_t* vrow = reinterpret_cast<const uint16_t*>(chunk_entry(1, where.chunk)) + ki * D + 8 * kg;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      kf[c] = lds_frag(reinterpret_cast<const unsigned char*>(krow + 16 * c));
      vf[c] = lds_frag(reinterpret_cast<const unsigned char*>(vrow + 16 * c));
    }
  }

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
    const unsigned char* dn = qn + NAT;
    const float* st = reinterpret_cast<const float*>(qn + 2 * NAT);  // lse2[64] then -delta[64]
    bf16x8 pf[2][2], dsf[2][2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      f32x16 s, dp;
#pragma unroll
      for (int i = 0; i < 16; ++i) s[i] = 0.0f;
      // dP starts from -delta of its queries (register i: query sb*32 + 8*(i/4) + 4*kg + i%4)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(st + BT + sb * 32 + 8 * j + 4 * kg);
#pragma unroll
        for (int e = 0; e < 4; ++e) dp[4 * j + e] = d4[e];
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nat_frag(qn, sb * 32 + ln, 2 * c + kg), kf[c], s, 0, 0, 0);
        dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nat_frag(dn, sb * 32 + ln, 2 * c + kg), vf[c], dp, 0, 0, 0);
      }
      // register i of this lane: query sb*32 + 8*(i/4) + 4*kg + i%4, key ln
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float pe[8], de[8];
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const int j = 2 * t + jj;
          const f32x4 l4 = *reinterpret_cast<const f32x4*>(st + sb * 32 + 8 * j + 4 * kg);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float pr = __builtin_amdgcn_exp2f(s[4 * j + e] * c2 - l4[e]);
            pe[4 * jj + e] = pr;
            de[4 * jj + e] = pr * dp[4 * j + e];
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
          dv[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(dn, tr_off[nb], sb * 32 + 16 * t), pf[sb][t], dv[nb], 0, 0, 0);
          dk[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr_frag(qn, tr_off[nb], sb * 32 + 16 * t), dsf[sb][t], dk[nb], 0, 0, 0);
        }
  };

  int buf = 0;
  store_stats(0);
  // The K / V fragments came straight from memory: they are waited for here, once. Left
  // to the first MFMA that reads them, the wait would sit inside the loop, behind the
  // tile loads that every iteration has just issued.
#pragma unroll
  for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(kf[c]), "+v"(vf[c]));
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const bool has_next = t + 1 < ntiles;
    if (has_next) issue_loads(t + 1, buf ^ 1);
    compute_tile(buf);
    if (has_next) store_stats(buf ^ 1);
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
  uint16_t* dk_out = reinterpret_cast<uint16_t*>(const_cast<char*>(chunk_entry(2, where.chunk)));
  uint16_t* dv_out = reinterpret_cast<uint16_t*>(const_cast<char*>(chunk_entry(3, where.chunk)));
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
      *reinterpret_cast<bf16x4*>(dk_out + ki * D + col) = __builtin_convertvector(a, bf16x4);
      *reinterpret_cast<bf16x4*>(dv_out + ki * D + col) = __builtin_convertvector(c, bf16x4);
    }
}

}  // namespace

namespace jg {

bool attn_mfma_bwd_supported(long long batch, int sq, int sk, int d, int dtype, bool has_bias) {
  return dtype == JG_BF16 && !has_bias && d == D && sq > 0 && sk > 0 && sq % BR == 0 &&
         sk % BR == 0 && sk % DKV_ROWS == 0 && batch > 0 && batch <= 65535;
}

size_t attn_mfma_bwd_workspace(long long batch, int sq, int) {
  return (size_t)batch * sq * sizeof(float);
}

// The ring backward over `nchunks` resident chunks: k[c], v[c] in, dk[c], dv[c] out, dq = the sum over
// the chunks, rounded once. nchunks = 1 is the plain backward of one chunk.
int attn_mfma_bwd_chunks(void* dq, void* const* dk, void* const* dv, const void* dout, const void* q,
                         const void* const* k, const void* const* v, int nchunks, const void* out, const float* lse,
                         long long batch, int sq, int sk, float scale, void* ws, hipStream_t s) {
  if (nchunks < 1 || nchunks > MAX_CHUNKS)
    JG_FAIL(JG_ERR_UNSUPPORTED, "jg_attn_bwd_chunks: 1 to %d chunks a call, got %d", MAX_CHUNKS, nchunks);
  ChunkTable tab;
  for (int c = 0; c < MAX_CHUNKS; ++c) {
    const int u = c < nchunks ? c : 0;
    tab.k[c] = static_cast<const uint16_t*>(k[u]);
    tab.v[c] = static_cast<const uint16_t*>(v[u]);
    tab.dk[c] = static_cast<uint16_t*>(dk[u]);
    tab.dv[c] = static_cast<uint16_t*>(dv[u]);
  }
  BwdArgs a;
  a.dout = static_cast<const uint16_t*>(dout);
  a.q = static_cast<const uint16_t*>(q);
  a.out = static_cast<const uint16_t*>(out);
  a.lse = lse;
  a.delta = static_cast<float*>(ws);
  a.dq = static_cast<uint16_t*>(dq);
  a.sq = sq;
  a.sk = sk;
  a.nchunks = nchunks;
  a.batch = batch;
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
  attn_bwd_dq_kernel<<<dim3((unsigned)(sq / BR), (unsigned)batch, 1), THREADS, DQ_LDS, s>>>(tab, a);
  JG_CHECK_LAUNCH("jg_attn_bwd(dq)");
  attn_bwd_dkv_kernel<<<dim3((unsigned)(sk / DKV_ROWS), (unsigned)batch, (unsigned)nchunks), DKV_THREADS, DKV_LDS, s>>>(tab, a);
  JG_CHECK_LAUNCH("jg_attn_bwd(dkv)");
  return JG_OK;
}

int attn_mfma_bwd(void* dq, void* dk, void* dv, const void* dout, const void* q, const void* k,
                  const void* v, const void* out, const float* lse, long long batch, int sq,
                  int sk, float scale, void* ws, hipStream_t s) {
  return attn_mfma_bwd_chunks(dq, &dk, &dv, dout, q, &k, &v, 1, out, lse, batch, sq, sk, scale, ws, s);
}

}  // namespace jg
