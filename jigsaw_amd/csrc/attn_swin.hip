// Swin window attention on the token grid itself: 8 x 8 windows, head size 32, bf16, with the
// learned relative-position bias and the shift mask formed inside the kernel
// (examples/swin.py:99-170: the index of 99-104, the mask of 107-126, the attention of 129-170).
//
//   Layout     q, k, v, out, dout are (images, heads, gh * gw tokens, 32): the tokens of an image
//              in row-major grid order, which is what the qkv projection writes and the output
//              projection reads. A wavefront takes one (image, window, head) entry and addresses
//              the 64 token rows of its window in that grid (8 runs of 8 consecutive rows), so the
//              window partition and its inverse are never materialised.
//   Bias       table is (225, heads) fp32, row (qy - ky + 7) * 15 + (qx - kx + 7) for query (qy, qx)
//              and key (ky, kx) of a window. The wavefront keeps its head's column in LDS (times
//              log2 e); with the accumulator layout of S^T = K Q^T (a lane is one query, its
//              registers 16 keys of a 32-key block) the row is a per-lane constant minus a
//              per-register constant, so a bias value is one LDS read at an immediate offset.
//   Mask       side is (windows, 64) bytes or NULL: a code per token of a window; a pair of tokens
//              with different codes must not attend each other (the roll brought them together
//              across an image border). Two ballots turn the codes of a window into bit masks;
//              windows whose tokens all carry the same code (nearly all) skip the masking.
//   Backward   the two passes of the plain window kernel (lane = query for dQ, lane = key for
//              dK / dV). The gradient of the table is what pass A's dS^T scatters by the same row
//              arithmetic: each wavefront adds it into 2 x 225 bins of its own in LDS (one set per
//              lane half, inside which the rows of an instruction's lanes are all different, so a
//              plain read, add, write per register is exact and its order fixed), writes the bins
//              out, and two small kernels add the entries' bins per head in a fixed order.
#include "attn_window_common.h"

namespace {

constexpr int WIN = 8;                       // window edge
constexpr int ROWS = (2 * WIN - 1) * (2 * WIN - 1);  // 225 table rows
constexpr int TOP = 15 * 7 + 7 - 4;          // 108: largest per-register constant of pass A

struct SwinArgs {
  const uint16_t *q, *k, *v, *out, *dout;  // (images, heads, tokens, 32)
  uint16_t *o, *dq, *dk, *dv;              // forward result / gradients, same layout
  float* lse;                              // (entries, 64), entry = (image * windows + window) * heads + head
  const float* table;                      // (225, heads)
  const uint8_t* side;                     // (windows, 64) or NULL
  float* bins;                             // (entries, 2, 225) or NULL: table-gradient parts
  int heads, gw, nwx, nwin;
  long long entries, tokens;
  float scale;
};

struct Entry {
  long long base;  // element offset of token row 0 of the image's head
  int rowoff[2];   // element offset of this lane's token row in blocks 0 / 1
  int head, win;
};

__device__ inline Entry locate(const SwinArgs& p, long long e, int ln) {
  Entry r;
  r.head = (int)(e % p.heads);
  const long long t = e / p.heads;
  r.win = (int)(t % p.nwin);
  const long long img = t / p.nwin;
  const int wy = r.win / p.nwx, wx = r.win - wy * p.nwx;
  r.base = (img * p.heads + r.head) * p.tokens * D;
#pragma unroll
  for (int b = 0; b < 2; ++b) r.rowoff[b] = ((wy * WIN + 4 * b + (ln >> 3)) * p.gw + wx * WIN + (ln & 7)) * D;
  return r;
}

__device__ inline bf16x8 load_row(const uint16_t* base, int rowoff, int ks, int kg) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(base + rowoff + ks * 16 + kg * 8));
}

// The head's column of the table into this wavefront's LDS, times log2 e.
__device__ inline void load_table(float* tab, const SwinArgs& p, int head, int lane) {
  for (int i = lane; i < ROWS; i += 64) tab[i] = p.table[(size_t)i * p.heads + head] * LOG2E;
}

// Bit masks of the window's side codes; `mixed` says whether any two tokens differ.
struct Sides {
  uint64_t s0, s1;
  bool mixed;
};
__device__ inline Sides load_sides(const SwinArgs& p, int win, int lane) {
  Sides r;
  r.s0 = 0; r.s1 = 0; r.mixed = false;
  if (p.side != nullptr) {
    const int code = p.side[(size_t)win * N + lane];
    r.s0 = __builtin_amdgcn_ballot_w64((code & 1) != 0);
    r.s1 = __builtin_amdgcn_ballot_w64((code & 2) != 0);
    r.mixed = (r.s0 != 0 && r.s0 != ~0ull) || (r.s1 != 0 && r.s1 != ~0ull);
  }
  return r;
}
// Bit t set: token t and token `mine` carry different codes.
__device__ inline uint64_t apart_from(const Sides& s, int mine) {
  const uint64_t a0 = ((s.s0 >> mine) & 1) ? ~s.s0 : s.s0;
  const uint64_t a1 = ((s.s1 >> mine) & 1) ? ~s.s1 : s.s1;
  return a0 | a1;
}

// ------------------------------------------------------------------- forward
__global__ __launch_bounds__(WAVES * 64) void attn_swin_fwd_kernel(SwinArgs p) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[WAVES * (TILE + 1024)];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  long long e = (long long)blockIdx.x * WAVES + wave;
  const bool valid = e < p.entries;
  if (!valid) e = p.entries - 1;  // computed again, not stored: every wavefront reaches the barrier
  const Entry en = locate(p, e, ln);
  unsigned char* vt = smem + wave * (TILE + 1024);
  float* tab = reinterpret_cast<float*>(vt + TILE);

  bf16x8 kf[2][2], qf[2][2], vf[2][2];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      kf[b][ks] = load_row(p.k + en.base, en.rowoff[b], ks, kg);
      qf[b][ks] = load_row(p.q + en.base, en.rowoff[b], ks, kg);
      vf[b][ks] = load_row(p.v + en.base, en.rowoff[b], ks, kg);
    }
  load_table(tab, p, en.head, lane);
  const Sides sd = load_sides(p, en.win, lane);
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
    // table row of (query qi, key 32 mb + 8 i4 + 4 kg + r) = 15 qy + qx + 112 - 4 kg - (60 mb + 15 i4 + r)
    const float* tl = tab + (15 * (qi >> 3) + (qi & 7) + 112 - 4 * kg - TOP);
    float x[2][16];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
#pragma unroll
        for (int r = 0; r < 4; ++r) x[mb][i4 * 4 + r] = s[mb][i4 * 4 + r] * c2 + tl[TOP - (60 * mb + 15 * i4 + r)];
    if (sd.mixed) {  // wave-uniform
      const uint64_t ap = apart_from(sd, qi) >> (4 * kg);
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        const uint32_t word = (uint32_t)(ap >> (32 * mb));
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if ((word >> (8 * (i >> 2) + (i & 3))) & 1u) x[mb][i] = -INFINITY;
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, x[mb][i]);
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
      uint16_t* orow = p.o + en.base + en.rowoff[nb];
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) *reinterpret_cast<u32x2*>(orow + i4 * 8 + kg * 4) = pack_rows(o, i4, inv);
      if (kg == 0) p.lse[e * N + qi] = sum > 0.0f ? ms * LN2 + __logf(sum) : -INFINITY;
    }
  }
}

// ------------------------------------------------------------------ backward
constexpr int BINS = 2 * ROWS;  // per wavefront: one set per lane half
constexpr int BWD_PER_WAVE = 3 * TILE + 2 * N * 4 + 1024 + (BINS * 4 + 15) / 16 * 16;  // 18704
constexpr int BWD_LDS = WAVES * BWD_PER_WAVE;                                            // 74816

template <bool DTABLE>
__global__ __launch_bounds__(WAVES * 64) void attn_swin_bwd_kernel(SwinArgs p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ln = lane & 31, kg = lane >> 5;
  long long e = (long long)blockIdx.x * WAVES + wave;
  const bool valid = e < p.entries;
  if (!valid) e = p.entries - 1;
  const Entry en = locate(p, e, ln);
  unsigned char* kt = smem + wave * BWD_PER_WAVE;
  unsigned char* qt = kt + TILE;
  unsigned char* dot = qt + TILE;
  float* lse_s = reinterpret_cast<float*>(dot + TILE);
  float* delta_s = lse_s + N;
  float* tab = delta_s + N;
  float* bins = tab + 256;

  bf16x8 kf[2][2], qf[2][2], vf[2][2], dof[2][2];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      kf[b][ks] = load_row(p.k + en.base, en.rowoff[b], ks, kg);
      qf[b][ks] = load_row(p.q + en.base, en.rowoff[b], ks, kg);
      vf[b][ks] = load_row(p.v + en.base, en.rowoff[b], ks, kg);
      dof[b][ks] = load_row(p.dout + en.base, en.rowoff[b], ks, kg);
    }
  load_table(tab, p, en.head, lane);
  const Sides sd = load_sides(p, en.win, lane);
  if (DTABLE)
    for (int i = lane; i < BINS; i += 64) bins[i] = 0.0f;
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
      const bf16x8 of = load_row(p.out + en.base, en.rowoff[nb], ks, kg);
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
    const int row0 = 15 * (qi >> 3) + (qi & 7) + 112 - 4 * kg - TOP;
    const float* tl = tab + row0;
    float* bl = bins + kg * ROWS + row0;
    const uint64_t ap = sd.mixed ? apart_from(sd, qi) >> (4 * kg) : 0ull;
    f32x16 dqa = zero16();
    float ds[2][16];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      const uint32_t word = (uint32_t)(ap >> (32 * mb));
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = i4 * 4 + r;
          const int c = TOP - (60 * mb + 15 * i4 + r);
          float pr = __builtin_amdgcn_exp2f(s[mb][i] * c2 + tl[c] - lse_q[nb]);
          if (sd.mixed && ((word >> (8 * i4 + r)) & 1u)) pr = 0.0f;
          ds[mb][i] = pr * (dp[mb][i] - delta_q[nb]);
        }
#pragma unroll
      for (int h = 0; h < 2; ++h)
        dqa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(kt, mb * 2 + h, ln, kg), pack_half(ds[mb], h), dqa, 0, 0, 0);
    }
    if (DTABLE && valid) {
      // dS^T into the bins, register by register: the 32 lanes of a half hit 32 different rows, and
      // so do a register of key block 0 and its twin of block 1 (their rows differ by 60, more
      // than the queries of a 32-lane block are apart), so the pair is read, added to and
      // written back as plain LDS accesses; the LDS keeps a wavefront's accesses in order.
      // (LDS float atomics do the same job at about 800 cycles an instruction.)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = i4 * 4 + r;
          const int c0 = TOP - (15 * i4 + r), c1 = c0 - 60;
          const float b0 = bl[c0], b1 = bl[c1];
          bl[c0] = b0 + ds[0][i];
          bl[c1] = b1 + ds[1][i];
          // for one lane the rows of different registers never coincide, so the compiler would be
          // free to read ahead; other lanes' rows do coincide with them: one step after the other
          asm volatile("" ::: "memory");
        }
    }
    if (valid) {
      uint16_t* row = p.dq + en.base + en.rowoff[nb];
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) *reinterpret_cast<u32x2*>(row + i4 * 8 + kg * 4) = pack_rows(dqa, i4, p.scale);
    }
  }
  if (DTABLE && valid) {
    float* dst = p.bins + e * BINS;
    for (int i = lane; i < BINS; i += 64) dst[i] = bins[i];
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
    // table row of (query 32 mbq + 8 i4 + 4 kg + r, key ki) = 112 + 4 kg - 15 ky - kx + (60 mbq + 15 i4 + r)
    const float* tl = tab + (112 + 4 * kg - 15 * (ki >> 3) - (ki & 7));
    const uint64_t ap = sd.mixed ? apart_from(sd, ki) >> (4 * kg) : 0ull;
    f32x16 dva = zero16(), dka = zero16();
#pragma unroll
    for (int mbq = 0; mbq < 2; ++mbq) {
      const uint32_t word = (uint32_t)(ap >> (32 * mbq));
      float pr[16], ds[16];
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int q0 = mbq * 32 + i4 * 8 + kg * 4;
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(lse_s + q0);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(delta_s + q0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = i4 * 4 + r;
          pr[i] = __builtin_amdgcn_exp2f(s[mbq][i] * c2 + tl[60 * mbq + 15 * i4 + r] - l4[r]);
          if (sd.mixed && ((word >> (8 * i4 + r)) & 1u)) pr[i] = 0.0f;
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
      uint16_t* vrow = p.dv + en.base + en.rowoff[nbk];
      uint16_t* krow = p.dk + en.base + en.rowoff[nbk];
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        *reinterpret_cast<u32x2*>(vrow + i4 * 8 + kg * 4) = pack_rows(dva, i4, 1.0f);
        *reinterpret_cast<u32x2*>(krow + i4 * 8 + kg * 4) = pack_rows(dka, i4, p.scale);
      }
    }
  }
}

// Table gradient, stage 1: block (head, chunk) adds the bins of its entries, entry after entry;
// thread i < 450 owns bin i. stage 2: block `head` adds the chunks and the two lane halves.
constexpr int CHUNKS = 32;
__global__ __launch_bounds__(512) void swin_bins_stage1(const float* __restrict__ bins, float* __restrict__ part,
                                                        long long entries, int heads) {
  const int head = blockIdx.x, chunk = blockIdx.y, i = threadIdx.x;
  if (i >= BINS) return;
  const long long groups = entries / heads;  // entries of one head
  const long long per = (groups + CHUNKS - 1) / CHUNKS;
  long long g0 = chunk * per, g1 = g0 + per;
  if (g1 > groups) g1 = groups;
  float acc = 0.0f;
  for (long long g = g0; g < g1; ++g) acc += bins[(g * heads + head) * BINS + i];
  part[((size_t)head * CHUNKS + chunk) * BINS + i] = acc;
}
__global__ __launch_bounds__(256) void swin_bins_stage2(const float* __restrict__ part, float* __restrict__ dtable, int heads) {
  const int head = blockIdx.x, i = threadIdx.x;
  if (i >= ROWS) return;
  float acc = 0.0f;
  for (int c = 0; c < CHUNKS; ++c) {
    const float* pc = part + ((size_t)head * CHUNKS + c) * BINS;
    acc += pc[i] + pc[ROWS + i];
  }
  dtable[(size_t)i * heads + head] = acc;
}

int check(const char* who, int64_t images, int64_t heads, int64_t gh, int64_t gw, int64_t d, int dtype, float scale) {
  JG_REQUIRE(dtype == JG_BF16, "%s: bf16 only", who);
  JG_REQUIRE(d == D, "%s: head size %lld, built for %d", who, (long long)d, D);
  JG_REQUIRE(images >= 0 && heads >= 1 && gh >= WIN && gw >= WIN && gh % WIN == 0 && gw % WIN == 0,
             "%s: the token grid (%lld x %lld) must be whole windows of %d x %d", who, (long long)gh, (long long)gw, WIN, WIN);
  JG_REQUIRE(gh * gw * D < (1ll << 31), "%s: token grid too large for 32-bit row offsets", who);
  JG_REQUIRE(scale > 0.0f, "%s: scale must be positive", who);
  return JG_OK;
}

bool al16(std::initializer_list<const void*> ptrs) {
  for (const void* q : ptrs)
    if ((reinterpret_cast<uintptr_t>(q) & 15) != 0) return false;
  return true;
}

SwinArgs common(int64_t images, int64_t heads, int64_t gh, int64_t gw, float scale, const float* table, const uint8_t* side) {
  SwinArgs a = {};
  a.table = table;
  a.side = side;
  a.heads = (int)heads;
  a.gw = (int)gw;
  a.nwx = (int)(gw / WIN);
  a.nwin = (int)((gh / WIN) * (gw / WIN));
  a.entries = images * a.nwin * heads;
  a.tokens = gh * gw;
  a.scale = scale;
  return a;
}

}  // namespace

// Windowed attention of a Swin block on the token grid (examples/swin.py:129-170 with the index of
// 99-104 and the mask of 107-126 formed in the kernel). lse: (images * windows * heads, 64) fp32.
extern "C" int jg_attn_swin_fwd(void* out, float* lse, const void* q, const void* k, const void* v, const float* table,
                                const uint8_t* side, int64_t images, int64_t heads, int64_t gh, int64_t gw, int64_t d,
                                float scale, int dtype, void* stream) {
  const char* who = "jg_attn_swin_fwd";
  int rc = check(who, images, heads, gh, gw, d, dtype, scale);
  if (rc) return rc;
  JG_REQUIRE(out && lse && q && k && v && table, "%s: NULL pointer", who);
  JG_REQUIRE(al16({out, q, k, v}), "%s: tensors must be 16-byte aligned", who);
  SwinArgs a = common(images, heads, gh, gw, scale, table, side);
  if (a.entries == 0) return JG_OK;
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k);
  a.v = static_cast<const uint16_t*>(v);
  a.o = static_cast<uint16_t*>(out);
  a.lse = lse;
  JG_REQUIRE((a.entries + WAVES - 1) / WAVES < (1ll << 31), "%s: too many windows", who);
  attn_swin_fwd_kernel<<<dim3((unsigned)((a.entries + WAVES - 1) / WAVES)), WAVES * 64, 0, static_cast<hipStream_t>(stream)>>>(a);
  JG_CHECK_LAUNCH(who);
  return JG_OK;
}

// Workspace of jg_attn_swin_bwd when the table gradient is wanted: the bins of every entry and
// the chunk sums of the first reduction stage.
extern "C" size_t jg_attn_swin_bwd_workspace_bytes(int64_t images, int64_t heads, int64_t gh, int64_t gw) {
  if (images <= 0 || heads <= 0 || gh <= 0 || gw <= 0) return 0;
  const size_t entries = (size_t)images * (size_t)((gh / WIN) * (gw / WIN)) * (size_t)heads;
  return (entries + (size_t)heads * CHUNKS) * BINS * sizeof(float);
}

extern "C" int jg_attn_swin_bwd(void* dq, void* dk, void* dv, float* dtable, const void* dout, const void* q, const void* k,
                                const void* v, const void* out, const float* lse, const float* table, const uint8_t* side,
                                int64_t images, int64_t heads, int64_t gh, int64_t gw, int64_t d, float scale, int dtype,
                                void* workspace, size_t workspace_bytes, void* stream) {
  const char* who = "jg_attn_swin_bwd";
  int rc = check(who, images, heads, gh, gw, d, dtype, scale);
  if (rc) return rc;
  JG_REQUIRE(dq && dk && dv && dout && q && k && v && out && lse && table, "%s: NULL pointer", who);
  JG_REQUIRE(al16({dq, dk, dv, dout, q, k, v, out}), "%s: tensors must be 16-byte aligned", who);
  SwinArgs a = common(images, heads, gh, gw, scale, table, side);
  if (a.entries == 0) return JG_OK;
  if (dtable != nullptr && (workspace == nullptr || workspace_bytes < jg_attn_swin_bwd_workspace_bytes(images, heads, gh, gw)))
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, workspace_bytes,
            jg_attn_swin_bwd_workspace_bytes(images, heads, gh, gw));
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k);
  a.v = static_cast<const uint16_t*>(v);
  a.out = static_cast<const uint16_t*>(out);
  a.dout = static_cast<const uint16_t*>(dout);
  a.dq = static_cast<uint16_t*>(dq);
  a.dk = static_cast<uint16_t*>(dk);
  a.dv = static_cast<uint16_t*>(dv);
  a.lse = const_cast<float*>(lse);
  a.bins = static_cast<float*>(workspace);
  JG_REQUIRE((a.entries + WAVES - 1) / WAVES < (1ll << 31), "%s: too many windows", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((a.entries + WAVES - 1) / WAVES));
  static bool lds_set = false;
  if (!lds_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_swin_bwd_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, BWD_LDS) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_swin_bwd_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, BWD_LDS) != hipSuccess)
      JG_FAIL(JG_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS", who, BWD_LDS);
    lds_set = true;
  }
  if (dtable != nullptr) {
    attn_swin_bwd_kernel<true><<<grid, WAVES * 64, BWD_LDS, s>>>(a);
    JG_CHECK_LAUNCH(who);
    float* part = a.bins + (size_t)a.entries * BINS;
    swin_bins_stage1<<<dim3((unsigned)heads, CHUNKS), 512, 0, s>>>(a.bins, part, a.entries, (int)heads);
    JG_CHECK_LAUNCH(who);
    swin_bins_stage2<<<dim3((unsigned)heads), 256, 0, s>>>(part, dtable, (int)heads);
    JG_CHECK_LAUNCH(who);
  } else {
    attn_swin_bwd_kernel<false><<<grid, WAVES * 64, BWD_LDS, s>>>(a);
    JG_CHECK_LAUNCH(who);
  }
  return JG_OK;
}
