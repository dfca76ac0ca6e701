// Weight gradient of the 3x3 (2-D) and 3x3x3 (3-D) convolution on the bf16 matrix
// cores, stride 1, dilation 1, channels-first tensors; a launch covers a block of 32 or
// 64 channels a side, any other channel counts are walked block by block. Optionally the
// bias gradient from the same pass over g. fp16 tensors run the same kernel on the fp16
// MFMA instruction (the gradient is reduced in fp32 and rounded to fp16 once); fp32 tensors
// run as sums of three bf16 parts per operand ("split mode": the parts are extra channels,
// their products are added up in fp32).
//
//   gw[co][ci][kd][kh][kw] = sum_{n,d,h,w} g[n][co][d][h][w] * x[n][ci][d+kd-pd][h+kh-ph][w+kw-pw]
//   gb[co]                 = sum_{n,d,h,w} g[n][co][d][h][w]
//
//   GEMM view   M = output channels, N = input channels (x depth taps), K = pixels.
//               Both operands are pixel-contiguous in the channels-first tensors, so
//               the tiles go to LDS untransposed. A 3-D problem is the 2-D one with
//               the depth taps folded into the x "channels": channel kd*Cin + ci of a
//               stage at output depth d is the plane x[n][ci][d + kd - pd].
//   MFMA roles  A = g (32 channels x 16 pixels of a row), B = x (16 pixels x 32
//               channels) shifted by the tap. The kw shift is not 16-byte aligned in
//               LDS, so a lane reads 10 consecutive pixels once (b128 + b32) and
//               builds the three kw fragments with funnel shifts.
//   Workgroup   one wavefront per (g channel block, x channel block, column half);
//               it keeps its 9 taps x 32x32 fp32 accumulators in registers for the
//               whole kernel (144 VGPRs) and walks the pixels. 64->64 2-D: 2x2x2 = 8
//               wavefronts (two per SIMD, which is what hides the barrier and LDS
//               write phases); 32->32 3-D: 1x3x2 = 6, plus two that only prefetch.
//   Stage       2 output rows x 64 columns; consecutive stages of a workgroup walk
//               down one column strip, so two of the four x rows a stage reads are
//               the previous stage's last two. The x rows therefore live in a ring of
//               6 rows per channel in LDS and a stage fetches only its two new rows
//               (each x element is read from memory once per strip, apart from the
//               8 halo columns), plus its two g rows (double buffered). Loads go
//               through registers and are issued a whole stage ahead. The first stage
//               of a strip or of a workgroup fetches its other two rows on the spot.
//               Channel strides in LDS are odd multiples of 16 bytes so that the 32
//               channel-lanes of a fragment read hit distinct banks.
//   Bias grad   the lanes that carry the g chunks to LDS add them up on the way
//               (fp32), one partial per workgroup and channel.
//   Reduction   every wavefront writes its partial to the workspace; a second kernel
//               sums the partials in a fixed order (deterministic) and writes gw in
//               the weight layout.
#include "conv_common.h"

namespace {

using jg::ConvGeom;
using jg::mfma_frame_bands;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

constexpr int SR = 2, SW = 64;        // output rows / columns per stage
constexpr int XR = SR + 2;            // x rows a stage reads
constexpr int RING = 6;               // x rows resident per channel
constexpr int G_CH = SR * SW * 2 + 16;        // 272 bytes per g channel
constexpr int X_ROW = 144;                    // 72 pixels
constexpr int X_CH = RING * X_ROW + 16;       // 880 bytes per x channel
constexpr int X_CPR = 8;                      // 8-pixel chunks per x row; 2 more pixels follow as one dword

struct WgradParams {
  const uint16_t* x;  // (N, Cin, Din, Hin, Win)
  const uint16_t* g;  // (N, Cout, Dout, Hout, Wout)
  const char* x_end;  // one past the last byte of x
  float* part;        // [wavefront slot][tap9][co][c']
  float* bias_part;   // [workgroup][co] or NULL
  // Framed input: xt (N, Cin, tn_d, tn_h, tn_w) is the own tile, at [tlo, tlo + tn) inside x.
  // A row pair whose window lies inside the tile is read from xt. NULL: all from x.
  const uint16_t* xt;
  int tlo_d, tlo_h, tlo_w, tn_d, tn_h, tn_w;
  int Cin, Cout;            // channels of the block this launch works on (32 or 64 a side)
  int cin_valid, cout_valid;  // how many of them exist; the others repeat the last one and are dropped
  int cin_total, cout_total;  // channels of the tensors (batch strides); x and g point at the block's first
  int Din, Hin, Win, Dout, Hout, Wout;
  int pad_d, pad_h, pad_w;
  int row_pairs, col_tiles;
  long long total_stages;  // N * Dout * col_tiles * row_pairs
  int w_first, w_last;     // what a stage of the first / last column strip costs, in stages of the other strips
  int wd_first, wd_last;   // the same for every stage of the first / last output depth (1: a plane like the others)
};

// Wavefronts per workgroup: (g block, x block) pairs x 2 column halves; a 6-wavefront
// shape gets two more wavefronts that only help with the prefetch.
constexpr int HALVES = 2;
constexpr int wgrad_threads(int cgb, int cxb) {
  return (cgb * cxb * HALVES > 4) ? 512 : 64 * cgb * cxb * HALVES;
}

// sum of the 8 bf16 values of a chunk
__device__ __forceinline__ float sum_bf16x8(const u32x4& v) {
  float s = __uint_as_float(v.x << 16) + __uint_as_float(v.x & 0xffff0000u);
  s += __uint_as_float(v.y << 16) + __uint_as_float(v.y & 0xffff0000u);
  s += __uint_as_float(v.z << 16) + __uint_as_float(v.z & 0xffff0000u);
  s += __uint_as_float(v.w << 16) + __uint_as_float(v.w & 0xffff0000u);
  return s;
}

// F16: x and g hold fp16 instead of bf16 (v_mfma_f32_32x32x16_f16); the partial sums are fp32 either way.
// EVEN: 0 = no assumption about the rows (every load checks its bounds), 1 = even row lengths,
// 4-byte aligned tensors and an even padding across W, so that a stage's windows start on dwords and
// the 16-byte vector loads apply, 2 = the same with an odd padding: the x window is staged from one
// pixel earlier, where it is dword aligned again, and the fragments are built one pixel further in.
// ALLIN: the host has checked that every window of every stage lies inside x and every stage's
// rows inside g (a convolution without padding over a tensor that holds its halo, tiles of whole
// stages): the kernel is built without the element-wise border path, and its stage loop loads and
// stores without conditions.
template <int CGB, int CXB, int EVEN, bool FRAMED, bool F16 = false, bool ALLIN = false>
__global__ __launch_bounds__(wgrad_threads(CGB, CXB)) void wgrad3x3_mfma_kernel(WgradParams p) {
  constexpr int THREADS = wgrad_threads(CGB, CXB);
  constexpr int LEAD = EVEN == 2 ? 1 : 0;
  static_assert(!(FRAMED && EVEN != 1), "the framed input is read with even windows only");
  constexpr int CWAVES = CGB * CXB * HALVES;  // wavefronts that own accumulators
  constexpr int GC = 32 * CGB, XC = 32 * CXB;
  constexpr int G_BYTES = GC * G_CH;          // one g buffer
  constexpr int G_CHUNKS = GC * SR * (SW / 8);
  constexpr int XP_CHUNKS = XC * 2 * X_CPR;   // one pair of x rows
  constexpr int CHUNKS = G_CHUNKS + XP_CHUNKS;
  constexpr int ROUNDS = (CHUNKS + THREADS - 1) / THREADS;
  static_assert(G_CHUNKS % THREADS == 0, "a load round holds g chunks or x chunks, never both");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char* const lds_x = smem + 2 * G_BYTES;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, kgp = lane >> 5;
  const int pair = wave % (CGB * CXB), half = (wave / (CGB * CXB)) % HALVES;
  const int cb = pair / CXB, ib = pair % CXB;

  // contiguous range of stages for this workgroup; stage -> (n, d, column tile, row pair),
  // row pair fastest, so consecutive stages walk down one column strip of one plane
  // Workgroups are dealt to the 8 XCDs round robin; the ranges are numbered so that one
  // XCD holds neighbouring column strips, whose x rows share cache lines in that XCD's L2.
  const unsigned wg_rank = gridDim.x % 8 == 0 ? (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8 : blockIdx.x;
  // The ranges hold equal cost, not equal counts: the stages of a column strip whose windows
  // stick out of the tensor (or whose last columns do not exist) load with bounds checks and
  // take several times as long, and a workgroup whose whole range lay in such a strip would set
  // the kernel's time. Cost runs like the stages: per plane the first strip at w_first a
  // stage, the middle strips at 1, the last at w_last; a plane at the first / last output depth
  // whose depth taps stick out is slow as a whole (wd_first / wd_last a stage). With all four at
  // 1 the ranges are counts.
  const long long strip_first = (long long)p.row_pairs * p.w_first;
  const long long strip_mid = (long long)p.row_pairs * (p.col_tiles > 2 ? p.col_tiles - 2 : 0);
  const long long strip_last = p.col_tiles > 1 ? (long long)p.row_pairs * p.w_last : 0;
  const long long plane_cost = strip_first + strip_mid + strip_last;
  const long long plane_stages = (long long)p.row_pairs * p.col_tiles;
  const long long head_cost = p.wd_first > 1 ? plane_stages * p.wd_first : plane_cost;
  const long long tail_cost = p.Dout > 1 ? (p.wd_last > 1 ? plane_stages * p.wd_last : plane_cost) : 0;
  const long long mid_cost = (p.Dout > 2 ? p.Dout - 2 : 0) * plane_cost;
  const long long entry_cost = head_cost + mid_cost + tail_cost;  // one batch entry
  const long long total_cost = (p.total_stages / (plane_stages * p.Dout)) * entry_cost;
  auto in_plane = [&](long long rem) -> long long {  // stage inside a plane of ordinary cost
    if (rem < strip_first) return rem / p.w_first;
    if (rem < strip_first + strip_mid) return p.row_pairs + (rem - strip_first);
    return (long long)p.row_pairs * (p.col_tiles - 1) + (rem - strip_first - strip_mid) / p.w_last;
  };
  auto stage_at = [&](long long cost) -> long long {
    if (cost >= total_cost) return p.total_stages;
    const long long n = cost / entry_cost;
    long long rem = cost - n * entry_cost, od, st;
    if (rem < head_cost) {
      od = 0;
      st = p.wd_first > 1 ? rem / p.wd_first : in_plane(rem);
    } else if (rem < head_cost + mid_cost) {
      rem -= head_cost;
      const long long k = rem / plane_cost;
      od = 1 + k;
      st = in_plane(rem - k * plane_cost);
    } else {
      rem -= head_cost + mid_cost;
      od = p.Dout - 1;
      st = p.wd_last > 1 ? rem / p.wd_last : in_plane(rem);
    }
    return (n * p.Dout + od) * plane_stages + st;
  };
  const long long per = (total_cost + gridDim.x - 1) / gridDim.x;
  const long long s_begin = stage_at(per * wg_rank);
  const long long s_end = stage_at(per * (wg_rank + 1));

  const size_t plane_x = (size_t)p.Hin * p.Win, plane_g = (size_t)p.Hout * p.Wout;
  const size_t x_cs = plane_x * p.Din, g_cs = plane_g * p.Dout;  // channel strides

  // ---- per-thread chunk bookkeeping, fixed for the whole kernel. Chunk q < G_CHUNKS
  // is 8 pixels of a g row, the others 8 pixels of one of the two x rows of a pair.
  uint32_t c_goff[ROUNDS];  // byte offset from the origin of its tensor window
  uint32_t c_lds[ROUNDS];   // byte offset inside the g buffer / inside the x ring, row slot 0
  uint32_t x_second = 0;    // bit rd: the chunk belongs to the second row of the pair
#pragma unroll
  for (int rd = 0; rd < ROUNDS; ++rd) {
    const int q = tid + rd * THREADS;
    if (q < G_CHUNKS) {
      const int c8 = q & 7, r = (q >> 3) % SR, ch = q / (8 * SR);
      const int che = ch < p.cout_valid ? ch : p.cout_valid - 1;  // a channel past the last one reads the last
      c_goff[rd] = (uint32_t)((che * g_cs + (size_t)r * p.Wout + c8 * 8) * 2);
      c_lds[rd] = (uint32_t)(ch * G_CH + r * (SW * 2) + c8 * 16);
    } else if (q < CHUNKS) {
      const int qx = q - G_CHUNKS;
      const int c8 = qx % X_CPR;
      const int rr = qx / X_CPR;
      const int r2 = rr & 1, ch = rr >> 1;      // ch = kd * Cin + ci
      const int kd = ch / p.Cin, cib = ch - kd * p.Cin;
      const int ci = cib < p.cin_valid ? cib : p.cin_valid - 1;
      c_goff[rd] = (uint32_t)((ci * x_cs + kd * plane_x + (size_t)r2 * p.Win + c8 * 8) * 2);
      c_lds[rd] = (uint32_t)(ch * X_CH + c8 * 16);
      x_second |= (uint32_t)r2 << rd;
    } else {
      c_goff[rd] = 0;
      c_lds[rd] = 0;
    }
  }
  // pixels 64, 65 of an x row (and 66, 67 of a window staged one pixel early): one or two dwords,
  // carried by the first 2 * XC threads
  const bool has_tail = tid < 2 * XC;
  uint32_t t_goff = 0, t_lds = 0;
  if (has_tail) {
    const int r2 = tid & 1, ch = tid >> 1;
    const int kd = ch / p.Cin, cib = ch - kd * p.Cin;
    const int ci = cib < p.cin_valid ? cib : p.cin_valid - 1;
    t_goff = (uint32_t)((ci * x_cs + kd * plane_x + (size_t)r2 * p.Win + SW) * 2);
    t_lds = (uint32_t)(ch * X_CH + SW * 2);
  }
  // the same x offsets inside the own tile (framed input)
  const size_t plane_t = (size_t)p.tn_h * p.tn_w, t_cs = plane_t * p.tn_d;
  uint32_t c_toff[ROUNDS];
  uint32_t t_toff = 0;
  uint32_t x_kd = 0;  // 2 bits per round: depth tap of the chunk; bits 30-31: of the tail
  if (FRAMED) {
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int q = tid + rd * THREADS;
      c_toff[rd] = 0;
      if (q >= G_CHUNKS && q < CHUNKS) {
        const int qx = q - G_CHUNKS;
        const int c8 = qx % X_CPR, rr = qx / X_CPR;
        const int r2 = rr & 1, ch = rr >> 1;
        const int kd = ch / p.Cin, ci = ch - kd * p.Cin;
        c_toff[rd] = (uint32_t)((ci * t_cs + kd * plane_t + (size_t)r2 * p.tn_w + c8 * 8) * 2);
        x_kd |= (uint32_t)kd << (2 * rd);
      }
    }
    if (has_tail) {
      const int r2 = tid & 1, ch = tid >> 1;
      const int kd = ch / p.Cin, ci = ch - kd * p.Cin;
      t_toff = (uint32_t)((ci * t_cs + kd * plane_t + (size_t)r2 * p.tn_w + SW) * 2);
      x_kd |= (uint32_t)kd << 30;
    }
  }

  struct Staged {
    u32x4 v[ROUNDS];
    uint32_t tail;
    uint32_t tail_b;  // LEAD only
  };

  // Loads of one stage into `v`: its two g rows (want_g) and one pair of its x rows
  // (pair 0: the rows shared with the stage above, pair 1: the two new rows).
  // Position of a stage: row pair (fastest), column tile, output depth, batch entry.
  // Decoded once with divisions, then stepped, so the stage loop has none.
  struct Cursor {
    int hp, ct, od, n;
  };
  auto decode = [&](long long stage) {
    Cursor c;
    c.hp = (int)(stage % p.row_pairs);
    long long t = stage / p.row_pairs;
    c.ct = (int)(t % p.col_tiles);
    t /= p.col_tiles;
    c.od = (int)(t % p.Dout);
    c.n = (int)(t / p.Dout);
    return c;
  };
  auto advance = [&](Cursor& c) {
    if (++c.hp == p.row_pairs) {
      c.hp = 0;
      if (++c.ct == p.col_tiles) {
        c.ct = 0;
        if (++c.od == p.Dout) {
          c.od = 0;
          ++c.n;
        }
      }
    }
  };

  auto issue_loads = [&](Staged& sg, const Cursor& cur, bool want_g, int xpair) {
    u32x4 (&v)[ROUNDS] = sg.v;
    const int hp = cur.hp, ct = cur.ct, od = cur.od, n = cur.n;
    const int oh0 = hp * SR, ow0 = ct * SW;
    const int id0 = od - p.pad_d, ih0 = oh0 - p.pad_h + 2 * xpair, iw0 = ow0 - p.pad_w - LEAD;
    const char* g_org = reinterpret_cast<const char*>(p.g) +
                        2 * (((size_t)n * p.cout_total * p.Dout + od) * plane_g + (size_t)oh0 * p.Wout + ow0);
    const char* x_org = reinterpret_cast<const char*>(p.x) +
                        2 * ((ptrdiff_t)((size_t)n * p.cin_total * p.Din * plane_x) + (ptrdiff_t)id0 * (ptrdiff_t)plane_x +
                             (ptrdiff_t)ih0 * p.Win + iw0);
    // (with LEAD the window's last dword holds one pixel more than is used; it shares its dword with one that is)
    const bool inside = ALLIN || (EVEN != 0 && oh0 + SR <= p.Hout && ow0 + SW <= p.Wout && ih0 >= 0 &&
                        ih0 + 2 <= p.Hin && iw0 >= 0 && iw0 + SW + 2 + LEAD <= p.Win && id0 >= 0 &&
                        id0 + (XC / p.Cin) <= p.Din);
    if (FRAMED && inside) {
      // Rows and columns of the pair's window inside the own tile (wave-uniform): a chunk
      // whose depth plane is a plane of the tile comes from the tile itself, at whatever
      // alignment its rows give the window; the planes outside the tile are halo planes,
      // which the frame holds whole.
      const int dt = id0 - p.tlo_d, ht = ih0 - p.tlo_h, wt = iw0 - p.tlo_w;
      if (ht >= 0 && ht + 2 <= p.tn_h && wt >= 0 && wt + SW + 2 <= p.tn_w) {
        const char* t_org = reinterpret_cast<const char*>(p.xt) +
                            2 * ((ptrdiff_t)((size_t)n * p.cin_total * t_cs) + (ptrdiff_t)dt * (ptrdiff_t)plane_t +
                                 (ptrdiff_t)ht * p.tn_w + wt);
        // 4-byte aligned accesses only (2-byte aligned vector loads run at a fraction of the
        // rate): a window that starts on an odd column is read one pixel early and shifted.
        // tn_w is even (checked on the host), so the parity is the same for every chunk.
        const bool odd = (reinterpret_cast<uintptr_t>(t_org) & 2) != 0;  // wave-uniform
        uint32_t lead[ROUNDS];
#pragma unroll
        for (int rd = 0; rd < ROUNDS; ++rd) {
          const int q = tid + rd * THREADS;
          lead[rd] = 0u;
          if (q < G_CHUNKS) {
            if (want_g) v[rd] = *reinterpret_cast<const u32x4_a4*>(g_org + c_goff[rd]);
          } else if (q < CHUNKS) {
            const int dd = dt + (int)((x_kd >> (2 * rd)) & 3u);
            if (dd >= 0 && dd < p.tn_d) {
              if (odd) {
                lead[rd] = *reinterpret_cast<const uint32_t*>(t_org + c_toff[rd] - 2);
                v[rd] = *reinterpret_cast<const u32x4_a4*>(t_org + c_toff[rd] + 2);
              } else {
                v[rd] = *reinterpret_cast<const u32x4_a4*>(t_org + c_toff[rd]);
              }
            } else {
              v[rd] = *reinterpret_cast<const u32x4_a4*>(x_org + c_goff[rd]);
            }
          }
        }
        uint32_t tail_lead = 0u;
        bool tail_shift = false;
        if (has_tail) {
          const int dd = dt + (int)(x_kd >> 30);
          if (dd >= 0 && dd < p.tn_d) {
            if (odd) {
              tail_lead = *reinterpret_cast<const uint32_t*>(t_org + t_toff - 2);
              sg.tail = *reinterpret_cast<const uint32_t*>(t_org + t_toff + 2);
              tail_shift = true;
            } else {
              sg.tail = *reinterpret_cast<const uint32_t*>(t_org + t_toff);
            }
          } else {
            sg.tail = *reinterpret_cast<const uint32_t*>(x_org + t_goff);
          }
        }
        if (odd) {
#pragma unroll
          for (int rd = 0; rd < ROUNDS; ++rd) {
            const int q = tid + rd * THREADS;
            if (q >= G_CHUNKS && q < CHUNKS) {
              const int dd = dt + (int)((x_kd >> (2 * rd)) & 3u);
              if (dd >= 0 && dd < p.tn_d) {
                const u32x4 t = v[rd];
                v[rd].x = __builtin_amdgcn_alignbit(t.x, lead[rd], 16);
                v[rd].y = __builtin_amdgcn_alignbit(t.y, t.x, 16);
                v[rd].z = __builtin_amdgcn_alignbit(t.z, t.y, 16);
                v[rd].w = __builtin_amdgcn_alignbit(t.w, t.z, 16);
              }
            }
          }
          if (tail_shift) sg.tail = __builtin_amdgcn_alignbit(sg.tail, tail_lead, 16);
        }
        return;
      }
    }
    if (inside) {
      // Every lane loads in every round it is asked for (the lanes past the last chunk and
      // those without a tail read offset 0 of the window, which is there): a load under a
      // per-lane condition merges the register with its old value, and the wait the
      // compiler puts before such a merge stands behind this stage's loads, which are
      // still in flight then.
#pragma unroll
      for (int rd = 0; rd < ROUNDS; ++rd) {
        const bool g_round = (rd + 1) * THREADS <= G_CHUNKS;  // THREADS divides G_CHUNKS
        if (want_g || !g_round) v[rd] = *reinterpret_cast<const u32x4_a4*>((g_round ? g_org : x_org) + c_goff[rd]);
      }
      sg.tail = *reinterpret_cast<const uint32_t*>(x_org + t_goff);
      if (LEAD) sg.tail_b = *reinterpret_cast<const uint32_t*>(x_org + t_goff + 4);
    } else {
#pragma unroll
      for (int rd = 0; rd < ROUNDS; ++rd) {
        const int q = tid + rd * THREADS;
        u32x4 val = {0u, 0u, 0u, 0u};
        if (q < CHUNKS && (want_g || q >= G_CHUNKS)) {
          const bool is_x = q >= G_CHUNKS;
          const uint16_t* src;
          int row, col, rows, cols;
          bool ok = true;
          if (!is_x) {
            const int c8 = q & 7, r = (q >> 3) % SR;
            src = reinterpret_cast<const uint16_t*>(g_org + c_goff[rd]);
            row = oh0 + r; col = ow0 + c8 * 8; rows = p.Hout; cols = p.Wout;
          } else {
            const int qx = q - G_CHUNKS;
            const int c8 = qx % X_CPR, rr = qx / X_CPR;
            const int r2 = rr & 1, ch = rr >> 1;
            src = reinterpret_cast<const uint16_t*>(x_org + c_goff[rd]);
            row = ih0 + r2; col = iw0 + c8 * 8; rows = p.Hin; cols = p.Win;
            const int dd = id0 + ch / p.Cin;
            ok = dd >= 0 && dd < p.Din;
          }
          if (ok && row >= 0 && row < rows) {
            if (col >= 0 && col + 8 <= cols && (reinterpret_cast<uintptr_t>(src) & 3) == 0) {
              val = *reinterpret_cast<const u32x4_a4*>(src);
            } else {
              uint32_t e[8];
#pragma unroll
              for (int k = 0; k < 8; ++k) e[k] = (col + k >= 0 && col + k < cols) ? (uint32_t)src[k] : 0u;
              val.x = e[0] | (e[1] << 16); val.y = e[2] | (e[3] << 16);
              val.z = e[4] | (e[5] << 16); val.w = e[6] | (e[7] << 16);
            }
          }
        }
        v[rd] = val;
      }
      if (has_tail) {
        const int r2 = tid & 1, ch = tid >> 1;
        const int row = ih0 + r2, col = iw0 + SW, dd = id0 + ch / p.Cin;
        const uint16_t* src = reinterpret_cast<const uint16_t*>(x_org + t_goff);
        uint32_t e[4] = {0u, 0u, 0u, 0u};
        if (dd >= 0 && dd < p.Din && row >= 0 && row < p.Hin) {
#pragma unroll
          for (int k = 0; k < 2 + 2 * LEAD; ++k)
            if (col + k >= 0 && col + k < p.Win) e[k] = src[k];
        }
        sg.tail = e[0] | (e[1] << 16);
        sg.tail_b = e[2] | (e[3] << 16);
      }
    }
  };

  // Registers of a stage to LDS: g rows into g buffer `gbuf`, the x pair into ring rows
  // `slot_a`, `slot_b`; the g chunks are added into the bias partials on the way.
  float bsum[ROUNDS];
#pragma unroll
  for (int rd = 0; rd < ROUNDS; ++rd) bsum[rd] = 0.0f;
  auto store_loads = [&](const Staged& sg, bool have_g, int gbuf, int slot_a, int slot_b, bool counted = true) {
    const u32x4 (&v)[ROUNDS] = sg.v;
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int q = tid + rd * THREADS;
      if (q < G_CHUNKS) {
        if (have_g) {
          *reinterpret_cast<u32x4*>(smem + gbuf * G_BYTES + c_lds[rd]) = v[rd];
          if (p.bias_part != nullptr) bsum[rd] += counted ? sum_bf16x8(v[rd]) : 0.0f;
        }
      } else if (q < CHUNKS) {
        const int slot = ((x_second >> rd) & 1u) ? slot_b : slot_a;
        *reinterpret_cast<u32x4*>(lds_x + c_lds[rd] + slot * X_ROW) = v[rd];
      }
    }
    if (has_tail) {
      unsigned char* at = lds_x + t_lds + ((tid & 1) ? slot_b : slot_a) * X_ROW;
      *reinterpret_cast<uint32_t*>(at) = sg.tail;
      if (LEAD) *reinterpret_cast<uint32_t*>(at + 4) = sg.tail_b;
    }
  };

  f32x16 acc[3][3];
#pragma unroll
  for (int a = 0; a < 3; ++a)
#pragma unroll
    for (int b = 0; b < 3; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.0f;

  // one 16-pixel column group (cgi = 0 or 1 of this wavefront's half) of a stage whose
  // four x rows sit in ring rows base .. base + 3 (mod RING): first all its LDS reads
  // (read_group), then its matrix instructions (mfma_group), so that a stage can ask for both
  // of its groups before the first matrix instruction and meets the LDS latency once.
  struct Frags {
    u32x4 a[SR];
    u32x4 d[XR];
    uint32_t d4[XR], d5[XR];
  };
  auto read_group = [&](Frags& f, int gbuf, int base, int cgi) __attribute__((always_inline)) {
    const unsigned char* gb = smem + gbuf * G_BYTES + (cb * 32 + ln) * G_CH + kgp * 16;
    const unsigned char* xb = lds_x + (ib * 32 + ln) * X_CH + kgp * 16;
    const int cg = half * (SW / 16 / HALVES) + cgi;  // 16-pixel column group of this wavefront
#pragma unroll
    for (int r = 0; r < SR; ++r) f.a[r] = *reinterpret_cast<const u32x4*>(gb + r * (SW * 2) + cg * 32);
#pragma unroll
    for (int rho = 0; rho < XR; ++rho) {
      int slot = base + rho;
      if (slot >= RING) slot -= RING;
      f.d[rho] = *reinterpret_cast<const u32x4*>(xb + slot * X_ROW + cg * 32);
      f.d4[rho] = *reinterpret_cast<const uint32_t*>(xb + slot * X_ROW + cg * 32 + 16);
      f.d5[rho] = 0u;
      if (LEAD) f.d5[rho] = *reinterpret_cast<const uint32_t*>(xb + slot * X_ROW + cg * 32 + 20);
    }
  };
  auto mfma_group = [&](Frags& f) __attribute__((always_inline)) {
    bf16x8 a[SR];
#pragma unroll
    for (int r = 0; r < SR; ++r) a[r] = __builtin_bit_cast(bf16x8, f.a[r]);
#pragma unroll
    for (int rho = 0; rho < XR; ++rho) {
      u32x4 d = f.d[rho];
      uint32_t d4 = f.d4[rho], d5 = f.d5[rho];
      // The values are made opaque so that the kw = 2 fragment below is built with register
      // moves: left alone, the compiler reads it again from LDS at a 4-byte offset, as dword
      // pairs whose 880-byte lane stride runs into 4-way bank conflicts.
      asm("" : "+v"(d), "+v"(d4), "+v"(d5));
      u32x4 s1, s2;
      s1.x = __builtin_amdgcn_alignbit(d.y, d.x, 16);
      s1.y = __builtin_amdgcn_alignbit(d.z, d.y, 16);
      s1.z = __builtin_amdgcn_alignbit(d.w, d.z, 16);
      s1.w = __builtin_amdgcn_alignbit(d4, d.w, 16);
      s2.x = d.y; s2.y = d.z; s2.z = d.w; s2.w = d4;
      u32x4 s3;  // LEAD: the window was staged one pixel early, the taps sit one pixel further in
      s3.x = __builtin_amdgcn_alignbit(d.z, d.y, 16);
      s3.y = __builtin_amdgcn_alignbit(d.w, d.z, 16);
      s3.z = __builtin_amdgcn_alignbit(d4, d.w, 16);
      s3.w = __builtin_amdgcn_alignbit(d5, d4, 16);
      const bf16x8 b0 = __builtin_bit_cast(bf16x8, LEAD ? s1 : d);
      const bf16x8 b1 = __builtin_bit_cast(bf16x8, LEAD ? s2 : s1);
      const bf16x8 b2 = __builtin_bit_cast(bf16x8, LEAD ? s3 : s2);
#pragma unroll
      for (int r = 0; r < SR; ++r) {
        const int kh = rho - r;
        if (kh >= 0 && kh < 3) {
          if (F16) {
            const f16x8 ah = __builtin_bit_cast(f16x8, a[r]);
            acc[kh][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, __builtin_bit_cast(f16x8, b0), acc[kh][0], 0, 0, 0);
            acc[kh][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, __builtin_bit_cast(f16x8, b1), acc[kh][1], 0, 0, 0);
            acc[kh][2] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, __builtin_bit_cast(f16x8, b2), acc[kh][2], 0, 0, 0);
          } else {
            acc[kh][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r], b0, acc[kh][0], 0, 0, 0);
            acc[kh][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r], b1, acc[kh][1], 0, 0, 0);
            acc[kh][2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r], b2, acc[kh][2], 0, 0, 0);
          }
        }
      }
    }
  };
  auto compute_group = [&](int gbuf, int base, int cgi) {
    Frags f;
    read_group(f, gbuf, base, cgi);
    mfma_group(f);
  };

  // Stage k of this workgroup reads ring rows base_k .. base_k + 3 with base_k = 2k mod 6:
  // its first two rows are where the stage before put its new rows (base_k-1 + 2, + 3), its
  // new rows go to base_k + 2, + 3. A stage that does not continue the strip of the stage
  // before fetches its first two rows itself, into those same ring rows.
  static_assert(SW / 16 / HALVES == 2, "the stage loop is written for two column groups per wavefront");
  auto wrap = [](int v) { return v >= RING ? v - RING : v; };
  if (s_begin < s_end) {
    Staged stg;
    int gbuf = 0, base = 0;
    Cursor c_next = decode(s_begin);  // stage whose loads are issued next
    issue_loads(stg, c_next, true, 1);
    store_loads(stg, true, 0, 2, 3);
    issue_loads(stg, c_next, false, 0);
    store_loads(stg, false, 0, 0, 1);
    if constexpr (ALLIN) {
      // The loads of a stage are issued, and the registers of the stage before stored, in EVERY
      // stage: the cursor stops at the workgroup's last stage, which the last two stages fetch
      // again for nothing, and what the last stage stores nobody reads. A load or a store under
      // a condition leaves the staged registers with two possible states where the paths meet;
      // the compiler then waits for the loads at the end of the stage that issued them (to copy
      // the registers together) instead of where they are stored, half a stage later.
      if (s_begin + 1 < s_end) advance(c_next);
      Cursor c_store = c_next;          // stage whose registers are stored next (st + 1)
      issue_loads(stg, c_next, true, 1);
      if (s_begin + 2 < s_end) advance(c_next);
      __syncthreads();
      // Wavefronts w and w + 4 share a SIMD and would do everything at the same time: both issue
      // matrix instructions, then both store and load while the matrix core idles (measured with
      // the cycle counter: 1150 cycles of a 4400-cycle stage spent by the older wavefront of each
      // SIMD waiting at the barrier for the younger one). So the two take the stage's halves in
      // opposite order: w multiplies while w + 4 stores the registers of the next stage and
      // issues the loads of the one after, then the other way round. What is stored goes to the
      // g buffer and the ring rows that no wavefront reads in this stage.
      // (With six multiplying wavefronts, two SIMDs hold a wavefront that only stages; there the
      // split measured slower, and every wavefront stores and loads between its two groups.)
      const bool stage_first = CWAVES == 8 && (wave & 4) != 0;
      for (long long st = s_begin; st < s_end; ++st) {
        Frags f0, f1;
        if (stage_first) {
          store_loads(stg, true, gbuf ^ 1, wrap(base + 4), wrap(base + 5), st + 1 < s_end);
          issue_loads(stg, c_next, true, 1);
        }
        if (wave < CWAVES) {
          read_group(f0, gbuf, base, 0);
          read_group(f1, gbuf, base, 1);
          mfma_group(f0);
          if (CWAVES == 8) mfma_group(f1);
        }
        if (!stage_first) {
          store_loads(stg, true, gbuf ^ 1, wrap(base + 4), wrap(base + 5), st + 1 < s_end);
          issue_loads(stg, c_next, true, 1);
        }
        if (CWAVES != 8 && wave < CWAVES) mfma_group(f1);
        if (st + 3 < s_end) advance(c_next);
        __syncthreads();
        if (st + 1 < s_end && c_store.hp == 0) {
          // the next stage starts a new strip: its first two x rows, on the spot
          Staged top;
          issue_loads(top, c_store, false, 0);
          store_loads(top, false, 0, wrap(base + 2), wrap(base + 3));
          // These loads have all been stored, but the tail's under a per-lane condition: where
          // the compiler cannot see a load waited for on every path, it waits at the loop's end,
          // and that wait takes the stage's own loads with it. vmcnt(0), said once, here:
          __builtin_amdgcn_s_waitcnt(0x0F70);
          __syncthreads();
        }
        advance(c_store);
        base = wrap(base + 2);
        gbuf ^= 1;
      }
    } else {
      advance(c_next);
      Cursor c_store = c_next;          // stage whose registers are stored next (st + 1)
      if (s_begin + 1 < s_end) {
        issue_loads(stg, c_next, true, 1);
        advance(c_next);
      }
      __syncthreads();
      for (long long st = s_begin; st < s_end; ++st) {
        if (wave < CWAVES) compute_group(gbuf, base, 0);
        if (st + 1 < s_end) store_loads(stg, true, gbuf ^ 1, wrap(base + 4), wrap(base + 5));
        if (st + 2 < s_end) {
          issue_loads(stg, c_next, true, 1);
          advance(c_next);
        }
        if (wave < CWAVES) compute_group(gbuf, base, 1);
        __syncthreads();
        if (st + 1 < s_end && c_store.hp == 0) {
          // the next stage starts a new strip: its first two x rows, on the spot
          Staged top;
          issue_loads(top, c_store, false, 0);
          store_loads(top, false, 0, wrap(base + 2), wrap(base + 3));
          __syncthreads();
        }
        advance(c_store);
        base = wrap(base + 2);
        gbuf ^= 1;
      }
    }
  }

  // bias partial of this workgroup: the 16 lanes that carried a channel's chunks add up
  if (p.bias_part != nullptr) {
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int q = tid + rd * THREADS;
      if (rd * THREADS < G_CHUNKS) {  // rounds that hold g chunks (whole rounds: THREADS divides G_CHUNKS)
        float s = bsum[rd];
        s += __shfl_xor(s, 8, 64);
        s += __shfl_xor(s, 4, 64);
        s += __shfl_xor(s, 2, 64);
        s += __shfl_xor(s, 1, 64);
        if (q < G_CHUNKS && (tid & 15) == 0) p.bias_part[(size_t)blockIdx.x * GC + q / (8 * SR)] = s;
      }
    }
  }

  // partial of this wavefront: slot = workgroup * HALVES + half, layout [tap9][co][c']
  if (wave >= CWAVES) return;
  float* out = p.part + ((size_t)blockIdx.x * HALVES + half) * (size_t)(9 * GC * XC);
#pragma unroll
  for (int kh = 0; kh < 3; ++kh)
#pragma unroll
    for (int kw = 0; kw < 3; ++kw)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int co = cb * 32 + 8 * (i >> 2) + 4 * kgp + (i & 3);
        out[((kh * 3 + kw) * GC + co) * XC + ib * 32 + ln] = acc[kh][kw][i];
      }
}

// gb[co] (bf16) = sum over the workgroups of bias_part[wg][co]; one wavefront per channel,
// fixed order. GC = channels per partial row, `valid` of them exist.
__global__ __launch_bounds__(256) void wgrad_bias_reduce_kernel(uint16_t* __restrict__ gb,
                                                                const float* __restrict__ part,
                                                                int wgs, int GC, int valid) {
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (c >= valid) return;
  float s = 0.0f;
  for (int k = lane; k < wgs; k += 64) s += part[(size_t)k * GC + c];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if (lane == 0) gb[c] = jg::f32_to_bf16(s);
}

// gw[co0 + co][ci0 + ci][kd][kh][kw] (bf16) = sum over the slots of
// part[slot][tap9][co][kd*CinB+ci] for the channels of the block that exist (gw points at
// the block's first element, cin_total is the channel count of the whole weight tensor).
// A block owns 64 consecutive outputs (one per lane, so a slot row is read coalesced);
// its 4 wavefronts take the slots s = w, w + 4, ... in 4 independent chains each, and the
// 16 chain sums are added in a fixed order (deterministic).
template <bool OUT32>
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(void* __restrict__ gw_out,
                                                           const float* __restrict__ part,
                                                           int slots, int GC, int XC, int CinB,
                                                           int cout_valid, int cin_valid, int cin_total, int accumulate) {
  __shared__ float red[4][64];
  const int count = 9 * GC * XC;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + lane;  // index in [tap9][co][c']
  float c0 = 0.f, c1 = 0.f, c2 = 0.f, c3 = 0.f;
  if (i < count) {
    int k = w;
    for (; k + 12 < slots; k += 16) {
      c0 += part[(size_t)(k + 0) * count + i];
      c1 += part[(size_t)(k + 4) * count + i];
      c2 += part[(size_t)(k + 8) * count + i];
      c3 += part[(size_t)(k + 12) * count + i];
    }
    for (; k < slots; k += 4) c0 += part[(size_t)k * count + i];
  }
  red[w][lane] = (c0 + c1) + (c2 + c3);
  __syncthreads();
  if (w != 0 || i >= count) return;
  const float s = (red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane]);
  const int cx = i % XC, co = (i / XC) % GC, tap = i / (XC * GC);
  const int kd = cx / CinB, ci = cx % CinB, KD = XC / CinB;
  if (co >= cout_valid || ci >= cin_valid) return;
  const size_t at = (((size_t)co * cin_total + ci) * KD + kd) * 9 + tap;
  if (OUT32) {
    // split mode: the six part products of a block are added up here, one launch after the other
    float* gw = static_cast<float*>(gw_out);
    gw[at] = accumulate ? gw[at] + s : s;
  } else {
    static_cast<uint16_t*>(gw_out)[at] = jg::f32_to_bf16(s);
  }
}

// gw[co][ci][t] (fp32) = sum over the part pairs (i, j), i + j <= parts - 1, smallest first, of
// tmp[i * cout + co][j * cin + ci][t]: the part products of the split mode from one launch.
__global__ __launch_bounds__(256) void wgrad_combine_parts_kernel(float* __restrict__ gw, const float* __restrict__ tmp,
                                                                  int cout, int cin, int taps, int parts) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= cout * cin * taps) return;
  const int t = idx % taps, ci = (idx / taps) % cin, co = idx / (taps * cin);
  float sum = 0.0f;
  for (int order = parts - 1; order >= 0; --order)
    for (int i = 0; i <= order; ++i) {
      const int j = order - i;
      sum += tmp[((size_t)(i * cout + co) * (parts * cin) + (j * cin + ci)) * taps + t];
    }
  gw[idx] = sum;
}

__global__ __launch_bounds__(256) void f32_to_f16_kernel(_Float16* __restrict__ dst, const float* __restrict__ src, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = (_Float16)src[i];
}

int cu_count() {
  static int cached = 0;
  if (cached) return cached;
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
    n = 256;
  cached = n;
  return n;
}

int wg_count(long long stages) {
  long long n = cu_count();
  if (n > stages) n = stages;
  if (n < 1) n = 1;
  return (int)n;
}

long long stage_count(const ConvGeom& g) {
  return g.batch * g.out[0] * ((g.out[1] + SR - 1) / SR) * ((g.out[2] + SW - 1) / SW);
}

// (CGB, CXB) of a geometry, or false when the kernel does not cover it
// Channel blocking. One launch accumulates a block of `cob` output x `cib` input channels
// (32 or 64 each; with a depth kernel of 3 always 32 x 32, so that the x side spans 96);
// more channels are covered block by block, a last block with fewer channels than its
// width re-reads its last channel and its extra rows and columns are dropped.
struct Blocking {
  int cob, cib;  // width of the first (largest) block
  int KD;
  int cob_max() const { return KD == 3 ? 32 : 64; }
  int cib_max() const { return KD == 3 ? 32 : 64; }
};
bool blocks_of(const ConvGeom& g, Blocking* b) {
  if (g.groups != 1) return false;
  if (g.k[1] != 3 || g.k[2] != 3 || (g.k[0] != 1 && g.k[0] != 3)) return false;
  if (g.k[0] == 1 && g.in[0] != 1) return false;
  for (int a = 0; a < 3; ++a)
    if (g.s[a] != 1 || g.d[a] != 1) return false;
  if (g.cin <= 0 || g.cout <= 0) return false;
  b->KD = g.k[0];
  if (b->KD == 3) {
    b->cob = 32; b->cib = 32;
  } else {
    b->cob = g.cout > 32 ? 64 : 32;
    b->cib = g.cin > 32 ? 64 : 32;
  }
  // per-lane byte offsets inside one batch entry are 32-bit
  const size_t xs = (size_t)g.cin * g.in[0] * g.in[1] * g.in[2] * 2;
  const size_t gs = (size_t)g.cout * g.out[0] * g.out[1] * g.out[2] * 2;
  return xs < (1ull << 31) && gs < (1ull << 31);
}
// width of the block that starts at channel c0 of `total`
int block_width(int total, int c0, int first) { return (first == 64 && total - c0 > 32) ? 64 : 32; }

template <int CGB, int CXB>
int launch(const WgradParams& p, int even, bool f16, bool all_inside, int wgs, hipStream_t s, const char* who) {
  constexpr int THREADS = wgrad_threads(CGB, CXB);
  const size_t lds = 2 * (size_t)(32 * CGB * G_CH) + (size_t)(32 * CXB * X_CH);
  void (*kern)(WgradParams);
  if (f16)  // never framed (checked by the caller)
    kern = even == 1 ? &wgrad3x3_mfma_kernel<CGB, CXB, 1, false, true>
                     : (even == 2 ? &wgrad3x3_mfma_kernel<CGB, CXB, 2, false, true> : &wgrad3x3_mfma_kernel<CGB, CXB, 0, false, true>);
  else if (p.xt != nullptr)
    kern = &wgrad3x3_mfma_kernel<CGB, CXB, 1, true>;  // the framed input needs the even layout (checked by the caller)
  else if (all_inside && even == 1)
    kern = &wgrad3x3_mfma_kernel<CGB, CXB, 1, false, false, true>;
  else
    kern = even == 1 ? &wgrad3x3_mfma_kernel<CGB, CXB, 1, false>
                     : (even == 2 ? &wgrad3x3_mfma_kernel<CGB, CXB, 2, false> : &wgrad3x3_mfma_kernel<CGB, CXB, 0, false>);
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) JG_FAIL(JG_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", who, lds);
  kern<<<wgs, THREADS, lds, s>>>(p);
  return JG_OK;
}

}  // namespace

namespace jg {

// fp32 is split into three bf16 parts per operand; fp16 has its own MFMA instruction and runs like bf16
static int parts_of(int dtype) { return dtype == JG_F32 ? 3 : 1; }
// Split mode with few channels: the parts of both operands fit one block.
static bool parts_fit_one_block(const ConvGeom& g, const Blocking& bl, int parts) {
  return parts > 1 && parts * g.cout <= bl.cob_max() && parts * g.cin <= bl.cib_max();
}
static size_t parts_tmp_bytes(const ConvGeom& g, const Blocking& bl, int parts) {
  if (!parts_fit_one_block(g, bl, parts)) return 0;
  return ((size_t)parts * parts * g.cout * g.cin * bl.KD * 9 * sizeof(float) + 255) / 256 * 256;
}
// fp16: the gradient is reduced into fp32 here before the one rounding to fp16
static size_t acc32_bytes(const ConvGeom& g, int dtype) {
  return dtype == JG_F16 ? ((size_t)g.cout * g.cin * g.k[0] * 9 * sizeof(float) + 255) / 256 * 256 : 0;
}

// fp32 runs in split mode: both operands are copied as three bf16 parts each (as extra channels) and
// the six part products whose indices add up to at most 2 are accumulated in fp32.
bool mfma_wgrad_supported(const ConvGeom& g, int dtype) {
  Blocking b;
  if ((dtype != JG_BF16 && dtype != JG_F32 && dtype != JG_F16) || g.batch <= 0) return false;
  return blocks_of(g, &b);
}

static size_t partial_bytes(const ConvGeom& g) {
  Blocking b{32, 32, 1};
  blocks_of(g, &b);
  const size_t wgs = (size_t)wg_count(stage_count(g));
  // sized for the widest block any mode launches
  const size_t n = wgs * HALVES * 9 * b.cob_max() * (b.KD * b.cib_max()) * sizeof(float) + wgs * b.cob_max() * sizeof(float);
  return (n + 255) / 256 * 256;
}
static size_t split_copy_bytes(size_t elements, int parts) { return (elements * parts * 2 + 255) / 256 * 256; }
// workspace: [partials | fp32 sum (fp16 only) | x parts | g parts (fp32 only) | part products of the one-block launch]
size_t mfma_wgrad_workspace(const ConvGeom& g, int dtype) {
  size_t n = partial_bytes(g);
  const int parts = parts_of(dtype);
  n += acc32_bytes(g, dtype);  // fp16 only, directly behind the partial sums
  if (parts > 1) {
    n += split_copy_bytes((size_t)g.batch * g.cin * g.in[0] * g.in[1] * g.in[2], parts);
    n += split_copy_bytes((size_t)g.batch * g.cout * g.out[0] * g.out[1] * g.out[2], parts);
    Blocking b{32, 32, 1};
    blocks_of(g, &b);
    n += parts_tmp_bytes(g, b, parts);
  }
  return n;
}

// Whether the framed weight-gradient kernel covers a geometry: even row lengths (its
// vector loads), and every row pair / column tile whose window leaves the own tile lies
// inside the bands that the frame holds.
bool mfma_wgrad_frame_ok(const ConvGeom& g, const int tlo[3], const int tn[3]) {
  if (g.in[2] % 2 != 0 || g.p[2] % 2 != 0 || g.out[2] % 2 != 0 || tn[2] % 2 != 0) return false;
  Blocking b;  // the framed input is read by a single block of exactly its width
  if (!blocks_of(g, &b) || g.cin != b.cib || g.cout != b.cob) return false;
  int blo[3], bhi[3];
  mfma_frame_bands(g, tlo, tn, blo, bhi);
  const int row_pairs = (g.out[1] + SR - 1) / SR, col_tiles = (g.out[2] + SW - 1) / SW;
  for (int j = 0; j < row_pairs + 1; ++j) {  // x row pairs of all stages: [2j - pad, 2j - pad + 2)
    const int r = 2 * j - g.p[1];
    const bool in_tile = r >= tlo[1] && r + 2 <= tlo[1] + tn[1];
    const int r_end = r + 2 < g.in[1] ? r + 2 : g.in[1];  // what lies past the tensor is not read
    const bool in_band = r_end <= blo[1] || r >= g.in[1] - bhi[1];
    if (!in_tile && !in_band) return false;
  }
  for (int ct = 0; ct < col_tiles; ++ct) {
    const int c = ct * SW - g.p[2];
    const bool in_tile = c >= tlo[2] && c + SW + 2 <= tlo[2] + tn[2];
    const int c_end = c + SW + 2 < g.in[2] ? c + SW + 2 : g.in[2];
    const bool in_band = c_end <= blo[2] || c >= g.in[2] - bhi[2];
    if (!in_tile && !in_band) return false;
  }
  return true;
}

int mfma_wgrad(void* gw, void* gb, const void* x, const void* go, const ConvGeom& g, void* ws,
               size_t ws_bytes, hipStream_t s, const void* xt, const int* tlo, const int* tn, int dtype) {
  const char* who = "jg_conv_wgrad(mfma)";
  Blocking bl;
  if (!blocks_of(g, &bl)) JG_FAIL(JG_ERR_UNSUPPORTED, "%s: geometry not covered", who);
  if (ws == nullptr || ws_bytes < mfma_wgrad_workspace(g, dtype))
    JG_FAIL(JG_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes,
            mfma_wgrad_workspace(g, dtype));
  JG_REQUIRE((reinterpret_cast<uintptr_t>(ws) & 15) == 0, "%s: workspace must be 16-byte aligned",
             who);
  const size_t x_cs = (size_t)g.in[0] * g.in[1] * g.in[2], g_cs = (size_t)g.out[0] * g.out[1] * g.out[2];
  const int parts = parts_of(dtype);
  const bool split = parts > 1;
  const bool f16 = dtype == JG_F16;
  float* sum32 = static_cast<float*>(gw);  // where the part products are added up (split mode)
  float* one_block_tmp = nullptr;
  if ((split || f16) && (gb != nullptr || xt != nullptr))
    JG_FAIL(JG_ERR_UNSUPPORTED, "%s: fp32 / fp16 have neither the fused bias gradient nor the framed input", who);
  if (f16) sum32 = reinterpret_cast<float*>(static_cast<char*>(ws) + partial_bytes(g));
  if (split) {
    char* base = static_cast<char*>(ws) + partial_bytes(g);
    uint16_t* xs = reinterpret_cast<uint16_t*>(base);
    base += split_copy_bytes((size_t)g.batch * g.cin * x_cs, parts);
    uint16_t* gs = reinterpret_cast<uint16_t*>(base);
    base += split_copy_bytes((size_t)g.batch * g.cout * g_cs, parts);
    one_block_tmp = reinterpret_cast<float*>(base);
    int rc = split_parts_bf16(xs, x, dtype, (size_t)g.batch, (size_t)g.cin * x_cs, s);
    if (rc) return rc;
    rc = split_parts_bf16(gs, go, dtype, (size_t)g.batch, (size_t)g.cout * g_cs, s);
    if (rc) return rc;
    x = xs;
    go = gs;
  }
  // 0, 1 or 2: the EVEN mode of the kernel (2: odd padding across W, windows staged one pixel early)
  const bool even_rows = (g.in[2] % 2 == 0) && (g.out[2] % 2 == 0) && ((reinterpret_cast<uintptr_t>(x) & 3) == 0) &&
                         ((reinterpret_cast<uintptr_t>(go) & 3) == 0);
  const int even = !even_rows ? 0 : (g.p[2] % 2 == 0 ? 1 : 2);
  if (xt != nullptr && (even != 1 || !mfma_wgrad_frame_ok(g, tlo, tn)))
    JG_FAIL(JG_ERR_UNSUPPORTED, "%s: the framed input does not cover this geometry / alignment", who);
  // part products (g part, x part), smallest first; plain mode: the one product
  static const int kPairs[6][2] = {{0, 2}, {1, 1}, {2, 0}, {0, 1}, {1, 0}, {0, 0}};
  const int npairs = parts == 3 ? 6 : (parts == 2 ? 3 : 1), first_pair = 6 - npairs;
  const int gw_count = g.cout * g.cin * g.k[0] * 9;
  auto finish = [&]() -> int {  // fp16: the one rounding of the fp32 sum
    if (dtype == JG_F16) {
      f32_to_f16_kernel<<<(gw_count + 255) / 256, 256, 0, s>>>(static_cast<_Float16*>(gw), sum32, gw_count);
      JG_CHECK_LAUNCH(who);
    }
    return JG_OK;
  };
  WgradParams p;
  p.part = static_cast<float*>(ws);
  p.x_end = static_cast<const char*>(x) + 2 * (size_t)g.batch * parts * g.cin * x_cs;
  p.cin_total = parts * g.cin; p.cout_total = parts * g.cout;
  p.Din = g.in[0]; p.Hin = g.in[1]; p.Win = g.in[2];
  p.Dout = g.out[0]; p.Hout = g.out[1]; p.Wout = g.out[2];
  p.pad_d = g.p[0]; p.pad_h = g.p[1]; p.pad_w = g.p[2];
  p.row_pairs = (g.out[1] + SR - 1) / SR;
  p.col_tiles = (g.out[2] + SW - 1) / SW;
  p.total_stages = stage_count(g);
  {
    // column strips outside the kernel's vector-load path (see the kernel's `inside`)
    const int last_ow0 = (p.col_tiles - 1) * SW;
    const bool first_slow = g.p[2] > 0;
    const int lead = even == 2 ? 1 : 0;
    const bool last_slow = last_ow0 + SW > g.out[2] || last_ow0 - g.p[2] - lead + SW + 2 + lead > g.in[2];
    p.w_first = p.w_last = p.wd_first = p.wd_last = 1;
    // measured: such a stage costs about four plain ones; 3 gave the shortest kernels over the shapes tried
    constexpr int SLOW = 3;
    if (even) {  // without the even layout every stage takes that path
      if (p.col_tiles == 1) p.w_first = (first_slow || last_slow) ? SLOW : 1;
      else { p.w_first = first_slow ? SLOW : 1; p.w_last = last_slow ? SLOW : 1; }
      // output depths whose depth taps reach outside x: all their stages take that path
      const bool head_slow = g.p[0] > 0, tail_slow = g.out[0] - 1 - g.p[0] + g.k[0] > g.in[0];
      if (g.out[0] == 1) p.wd_first = (head_slow || tail_slow) ? SLOW : 1;
      else { p.wd_first = head_slow ? SLOW : 1; p.wd_last = tail_slow ? SLOW : 1; }
    }
  }
  // Every stage whole and every window inside x: the kernel without the border path (see ALLIN).
  const bool all_inside = even == 1 && xt == nullptr && g.p[0] == 0 && g.p[1] == 0 && g.p[2] == 0 &&
                          g.out[1] % SR == 0 && g.out[2] % SW == 0 && g.out[1] + 2 <= g.in[1] &&
                          g.out[2] + 2 <= g.in[2] && g.out[0] - 1 + g.k[0] <= g.in[0];
  const int wgs = wg_count(p.total_stages);
  p.xt = static_cast<const uint16_t*>(xt);
  p.tlo_d = tlo ? tlo[0] : 0; p.tlo_h = tlo ? tlo[1] : 0; p.tlo_w = tlo ? tlo[2] : 0;
  p.tn_d = tn ? tn[0] : 0; p.tn_h = tn ? tn[1] : 0; p.tn_w = tn ? tn[2] : 0;
  // One block of channels: g channels [gch, gch + cout_valid), x channels [xch, xch + cin_valid) of the
  // tensors as they lie in memory (split mode: parts are channel groups), into out (+ gb_out).
  auto run_block = [&](size_t gch, size_t xch, int cob, int cib, int cout_valid, int cin_valid, void* out,
                       int out_cin_total, bool out32, bool accumulate, uint16_t* gb_out) -> int {
    const int cgb = cob / 32, cxb = bl.KD * cib / 32;
    p.Cin = cib; p.Cout = cob;
    p.cin_valid = cin_valid; p.cout_valid = cout_valid;
    p.x = static_cast<const uint16_t*>(x) + xch * x_cs;
    p.g = static_cast<const uint16_t*>(go) + gch * g_cs;
    p.bias_part = gb_out != nullptr ? p.part + (size_t)wgs * HALVES * 9 * cob * (bl.KD * cib) : nullptr;
    int rc;
    if (cgb == 2 && cxb == 2) rc = launch<2, 2>(p, even, f16, all_inside, wgs, s, who);
    else if (cgb == 1 && cxb == 3) rc = launch<1, 3>(p, even, f16, all_inside, wgs, s, who);
    else if (cgb == 1 && cxb == 1) rc = launch<1, 1>(p, even, f16, all_inside, wgs, s, who);
    else if (cgb == 2 && cxb == 1) rc = launch<2, 1>(p, even, f16, all_inside, wgs, s, who);
    else if (cgb == 1 && cxb == 2) rc = launch<1, 2>(p, even, f16, all_inside, wgs, s, who);
    else JG_FAIL(JG_ERR_UNSUPPORTED, "%s: channel blocking (%d, %d) not built", who, cgb, cxb);
    if (rc) return rc;
    JG_CHECK_LAUNCH(who);
    const int count = 9 * cob * bl.KD * cib;
    if (out32)
      wgrad_reduce_kernel<true><<<(count + 63) / 64, 256, 0, s>>>(out, p.part, wgs * HALVES, cob, bl.KD * cib, cib,
                                                                    cout_valid, cin_valid, out_cin_total, accumulate);
    else
      wgrad_reduce_kernel<false><<<(count + 63) / 64, 256, 0, s>>>(out, p.part, wgs * HALVES, cob, bl.KD * cib, cib,
                                                                     cout_valid, cin_valid, out_cin_total, 0);
    JG_CHECK_LAUNCH(who);
    if (gb_out != nullptr) {
      wgrad_bias_reduce_kernel<<<(cob + 3) / 4, 256, 0, s>>>(gb_out, p.bias_part, wgs, cob, cout_valid);
      JG_CHECK_LAUNCH(who);
    }
    return JG_OK;
  };

  if (parts_fit_one_block(g, bl, parts)) {
    // few channels: all part products in one launch (the parts are parts x cout and parts x cin
    // channels of one block), then the ones that count are added up
    const int cob = parts * g.cout > 32 ? 64 : 32, cib = parts * g.cin > 32 ? 64 : 32;  // within the block limits (checked)
    int rc = run_block(0, 0, cob, cib, parts * g.cout, parts * g.cin, one_block_tmp, parts * g.cin, true, false, nullptr);
    if (rc) return rc;
    wgrad_combine_parts_kernel<<<(gw_count + 255) / 256, 256, 0, s>>>(sum32, one_block_tmp, g.cout, g.cin, bl.KD * 9,
                                                                      parts);
    JG_CHECK_LAUNCH(who);
    return finish();
  }
  for (int co0 = 0; co0 < g.cout;) {
    const int cob = block_width(g.cout, co0, bl.cob);
    for (int ci0 = 0; ci0 < g.cin;) {
      const int cib = block_width(g.cin, ci0, bl.cib);
      const int cin_valid = g.cin - ci0 < cib ? g.cin - ci0 : cib;
      const int cout_valid = g.cout - co0 < cob ? g.cout - co0 : cob;
      const size_t blk_at = ((size_t)co0 * g.cin + ci0) * bl.KD * 9;
      for (int pr = 0; pr < npairs; ++pr) {
        const int gpart = kPairs[first_pair + pr][0], xpart = kPairs[first_pair + pr][1];
        void* out = (split || f16) ? static_cast<void*>(sum32 + blk_at)
                                   : static_cast<void*>(static_cast<uint16_t*>(gw) + blk_at);
        // the bias gradient comes from the g rows: once per block of output channels
        uint16_t* gb_out = (gb != nullptr && ci0 == 0) ? static_cast<uint16_t*>(gb) + co0 : nullptr;
        int rc = run_block((size_t)gpart * g.cout + co0, (size_t)xpart * g.cin + ci0, cob, cib, cout_valid, cin_valid,
                           out, g.cin, split || f16, pr > 0, gb_out);
        if (rc) return rc;
      }
      ci0 += cib;
    }
    co0 += cob;
  }
  return finish();
}

}  // namespace jg
