// Halo movement for the halo-exchange convolution: assemble (own tile + up to
// 26 neighbour strips -> zero-padded tile), pack (cut the strips a rank sends)
// and fold (padded gradient + neighbour strips -> owned gradient, in the
// reference's association order). All three are destination-driven single
// passes: every output element is produced exactly once, stores are 16-byte
// vectors, and the work is pure HBM traffic (no LDS, no MFMA).
//
// Reference behaviour restated here:
//   jigsaw/modules/convolution/_conv/halo.py:66-156   (halo_gather)
//   jigsaw/modules/convolution/_conv/halo.py:159-251  (halo_scatter_add)
//   jigsaw/modules/convolution/_conv/distributed.py:264-275, 378-389 (axis order)
#include "jg_common.h"

namespace {

struct Geom {
  long long planes;
  int n[3];   // interior D, H, W
  int lo[3];  // halo before
  int hi[3];  // halo after
};

struct Table {
  const void* p[27];
};

struct MutTable {
  void* p[27];
};

// 16-byte vector of raw bits.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

template <typename T>
struct Bits;
template <>
struct Bits<uint16_t> {
  static constexpr int V = 8;
};
template <>
struct Bits<uint32_t> {
  static constexpr int V = 4;
};

// `0 + v` for every element of a dword: the only value the addition changes is -0.0, which
// becomes +0.0. On the packed 16-bit halves without unpacking them: bit 15 of (t + 0x7fff) | t
// is set exactly where the 15 magnitude bits t of a half are not all zero, and only there the
// sign is kept.
template <typename T>
__device__ __forceinline__ uint32_t zero_plus(uint32_t v);
template <>
__device__ __forceinline__ uint32_t zero_plus<uint32_t>(uint32_t v) {
  return v == 0x80000000u ? 0u : v;
}
template <>
__device__ __forceinline__ uint32_t zero_plus<uint16_t>(uint32_t v) {
  const uint32_t t = v & 0x7fff7fffu;
  const uint32_t keep = ((t + 0x7fff7fffu) | t) & 0x80008000u;
  return t | (v & keep);
}

// One element from an address that is the same in every lane, through the scalar cache: the
// aligned dword that holds it (which lies in the same page) and, for a 16-bit element, a shift.
__device__ __forceinline__ uint32_t uniform_dword(const uint32_t* q) {
  // the address in scalar registers, whatever the compiler worked out about it
  const uint64_t a = reinterpret_cast<uint64_t>(q);
  const uint64_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a);
  const uint64_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32));
  q = reinterpret_cast<const uint32_t*>((hi << 32) | lo);
  uint32_t w;
  asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(w) : "s"(q) : "memory");
  return w;
}
__device__ __forceinline__ uint32_t uniform_element(const uint32_t* s) { return uniform_dword(s); }
__device__ __forceinline__ uint16_t uniform_element(const uint16_t* s) {
  const uint32_t odd = (uint32_t)(reinterpret_cast<uintptr_t>(s) >> 1) & 1u;
  return (uint16_t)(uniform_dword(reinterpret_cast<const uint32_t*>(s - odd)) >> (odd * 16));
}

// Load 16 bytes from an address that is only sizeof(T)-aligned.
template <typename T>
__device__ __forceinline__ u32x4 load16_unaligned(const T* s);

template <>
__device__ __forceinline__ u32x4 load16_unaligned<uint32_t>(const uint32_t* s) {
  return *reinterpret_cast<const u32x4_a4*>(s);
}

template <>
__device__ __forceinline__ u32x4 load16_unaligned<uint16_t>(const uint16_t* s) {
  // The memory pipeline takes vector accesses at any alignment, but one that starts on an odd
  // halfword runs at a fraction of the rate of a dword-aligned one. Such a piece is read from one
  // element earlier, with the dword that follows, and shifted; no branch, and the extra dword of a
  // piece that needs none is its own last one, so nothing past the piece is touched.
  const uint32_t odd = (uint32_t)(reinterpret_cast<uintptr_t>(s) >> 1) & 1u;
  const uint32_t* q = reinterpret_cast<const uint32_t*>(s - odd);
  const u32x4 v = *reinterpret_cast<const u32x4_a4*>(q);
  const uint32_t x = q[3 + odd];
  const uint32_t sh = odd << 4;
  u32x4 r;
  r.x = __builtin_amdgcn_alignbit(v.y, v.x, sh);
  r.y = __builtin_amdgcn_alignbit(v.z, v.y, sh);
  r.z = __builtin_amdgcn_alignbit(v.w, v.z, sh);
  r.w = __builtin_amdgcn_alignbit(x, v.w, sh);
  return r;
}

// Store 16 bytes to an address that is only sizeof(T)-aligned.
__device__ __forceinline__ void store16_unaligned(uint32_t* d, u32x4 v) { *reinterpret_cast<u32x4_a4*>(d) = v; }
__device__ __forceinline__ void store16_unaligned(uint16_t* d, u32x4 v) {
  typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
  *reinterpret_cast<u32x4_a2*>(d) = v;
}

// Region of a padded coordinate: 0 = lower halo, 1 = interior, 2 = upper halo.
__device__ __forceinline__ void region(int x, int lo, int n, int hi, int& r, int& c,
                                       int& ext) {
  if (x < lo) {
    r = 0; c = x; ext = lo;
  } else if (x < lo + n) {
    r = 1; c = x - lo; ext = n;
  } else {
    r = 2; c = x - lo - n; ext = hi;
  }
}

// The neighbour table is the FIRST parameter of every kernel that looks it up
// with a per-lane index: it is then read straight from the kernel-argument
// segment (constant memory, offset 0) instead of being copied to scratch.
__device__ __forceinline__ const void* table_entry(int idx) {
#if defined(__HIP_DEVICE_COMPILE__)
  const void* const* kt = (const void* const*)__builtin_amdgcn_kernarg_segment_ptr();
  return kt[idx];
#else  // host pass of hipcc: never called
  (void)idx;
  return nullptr;
#endif
}

// ------------------------------------------------------------------ assemble
template <typename T>
__device__ __forceinline__ T assemble_fetch(const Geom& g, long long p, int da, int ha, int wa) {
  int rd, cd, ed, rh, ch, eh, rw, cw, ew;
  region(da, g.lo[0], g.n[0], g.hi[0], rd, cd, ed);
  region(ha, g.lo[1], g.n[1], g.hi[1], rh, ch, eh);
  region(wa, g.lo[2], g.n[2], g.hi[2], rw, cw, ew);
  const T* s = static_cast<const T*>(table_entry(rd * 9 + rh * 3 + rw));
  if (s == nullptr) return T(0);
  long long off = ((p * ed + cd) * eh + ch) * (long long)ew + cw;
  return s[off];
}

template <typename T, typename I>
__global__ __launch_bounds__(256) void assemble_kernel(Table tab, T* __restrict__ dst,
                                                       Geom g, I total) {
  constexpr int V = Bits<T>::V;
  const I nvec = (total + V - 1) / V;
  const int Da = g.lo[0] + g.n[0] + g.hi[0];
  const int Ha = g.lo[1] + g.n[1] + g.hi[1];
  const int Wa = g.lo[2] + g.n[2] + g.hi[2];
  for (I v = (I)blockIdx.x * 256 + threadIdx.x; v < nvec; v += (I)gridDim.x * 256) {
    const I e0 = v * V;
    I row = e0 / (I)Wa;
    int wa = (int)(e0 - row * (I)Wa);
    I t = row / (I)Ha;
    int ha = (int)(row - t * (I)Ha);
    I pp = t / (I)Da;
    int da = (int)(t - pp * (I)Da);
    long long p = (long long)pp;

    bool fast = (wa + V <= Wa) && (e0 + V <= total);
    int rw = 0, cw = 0, ew = 0;
    if (fast) {
      int rw2, cw2, ew2;
      region(wa, g.lo[2], g.n[2], g.hi[2], rw, cw, ew);
      region(wa + V - 1, g.lo[2], g.n[2], g.hi[2], rw2, cw2, ew2);
      fast = (rw == rw2);
    }
    if (fast) {
      int rd, cd, ed, rh, ch, eh;
      region(da, g.lo[0], g.n[0], g.hi[0], rd, cd, ed);
      region(ha, g.lo[1], g.n[1], g.hi[1], rh, ch, eh);
      const T* s = static_cast<const T*>(table_entry(rd * 9 + rh * 3 + rw));
      u32x4 val = {0u, 0u, 0u, 0u};
      if (s != nullptr) {
        long long off = ((p * ed + cd) * eh + ch) * (long long)ew + cw;
        val = load16_unaligned<T>(s + off);
      }
      *reinterpret_cast<u32x4*>(dst + e0) = val;
    } else {
      T tmp[V];
#pragma unroll
      for (int i = 0; i < V; ++i) {
        tmp[i] = T(0);
        if (e0 + i < total) tmp[i] = assemble_fetch<T>(g, p, da, ha, wa);
        if (++wa == Wa) {
          wa = 0;
          if (++ha == Ha) {
            ha = 0;
            if (++da == Da) {
              da = 0;
              ++p;
            }
          }
        }
      }
      if (e0 + V <= total) {
        u32x4 val;
        __builtin_memcpy(&val, tmp, 16);
        *reinterpret_cast<u32x4*>(dst + e0) = val;
      } else {
        for (int i = 0; i < V && e0 + i < total; ++i) dst[e0 + i] = tmp[i];
      }
    }
  }
}

// ---------------------------------------------------------------------- pack
struct Box {
  int org[3];  // origin in the source, per axis
  int ext[3];  // extent, per axis
};
struct PackArgs {
  void* dst[27];
  Box box[27];
};

// I: index type (32-bit when the source tensor has fewer than 2^31 elements). A thread moves one
// chunk of up to V = 16 / sizeof(T) consecutive elements of a strip row: one 16-byte access each
// way for the faces whose rows run along W, single elements for the faces that are one column wide.
template <typename T, typename I>
__global__ __launch_bounds__(256) void pack_kernel(PackArgs a, const T* __restrict__ src,
                                                   long long planes, int Sd, int Sh,
                                                   int Sw) {
  constexpr int V = Bits<T>::V;
  const int slot = blockIdx.y;
  T* d = static_cast<T*>(a.dst[slot]);
  if (d == nullptr) return;
  const Box b = a.box[slot];
  const I e0 = (I)b.ext[0], e1 = (I)b.ext[1], e2 = (I)b.ext[2];
  const I cpr = (e2 + V - 1) / V;  // chunks per row
  const I total = (I)planes * e0 * e1 * cpr;
  for (I i = (I)blockIdx.x * 256 + threadIdx.x; i < total; i += (I)gridDim.x * 256) {
    const I r = i / cpr;
    const I cw = (i - r * cpr) * V;
    const I r2 = r / e1;
    const I ch = r - r2 * e1;
    const I p = r2 / e0;
    const I cd = r2 - p * e0;
    const I so = ((p * (I)Sd + ((I)b.org[0] + cd)) * (I)Sh + ((I)b.org[1] + ch)) * (I)Sw + ((I)b.org[2] + cw);
    const I to = r * e2 + cw;
    if (cw + V <= e2) {
      store16_unaligned(d + to, load16_unaligned<T>(src + so));
    } else {
      for (I k = 0; cw + k < e2; ++k) d[to + k] = src[so + k];
    }
  }
}

// The two faces across W (slots 12 and 14) of a tile whose rows are longer than a cache line:
// every row gives a few cells from each end, so each face alone touches one line of every row.
// One thread takes both ends of ROWS rows, 256 rows apart, all loads before the first store: the
// two lines of a row are asked for together (neighbouring lanes: neighbouring rows, so whole
// DRAM pages are read in one go instead of half now and half when the other face is packed),
// and a lane has up to 2 * ROWS * ext loads in flight.
template <typename T>
__global__ __launch_bounds__(256) void pack_w_faces_kernel(T* __restrict__ dlo, T* __restrict__ dhi,
                                                           const T* __restrict__ src, Box blo, Box bhi,
                                                           unsigned rows, int Sd, int Sh, int Sw) {
  constexpr int ROWS = 4;
  const unsigned e0 = (unsigned)blo.ext[0], e1 = (unsigned)blo.ext[1];
  const int nlo = blo.ext[2], nhi = bhi.ext[2];
  const unsigned first = blockIdx.x * (256u * ROWS) + threadIdx.x;
  T vlo[ROWS][2], vhi[ROWS][2];
#pragma unroll
  for (int k = 0; k < ROWS; ++k) {
    const unsigned r = first + 256u * k;
    if (r < rows) {
      const unsigned r2 = r / e1, ch = r - r2 * e1;
      const unsigned pl = r2 / e0, cd = r2 - pl * e0;
      const T* row = src + (((size_t)pl * Sd + (blo.org[0] + cd)) * Sh + (blo.org[1] + ch)) * (size_t)Sw;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (j < nlo) vlo[k][j] = row[blo.org[2] + j];
        if (j < nhi) vhi[k][j] = row[bhi.org[2] + j];
      }
    }
  }
#pragma unroll
  for (int k = 0; k < ROWS; ++k) {
    const unsigned r = first + 256u * k;
    if (r < rows) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (j < nlo) dlo[(size_t)r * nlo + j] = vlo[k][j];
        if (j < nhi) dhi[(size_t)r * nhi + j] = vhi[k][j];
      }
    }
  }
}

// ---------------------------------------------------------------------- fold
// Arithmetic of one `acc += v` in the tensor dtype (what Tensor.add_ does).
template <int DT>
struct Arith;
template <>
struct Arith<JG_F32> {
  typedef uint32_t T;
  __device__ static __forceinline__ float up(uint32_t b) { return __uint_as_float(b); }
  __device__ static __forceinline__ uint32_t down(float f) { return __float_as_uint(f); }
};
template <>
struct Arith<JG_BF16> {
  typedef uint16_t T;
  __device__ static __forceinline__ float up(uint16_t b) { return jg::bf16_to_f32(b); }
  __device__ static __forceinline__ uint16_t down(float f) { return jg::f32_to_bf16(f); }
};
template <>
struct Arith<JG_F16> {
  typedef uint16_t T;
  __device__ static __forceinline__ float up(uint16_t b) {
    _Float16 h;
    __builtin_memcpy(&h, &b, 2);
    return (float)h;
  }
  __device__ static __forceinline__ uint16_t down(float f) {
    _Float16 h = (_Float16)f;
    uint16_t b;
    __builtin_memcpy(&b, &h, 2);
    return b;
  }
};

// Which neighbour offsets reach interior coordinate x of an axis, and where in
// that neighbour's strip. o = -1: the lower neighbour's upper halo covers
// [0, hi); o = +1: the upper neighbour's lower halo covers [n - lo, n).
__device__ __forceinline__ bool reach(int o, int x, int lo, int n, int hi, int& c,
                                      int& ext) {
  if (o < 0) {
    c = x; ext = hi;
    return x < hi;
  }
  if (o == 0) {
    c = x; ext = n;
    return true;
  }
  c = x - (n - lo); ext = lo;
  return x >= n - lo;
}

template <int DT>
__device__ __forceinline__ typename Arith<DT>::T fold_one(
    const typename Arith<DT>::T* __restrict__ own, const Table& tab, const Geom& g,
    long long p, int d, int h, int w) {
  typedef typename Arith<DT>::T T;
  const int Ha = g.lo[1] + g.n[1] + g.hi[1];
  const int Wa = g.lo[2] + g.n[2] + g.hi[2];
  const int Da = g.lo[0] + g.n[0] + g.hi[0];
  float acc_d = 0.0f;
  for (int od = -1; od <= 1; ++od) {
    int cd, ed;
    if (!reach(od, d, g.lo[0], g.n[0], g.hi[0], cd, ed)) continue;
    float acc_h = 0.0f;
    for (int oh = -1; oh <= 1; ++oh) {
      int ch, eh;
      if (!reach(oh, h, g.lo[1], g.n[1], g.hi[1], ch, eh)) continue;
      float acc_w = 0.0f;
      for (int ow = -1; ow <= 1; ++ow) {
        int cw, ew;
        if (!reach(ow, w, g.lo[2], g.n[2], g.hi[2], cw, ew)) continue;
        T bits;
        if (od == 0 && oh == 0 && ow == 0) {
          long long off = ((p * Da + (d + g.lo[0])) * Ha + (h + g.lo[1])) * (long long)Wa +
                          (w + g.lo[2]);
          bits = own[off];
        } else {
          const T* s = static_cast<const T*>(tab.p[(od + 1) * 9 + (oh + 1) * 3 + (ow + 1)]);
          if (s == nullptr) continue;
          long long off = ((p * ed + cd) * eh + ch) * (long long)ew + cw;
          bits = s[off];
        }
        acc_w = Arith<DT>::up(Arith<DT>::down(acc_w + Arith<DT>::up(bits)));
      }
      acc_h = Arith<DT>::up(Arith<DT>::down(acc_h + acc_w));
    }
    acc_d = Arith<DT>::up(Arith<DT>::down(acc_d + acc_h));
  }
  return Arith<DT>::down(acc_d);
}

template <int DT, typename I>
__global__ __launch_bounds__(256) void fold_kernel(typename Arith<DT>::T* __restrict__ dst,
                                                   const typename Arith<DT>::T* __restrict__ own,
                                                   Table tab, Geom g, I total) {
  typedef typename Arith<DT>::T T;
  constexpr int V = Bits<T>::V;
  const I nvec = (total + V - 1) / V;
  const int D = g.n[0], H = g.n[1], W = g.n[2];
  const int Ha = g.lo[1] + H + g.hi[1];
  const int Wa = g.lo[2] + W + g.hi[2];
  const int Da = g.lo[0] + D + g.hi[0];
  for (I v = (I)blockIdx.x * 256 + threadIdx.x; v < nvec; v += (I)gridDim.x * 256) {
    const I e0 = v * V;
    I row = e0 / (I)W;
    int w = (int)(e0 - row * (I)W);
    I t = row / (I)H;
    int h = (int)(row - t * (I)H);
    I pp = t / (I)D;
    int d = (int)(t - pp * (I)D);
    long long p = (long long)pp;

    // Interior of the tile: nothing but `0 + own`, which only clears the sign
    // of a zero.
    bool fast = (e0 + V <= total) && (w >= g.hi[2]) && (w + V <= W - g.lo[2]) &&
                (h >= g.hi[1]) && (h < H - g.lo[1]) && (d >= g.hi[0]) && (d < D - g.lo[0]);
    if (fast) {
      long long off = ((p * Da + (d + g.lo[0])) * Ha + (h + g.lo[1])) * (long long)Wa +
                      (w + g.lo[2]);
      u32x4 val = load16_unaligned<T>(own + off);
      val.x = zero_plus<T>(val.x);
      val.y = zero_plus<T>(val.y);
      val.z = zero_plus<T>(val.z);
      val.w = zero_plus<T>(val.w);
      *reinterpret_cast<u32x4*>(dst + e0) = val;
    } else {
      T tmp[V];
#pragma unroll
      for (int i = 0; i < V; ++i) {
        tmp[i] = T(0);
        if (e0 + i < total) tmp[i] = fold_one<DT>(own, tab, g, p, d, h, w);
        if (++w == W) {
          w = 0;
          if (++h == H) {
            h = 0;
            if (++d == D) {
              d = 0;
              ++p;
            }
          }
        }
      }
      if (e0 + V <= total) {
        u32x4 val;
        __builtin_memcpy(&val, tmp, 16);
        *reinterpret_cast<u32x4*>(dst + e0) = val;
      } else {
        for (int i = 0; i < V && e0 + i < total; ++i) dst[e0 + i] = tmp[i];
      }
    }
  }
}


// ===================================================================== row kernels
// Bandwidth versions of assemble and fold. A destination ROW (one (plane, d, h)
// line along W) is owned by a group of LPR lanes (a whole wavefront for long
// rows), each lane producing 16-byte vectors j, j + LPR, ... of that row. Row
// coordinates are decomposed once per lane with multiply-high divisions, the
// three sources of the row (lower-W strip, middle, upper-W strip) are looked up
// once, and only the vectors that straddle a region boundary take the
// element-wise path. Rows start on 4-byte boundaries, which is all the 16-byte
// global accesses of gfx9 need.
struct Magic {
  uint32_t m, s, one;  // n / d = one ? n : (t + ((n - t) >> 1)) >> (s - 1), t = mulhi(m, n)
};

__device__ __forceinline__ uint32_t mdiv(uint32_t n, const Magic& k) {
  if (k.one) return n;
  const uint32_t t = __umulhi(k.m, n);
  return (t + ((n - t) >> 1)) >> (k.s - 1);
}

struct RowPlan {
  uint32_t nrows;   // planes * Da * Ha (assemble) or planes * D * H (fold)
  int lpr_log2;     // lanes per row = 1 << lpr_log2
  int iters;        // vectors per lane
  int nvec;         // vectors per row
  Magic div_h, div_d;
};

typedef uint32_t u32x4_s4 __attribute__((ext_vector_type(4), aligned(4)));
constexpr int ROW_BATCH = 4;  // vectors a lane keeps in flight

template <typename T>
__global__ __launch_bounds__(256) void assemble_rows_kernel(Table tab, T* __restrict__ dst,
                                                            Geom g, RowPlan pl) {
  constexpr int V = Bits<T>::V;
  const uint32_t t = blockIdx.x * 256u + threadIdx.x;
  const uint32_t row = t >> pl.lpr_log2;
  if (row >= pl.nrows) return;
  const int lir = (int)(t & ((1u << pl.lpr_log2) - 1));
  const int Da = g.lo[0] + g.n[0] + g.hi[0];
  const int Ha = g.lo[1] + g.n[1] + g.hi[1];
  const int Wa = g.lo[2] + g.n[2] + g.hi[2];
  const uint32_t t2 = mdiv(row, pl.div_h);
  const int ha = (int)(row - t2 * (uint32_t)Ha);
  const uint32_t pp = mdiv(t2, pl.div_d);
  const int da = (int)(t2 - pp * (uint32_t)Da);
  int rd, cd, ed, rh, ch, eh;
  region(da, g.lo[0], g.n[0], g.hi[0], rd, cd, ed);
  region(ha, g.lo[1], g.n[1], g.hi[1], rh, ch, eh);
  const long long line = ((long long)pp * ed + cd) * eh + ch;  // row index inside a source
  const int base_idx = rd * 9 + rh * 3;
  // Rows of the tile itself (all but the halo rows): their three sources are table entries
  // with constant indices, which are scalar loads done once at the head of the kernel. Only
  // the halo rows look the table up with a per-lane index, a trip to memory that the row's
  // own loads would have to wait for.
  const T* s0 = static_cast<const T*>(tab.p[12]);
  const T* s1 = static_cast<const T*>(tab.p[13]);
  const T* s2 = static_cast<const T*>(tab.p[14]);
  if (base_idx != 12) {
    s0 = static_cast<const T*>(table_entry(base_idx + 0));
    s1 = static_cast<const T*>(table_entry(base_idx + 1));
    s2 = static_cast<const T*>(table_entry(base_idx + 2));
  }
  if (s0 != nullptr) s0 += line * g.lo[2];
  if (s1 != nullptr) s1 += line * g.n[2];
  if (s2 != nullptr) s2 += line * g.hi[2];
  T* drow = dst + (long long)row * Wa;
  const int mid_lo = g.lo[2], mid_hi = g.lo[2] + g.n[2];
  // The middle source in 16-byte vectors of ITS row (aligned loads when the tile rows
  // are), stored at whatever alignment the padded row gives them; all the loads of a
  // batch are issued before its first store.
  typedef uint32_t u32x4_any __attribute__((ext_vector_type(4), aligned(2)));
  const int n_full = g.n[2] / V;
  for (int it0 = 0; (it0 << pl.lpr_log2) < n_full; it0 += ROW_BATCH) {
    u32x4 val[ROW_BATCH];
#pragma unroll
    for (int u = 0; u < ROW_BATCH; ++u) {
      const int j = lir + ((it0 + u) << pl.lpr_log2);
      val[u] = u32x4{0u, 0u, 0u, 0u};
      if (j < n_full && s1 != nullptr) val[u] = *reinterpret_cast<const u32x4_any*>(s1 + j * V);
    }
#pragma unroll
    for (int u = 0; u < ROW_BATCH; ++u) {
      const int j = lir + ((it0 + u) << pl.lpr_log2);
      if (j < n_full) *reinterpret_cast<u32x4_any*>(drow + mid_lo + j * V) = val[u];
    }
  }
  // The W halos and the tail of the middle, one element per lane.
  const int head = mid_lo;                    // columns [0, head)
  const int tail0 = mid_lo + n_full * V;      // columns [tail0, Wa)
  const int n_edge = head + (Wa - tail0);
  for (int q = lir; q < n_edge; q += (1 << pl.lpr_log2)) {
    const int c = q < head ? q : tail0 + (q - head);
    const T* src = nullptr;
    if (c < mid_lo) {
      if (s0 != nullptr) src = s0 + c;
    } else if (c < mid_hi) {
      if (s1 != nullptr) src = s1 + (c - mid_lo);
    } else {
      if (s2 != nullptr) src = s2 + (c - mid_hi);
    }
    drow[c] = src != nullptr ? *src : T(0);
  }
}

// k-th border coordinate of an axis of extent n reached over [0, hi) and [n - lo, n)
__device__ __forceinline__ int border_coord(int k, int n, int lo, int hi) {
  if (hi + lo >= n) return k;
  return k < hi ? k : n - lo + (k - hi);
}

// Assemble restricted to a frame of the padded tile: only the cells whose padded
// coordinate lies in the first band_lo or the last band_hi positions of some axis are
// written. Two kinds of launches of one kernel: `full_rows` = the rows inside a D or H
// band, written whole; otherwise the remaining rows, of which only columns
// [c_begin, c_end) (a W band) are written.
struct FramePlan {
  uint32_t rows_per_plane, total_rows;
  int full_rows;
  int nbd, nbh;                 // band rows along D / H (first + last), clipped to the extent
  int bd_lo, bd_hi, bh_lo, bh_hi;
  int c_begin, c_end;
  int lpr_log2;
  Magic div_rows, div_a, div_b;
};

template <typename T>
__global__ __launch_bounds__(256) void assemble_frame_kernel(Table tab, T* __restrict__ dst, Geom g,
                                                             FramePlan fp) {
  constexpr int V = Bits<T>::V;
  typedef uint32_t u32x4_any __attribute__((ext_vector_type(4), aligned(2)));
  const uint32_t t = blockIdx.x * 256u + threadIdx.x;
  const uint32_t item = t >> fp.lpr_log2;
  if (item >= fp.total_rows) return;
  const int lir = (int)(t & ((1u << fp.lpr_log2) - 1));
  const int Da = g.lo[0] + g.n[0] + g.hi[0];
  const int Ha = g.lo[1] + g.n[1] + g.hi[1];
  const int Wa = g.lo[2] + g.n[2] + g.hi[2];
  const uint32_t pp = mdiv(item, fp.div_rows);
  const uint32_t idx = item - pp * fp.rows_per_plane;
  int da, ha;
  if (fp.full_rows) {
    if (idx < (uint32_t)fp.nbd * (uint32_t)Ha) {
      const uint32_t k = mdiv(idx, fp.div_a);  // / Ha
      da = border_coord((int)k, Da, fp.bd_hi, fp.bd_lo);
      ha = (int)(idx - k * (uint32_t)Ha);
    } else {
      const uint32_t idx2 = idx - (uint32_t)fp.nbd * (uint32_t)Ha;
      const uint32_t di = mdiv(idx2, fp.div_b);  // / nbh
      da = fp.bd_lo + (int)di;
      ha = border_coord((int)(idx2 - di * (uint32_t)fp.nbh), Ha, fp.bh_hi, fp.bh_lo);
    }
  } else {
    const uint32_t di = mdiv(idx, fp.div_a);  // / (Ha - nbh)
    da = fp.bd_lo + (int)di;
    ha = fp.bh_lo + (int)(idx - di * (uint32_t)(Ha - fp.nbh));
  }
  int rd, cd, ed, rh, ch, eh;
  region(da, g.lo[0], g.n[0], g.hi[0], rd, cd, ed);
  region(ha, g.lo[1], g.n[1], g.hi[1], rh, ch, eh);
  const long long line = ((long long)pp * ed + cd) * eh + ch;
  const int base_idx = rd * 9 + rh * 3;
  // Rows of the tile itself (all but the halo rows): their three sources are table entries
  // with constant indices, which are scalar loads done once at the head of the kernel. Only
  // the halo rows look the table up with a per-lane index, a trip to memory that the row's
  // own loads would have to wait for.
  const T* s0 = static_cast<const T*>(tab.p[12]);
  const T* s1 = static_cast<const T*>(tab.p[13]);
  const T* s2 = static_cast<const T*>(tab.p[14]);
  if (base_idx != 12) {
    s0 = static_cast<const T*>(table_entry(base_idx + 0));
    s1 = static_cast<const T*>(table_entry(base_idx + 1));
    s2 = static_cast<const T*>(table_entry(base_idx + 2));
  }
  if (s0 != nullptr) s0 += line * g.lo[2];
  if (s1 != nullptr) s1 += line * g.n[2];
  if (s2 != nullptr) s2 += line * g.hi[2];
  T* drow = dst + (((long long)pp * Da + da) * Ha + ha) * (long long)Wa;
  const int mid_lo = g.lo[2], mid_hi = g.lo[2] + g.n[2];
  // middle source in 16-byte vectors of its own row, clipped to the column window
  const int m_begin = fp.c_begin > mid_lo ? fp.c_begin : mid_lo;
  const int m_end = fp.c_end < mid_hi ? fp.c_end : mid_hi;
  const int j0 = (m_begin - mid_lo + V - 1) / V, j1 = (m_end - mid_lo) / V;  // whole vectors [j0, j1)
  const int n_full = j1 > j0 ? j1 - j0 : 0;
  for (int it0 = 0; (it0 << fp.lpr_log2) < n_full; it0 += ROW_BATCH) {
    u32x4 val[ROW_BATCH];
#pragma unroll
    for (int u = 0; u < ROW_BATCH; ++u) {
      const int j = lir + ((it0 + u) << fp.lpr_log2);
      val[u] = u32x4{0u, 0u, 0u, 0u};
      if (j < n_full && s1 != nullptr) val[u] = *reinterpret_cast<const u32x4_any*>(s1 + (j0 + j) * V);
    }
#pragma unroll
    for (int u = 0; u < ROW_BATCH; ++u) {
      const int j = lir + ((it0 + u) << fp.lpr_log2);
      if (j < n_full) *reinterpret_cast<u32x4_any*>(drow + mid_lo + (j0 + j) * V) = val[u];
    }
  }
  // what the vectors left of the window: [c_begin, head_end) and [tail0, c_end)
  const int head_end = n_full > 0 ? mid_lo + j0 * V : fp.c_end;
  const int tail0 = n_full > 0 ? mid_lo + j1 * V : fp.c_end;
  const int n_head = head_end - fp.c_begin;
  const int n_edge = n_head + (fp.c_end - tail0);
  for (int q = lir; q < n_edge; q += (1 << fp.lpr_log2)) {
    const int c = q < n_head ? fp.c_begin + q : tail0 + (q - n_head);
    const T* src = nullptr;
    if (c < mid_lo) {
      if (s0 != nullptr) src = s0 + c;
    } else if (c < mid_hi) {
      if (s1 != nullptr) src = s1 + (c - mid_lo);
    } else {
      if (s2 != nullptr) src = s2 + (c - mid_hi);
    }
    drow[c] = src != nullptr ? *src : T(0);
  }
}

// One element of the fold with the loops left rolled: only the offsets that reach
// the element cost anything (most edge elements see one or two neighbours).
template <int DT>
__device__ __forceinline__ typename Arith<DT>::T fold_one_rolled(
    const typename Arith<DT>::T* __restrict__ own, const Geom& g, long long p, int d, int h, int w) {
  typedef typename Arith<DT>::T T;
  const int Ha = g.lo[1] + g.n[1] + g.hi[1];
  const int Wa = g.lo[2] + g.n[2] + g.hi[2];
  const int Da = g.lo[0] + g.n[0] + g.hi[0];
  float acc_d = 0.0f;
#pragma unroll 1
  for (int od = -1; od <= 1; ++od) {
    int cd, ed;
    if (!reach(od, d, g.lo[0], g.n[0], g.hi[0], cd, ed)) continue;
    float acc_h = 0.0f;
#pragma unroll 1
    for (int oh = -1; oh <= 1; ++oh) {
      int ch, eh;
      if (!reach(oh, h, g.lo[1], g.n[1], g.hi[1], ch, eh)) continue;
      float acc_w = 0.0f;
#pragma unroll 1
      for (int ow = -1; ow <= 1; ++ow) {
        int cw, ew;
        if (!reach(ow, w, g.lo[2], g.n[2], g.hi[2], cw, ew)) continue;
        T bits;
        if (od == 0 && oh == 0 && ow == 0) {
          long long off = ((p * Da + (d + g.lo[0])) * Ha + (h + g.lo[1])) * (long long)Wa +
                          (w + g.lo[2]);
          bits = own[off];
        } else {
          const T* s = static_cast<const T*>(table_entry((od + 1) * 9 + (oh + 1) * 3 + (ow + 1)));
          if (s == nullptr) continue;
          long long off = ((p * ed + cd) * eh + ch) * (long long)ew + cw;
          bits = s[off];
        }
        acc_w = Arith<DT>::up(Arith<DT>::down(acc_w + Arith<DT>::up(bits)));
      }
      acc_h = Arith<DT>::up(Arith<DT>::down(acc_h + acc_w));
    }
    acc_d = Arith<DT>::up(Arith<DT>::down(acc_d + acc_h));
  }
  return Arith<DT>::down(acc_d);
}

// Columns [c0, c0 + cnt), cnt <= V, of a row that D or H neighbours may reach: the full
// ordered sum. Per (od, oh) the middle term is one 16-byte load (cnt == V) from the own
// row or from that neighbour's strip; the W-neighbour terms touch only the first and
// last columns. `self_row` points at column 0 of the own contribution of this row (the
// padded gradient, or the destination itself for an in-place fold).
template <int DT>
__device__ __forceinline__ void fold_span(typename Arith<DT>::T* drow,
                                          const typename Arith<DT>::T* self_row, const Geom& g,
                                          long long p, int d, int h, int c0, int cnt) {
  typedef typename Arith<DT>::T T;
  constexpr int V = Bits<T>::V;
  typedef uint32_t u32x4_e __attribute__((ext_vector_type(4), aligned(2)));
  const int D = g.n[0], H = g.n[1], W = g.n[2];
  const int up0 = W - g.lo[2];
  const bool edge = c0 < g.hi[2] || c0 + cnt > up0;
  float acc_d[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc_d[e] = 0.0f;
#pragma unroll 1
  for (int od = -1; od <= 1; ++od) {
    int cd, ed;
    if (!reach(od, d, g.lo[0], D, g.hi[0], cd, ed)) continue;
    float acc_h[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc_h[e] = 0.0f;
#pragma unroll 1
    for (int oh = -1; oh <= 1; ++oh) {
      int ch, eh;
      if (!reach(oh, h, g.lo[1], H, g.hi[1], ch, eh)) continue;
      const long long line = (p * ed + cd) * eh + ch;  // row index inside a strip of (od, oh)
      const int slot = (od + 1) * 9 + (oh + 1) * 3;
      const bool self = od == 0 && oh == 0;
      const T* mid = self ? self_row : static_cast<const T*>(table_entry(slot + 1));
      if (!self && mid != nullptr) mid += line * W;
      T mb[V];
#pragma unroll
      for (int e = 0; e < V; ++e) mb[e] = T(0);
      if (mid != nullptr) {
        if (cnt == V) {
          const u32x4 mv = *reinterpret_cast<const u32x4_e*>(mid + c0);
          __builtin_memcpy(mb, &mv, 16);
        } else {
#pragma unroll
          for (int e = 0; e < V; ++e)
            if (e < cnt) mb[e] = mid[c0 + e];
        }
      }
      float acc_w[V];
      if (!edge) {
#pragma unroll
        for (int e = 0; e < V; ++e) acc_w[e] = Arith<DT>::up(Arith<DT>::down(0.0f + Arith<DT>::up(mb[e])));
      } else {
        const T* s_lo = static_cast<const T*>(table_entry(slot + 0));
        const T* s_hi = static_cast<const T*>(table_entry(slot + 2));
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const int c = c0 + e;
          float a = 0.0f;
          if (e < cnt && c < g.hi[2] && s_lo != nullptr)
            a = Arith<DT>::up(Arith<DT>::down(a + Arith<DT>::up(s_lo[line * g.hi[2] + c])));
          a = Arith<DT>::up(Arith<DT>::down(a + Arith<DT>::up(mb[e])));
          if (e < cnt && c >= up0 && s_hi != nullptr)
            a = Arith<DT>::up(Arith<DT>::down(a + Arith<DT>::up(s_hi[line * g.lo[2] + (c - up0)])));
          acc_w[e] = a;
        }
      }
#pragma unroll
      for (int e = 0; e < V; ++e) acc_h[e] = Arith<DT>::up(Arith<DT>::down(acc_h[e] + acc_w[e]));
    }
#pragma unroll
    for (int e = 0; e < V; ++e) acc_d[e] = Arith<DT>::up(Arith<DT>::down(acc_d[e] + acc_h[e]));
  }
  T ob[V];
#pragma unroll
  for (int e = 0; e < V; ++e) ob[e] = Arith<DT>::down(acc_d[e]);
  if (cnt == V) {
    u32x4 out;
    __builtin_memcpy(&out, ob, 16);
    *reinterpret_cast<u32x4_e*>(drow + c0) = out;
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e)
      if (e < cnt) drow[c0 + e] = ob[e];
  }
}

template <int DT>
__global__ __launch_bounds__(256) void fold_rows_kernel(Table tab,
                                                        typename Arith<DT>::T* __restrict__ dst,
                                                        const typename Arith<DT>::T* __restrict__ own,
                                                        Geom g, RowPlan pl, bool defer_border) {
  typedef typename Arith<DT>::T T;
  constexpr int V = Bits<T>::V;
  const uint32_t t = blockIdx.x * 256u + threadIdx.x;
  const uint32_t row = t >> pl.lpr_log2;
  if (row >= pl.nrows) return;
  const int lir = (int)(t & ((1u << pl.lpr_log2) - 1));
  const int D = g.n[0], H = g.n[1], W = g.n[2];
  const int Ha = g.lo[1] + H + g.hi[1];
  const int Wa = g.lo[2] + W + g.hi[2];
  const int Da = g.lo[0] + D + g.hi[0];
  const uint32_t t2 = mdiv(row, pl.div_h);
  const int h = (int)(row - t2 * (uint32_t)H);
  const uint32_t pp = mdiv(t2, pl.div_d);
  const int d = (int)(t2 - pp * (uint32_t)D);
  const long long p = (long long)pp;
  // rows that a lower / upper neighbour along D or H reaches take the element path
  const bool row_plain = (d >= g.hi[0]) && (d < D - g.lo[0]) && (h >= g.hi[1]) && (h < H - g.lo[1]);
  const T* orow = own + ((p * Da + (d + g.lo[0])) * Ha + (h + g.lo[1])) * (long long)Wa + g.lo[2];
  T* drow = dst + (long long)row * W;
  // defer_border: such a row only gets `0 + own` here, like the columns of a plain row that no
  // neighbour reaches, and fold_border_rows_kernel sums it in full afterwards, a whole wavefront
  // per row (in a volume every eighth wavefront of this kernel holds such a row and would walk
  // the long path with a few lanes active).
  if (!row_plain && !defer_border) {
    const int n_vec = W / V;
    for (int j = lir; j < n_vec; j += (1 << pl.lpr_log2)) fold_span<DT>(drow, orow, g, p, d, h, j * V, V);
    if (lir == 0 && n_vec * V < W) fold_span<DT>(drow, orow, g, p, d, h, n_vec * V, W - n_vec * V);
    return;
  }
  // Only W neighbours reach this row. The sums over D and H then add a single term to
  // zero, which changes nothing after the first rounding, so an element is
  // ((0 + lower) + own) + upper with the terms that exist.
  const T* s_lo = static_cast<const T*>(table_entry(9 + 3 + 0));
  const T* s_hi = static_cast<const T*>(table_entry(9 + 3 + 2));
  if (s_lo != nullptr) s_lo += (long long)row * g.hi[2];
  if (s_hi != nullptr) s_hi += (long long)row * g.lo[2];
  if (!row_plain) s_lo = s_hi = nullptr;  // deferred: no neighbour's term here
  const int up0 = W - g.lo[2];  // first column the upper neighbour reaches
  auto element = [&](int c, T own_bits) {
    float acc = 0.0f;
    if (c < g.hi[2] && s_lo != nullptr) acc = Arith<DT>::up(Arith<DT>::down(acc + Arith<DT>::up(s_lo[c])));
    acc = Arith<DT>::up(Arith<DT>::down(acc + Arith<DT>::up(own_bits)));
    if (c >= up0 && s_hi != nullptr) acc = Arith<DT>::up(Arith<DT>::down(acc + Arith<DT>::up(s_hi[c - up0])));
    return Arith<DT>::down(acc);
  };
  // Whole 16-byte vectors: `0 + own` for the columns no W neighbour reaches, which only
  // clears the sign of a zero; the few columns at either end of the row that a neighbour
  // does reach are patched inside their vector. All the loads of a batch precede its
  // first store.
  const int n_vec = W / V;
  // Halos one column wide (3-wide kernels): column 0 and column W - 1 are the only ones a W
  // neighbour reaches. Their strip values are asked for here, with the row's own loads, and their
  // own values are taken from the vectors as they pass, so that finishing them below costs no
  // further trip to memory.
  const int lpr_mask = (1 << pl.lpr_log2) - 1;
  const bool thin = g.hi[2] == 1 && g.lo[2] == 1 && n_vec >= 2;
  const bool owns_first = thin && lir == 0, owns_last = thin && lir == ((n_vec - 1) & lpr_mask);
  // One load instruction for both: the lane that owns the first vector reads the lower strip,
  // the lane that owns the last one the upper strip (a row with a single vector per lane
  // group has one lane that owns both; it takes the second value with a load of its own).
  T strip_first = T(0), strip_last = T(0);
  // A whole wavefront per row: the row and with it the two addresses are the same in every
  // lane, so the two values come through the scalar cache (the aligned dword that holds the
  // element) and cost the vector memory pipeline nothing. They are fetched below, behind the
  // first batch of vector loads, whose latency covers the wait.
  const bool by_scalar = thin && pl.lpr_log2 == 6;
  const long long row_u = (long long)__builtin_amdgcn_readfirstlane((int)row);
  const T* const base_lo = by_scalar && row_plain ? static_cast<const T*>(table_entry(9 + 3 + 0)) : nullptr;
  const T* const base_hi = by_scalar && row_plain ? static_cast<const T*>(table_entry(9 + 3 + 2)) : nullptr;
  if (!by_scalar) {
    const T* sp = nullptr;
    if (owns_first && s_lo != nullptr) sp = s_lo;
    else if (owns_last && s_hi != nullptr) sp = s_hi + (W - 1 - up0);
    T got = T(0);
    if (sp != nullptr) got = *sp;
    if (owns_first) strip_first = got;
    else strip_last = got;
    if (owns_first && owns_last && s_hi != nullptr) strip_last = s_hi[W - 1 - up0];
  }
  auto ends = [&](T lower, T own_bits, T upper, bool has_lower, bool has_upper) {
    float acc = 0.0f;
    if (has_lower) acc = Arith<DT>::up(Arith<DT>::down(acc + Arith<DT>::up(lower)));
    acc = Arith<DT>::up(Arith<DT>::down(acc + Arith<DT>::up(own_bits)));
    if (has_upper) acc = Arith<DT>::up(Arith<DT>::down(acc + Arith<DT>::up(upper)));
    return Arith<DT>::down(acc);
  };
  for (int it0 = 0; (it0 << pl.lpr_log2) < n_vec; it0 += ROW_BATCH) {
    u32x4 val[ROW_BATCH];
#pragma unroll
    for (int u = 0; u < ROW_BATCH; ++u) {
      const int j = lir + ((it0 + u) << pl.lpr_log2);
      val[u] = u32x4{0u, 0u, 0u, 0u};
      if (j < n_vec) val[u] = load16_unaligned<T>(orow + j * V);
    }
    if (by_scalar && it0 == 0) {
      if (base_lo != nullptr) strip_first = uniform_element(base_lo + row_u * g.hi[2]);
      if (base_hi != nullptr) strip_last = uniform_element(base_hi + row_u * g.lo[2] + (W - 1 - up0));
    }
#pragma unroll
    for (int u = 0; u < ROW_BATCH; ++u) {
      const int j = lir + ((it0 + u) << pl.lpr_log2);
      if (j < n_vec) {
        const int c0 = j * V;
        constexpr int EB = (int)sizeof(T) * 8;
        const T first_bits = (T)val[u].x, last_bits = (T)(val[u].w >> (32 - EB));
        // `0 + own` for every column; then the two columns of a thin halo get their ordered sum
        // (wider halos: below). Running the ordered sum for all 8 elements of the first and of the
        // last vector, one lane active, was three quarters of the kernel's instructions.
        u32x4 out;
        out.x = zero_plus<T>(val[u].x);
        out.y = zero_plus<T>(val[u].y);
        out.z = zero_plus<T>(val[u].z);
        out.w = zero_plus<T>(val[u].w);
        if (owns_first && j == 0) {
          const uint32_t e = (uint32_t)ends(strip_first, first_bits, T(0), s_lo != nullptr, false);
          out.x = EB == 32 ? e : ((out.x & 0xffff0000u) | e);
        }
        if (owns_last && j == n_vec - 1 && n_vec * V == W) {
          const uint32_t e = (uint32_t)ends(T(0), last_bits, strip_last, false, s_hi != nullptr);
          out.w = EB == 32 ? e : ((out.w & 0x0000ffffu) | (e << 16));
        }
        *reinterpret_cast<u32x4_s4*>(drow + c0) = out;
      }
    }
  }
  // Wider halos: the columns a W neighbour reaches, one at a time, by the lane whose vector store
  // covered them (a lane's own stores to one address keep their order): vector j belongs to lane
  // j % lanes-per-row.
  if (!thin) {
    const int head = g.hi[2] < n_vec * V ? g.hi[2] : n_vec * V;
    for (int c = 0; c < head; ++c)
      if (((c / V) & lpr_mask) == lir) drow[c] = element(c, orow[c]);
    const int tail0 = up0 > head ? up0 : head;
    for (int c = tail0; c < n_vec * V; ++c)
      if (((c / V) & lpr_mask) == lir) drow[c] = element(c, orow[c]);
  }
  // what is left of a row that is not a whole number of vectors, one element per lane
  for (int c = n_vec * V + lir; c < W; c += (1 << pl.lpr_log2)) drow[c] = element(c, orow[c]);
}


// In-place second half of a fold: gx already holds `0 + own`; only the cells that a
// neighbour reaches change. Two kernels: the rows that a D or H neighbour reaches are
// summed in full, one wavefront per row; of the other rows only the first and last
// columns change, one lane per cell.
struct BorderPlan {
  uint32_t rows_per_plane;  // rows of a plane that a D or H neighbour reaches
  uint32_t total;           // work items of the launch
  int nbd, nbh;             // border depths / border rows of a non-border depth
  int n_edge, head;         // W-edge cells of a row: columns [0, head) and [W - lo, W)
  int lpr;                  // lanes per row of the rows kernel
  Magic div_rows, div_h, div_nbh, div_edge, div_hh, div_d;
};


template <int DT>
__global__ __launch_bounds__(256) void fold_border_rows_kernel(Table tab, typename Arith<DT>::T* __restrict__ gx,
                                                               Geom g, BorderPlan bp) {
  typedef typename Arith<DT>::T T;
  constexpr int V = Bits<T>::V;
  // a row is owned by bp.lpr lanes (a power of two up to 64: a whole wavefront for long rows)
  const uint32_t item = (blockIdx.x * 256u + threadIdx.x) / (uint32_t)bp.lpr;
  if (item >= bp.total) return;
  const int lane = threadIdx.x & (bp.lpr - 1);
  const int D = g.n[0], H = g.n[1], W = g.n[2];
  const uint32_t pp = mdiv(item, bp.div_rows);
  const uint32_t idx = item - pp * bp.rows_per_plane;
  int d, h;
  if (idx < (uint32_t)bp.nbd * (uint32_t)H) {
    const uint32_t k = mdiv(idx, bp.div_h);
    d = border_coord((int)k, D, g.lo[0], g.hi[0]);
    h = (int)(idx - k * (uint32_t)H);
  } else {
    const uint32_t idx2 = idx - (uint32_t)bp.nbd * (uint32_t)H;
    const uint32_t di = mdiv(idx2, bp.div_nbh);
    d = g.hi[0] + (int)di;
    h = border_coord((int)(idx2 - di * (uint32_t)bp.nbh), H, g.lo[1], g.hi[1]);
  }
  const long long p = (long long)pp;
  T* drow = gx + ((p * D + d) * H + h) * (long long)W;
  const int n_vec = W / V;
  for (int j = lane; j < n_vec; j += bp.lpr) fold_span<DT>(drow, drow, g, p, d, h, j * V, V);
  if (lane == 0 && n_vec * V < W) fold_span<DT>(drow, drow, g, p, d, h, n_vec * V, W - n_vec * V);
}

template <int DT>
__global__ __launch_bounds__(256) void fold_border_cols_kernel(Table tab, typename Arith<DT>::T* __restrict__ gx,
                                                               Geom g, BorderPlan bp) {
  typedef typename Arith<DT>::T T;
  const uint32_t item = blockIdx.x * 256u + threadIdx.x;  // (row, edge cell), cell fastest
  if (item >= bp.total) return;
  const int D = g.n[0], H = g.n[1], W = g.n[2];
  const uint32_t row = mdiv(item, bp.div_edge);
  const int q = (int)(item - row * (uint32_t)bp.n_edge);
  const uint32_t t2 = mdiv(row, bp.div_hh);
  const int h = (int)(row - t2 * (uint32_t)H);
  const uint32_t pp = mdiv(t2, bp.div_d);
  const int d = (int)(t2 - pp * (uint32_t)D);
  // rows that a D or H neighbour reaches belong to the other kernel
  if (!((d >= g.hi[0]) && (d < D - g.lo[0]) && (h >= g.hi[1]) && (h < H - g.lo[1]))) return;
  const int up0 = W - g.lo[2];
  const int c = q < bp.head ? q : up0 + (q - bp.head);
  T* cell = gx + (long long)row * W + c;
  float acc = 0.0f;
  if (c < g.hi[2]) {
    const T* s_lo = static_cast<const T*>(table_entry(9 + 3 + 0));
    if (s_lo != nullptr) acc = Arith<DT>::up(Arith<DT>::down(acc + Arith<DT>::up(s_lo[(long long)row * g.hi[2] + c])));
  }
  acc = Arith<DT>::up(Arith<DT>::down(acc + Arith<DT>::up(*cell)));
  if (c >= up0) {
    const T* s_hi = static_cast<const T*>(table_entry(9 + 3 + 2));
    if (s_hi != nullptr)
      acc = Arith<DT>::up(Arith<DT>::down(acc + Arith<DT>::up(s_hi[(long long)row * g.lo[2] + (c - up0)])));
  }
  *cell = Arith<DT>::down(acc);
}

Magic make_magic(uint32_t d) {
  Magic k;
  k.one = (d == 1);
  k.m = 0;
  k.s = 1;
  if (d <= 1) return k;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;  // ceil(log2 d)
  k.s = s;
  k.m = (uint32_t)(((1ull << 32) * ((1ull << s) - d)) / d + 1);
  return k;
}

// Lanes per row / vectors per lane for rows of `nvec` 16-byte vectors.
bool make_plan(unsigned long long nrows, int nvec, uint32_t div_h, uint32_t div_d, RowPlan* pl) {
  int lg = 0;  // fewest lanes that cover the row with one batch each, at most a wavefront
  while ((1 << lg) * 2 < nvec && lg < 6) ++lg;
  const int lpr = 1 << lg;
  if (nrows == 0 || nrows * (unsigned long long)lpr >= (1ull << 32)) return false;
  pl->nrows = (uint32_t)nrows;
  pl->lpr_log2 = lg;
  pl->nvec = nvec;
  pl->iters = (nvec + lpr - 1) / lpr;
  pl->div_h = make_magic(div_h);
  pl->div_d = make_magic(div_d);
  return true;
}

// ---------------------------------------------------------------- host side
int check_geom(const jg_halo_geom* g, const char* who, bool adjacent_only) {
  JG_REQUIRE(g != nullptr, "%s: geom is NULL", who);
  JG_REQUIRE(g->planes >= 0, "%s: planes < 0", who);
  for (int a = 0; a < 3; ++a) {
    JG_REQUIRE(g->size[a] >= 1, "%s: size[%d] = %d must be >= 1", who, a, g->size[a]);
    JG_REQUIRE(g->lo[a] >= 0 && g->hi[a] >= 0, "%s: negative halo on axis %d", who, a);
    if (adjacent_only)
      JG_REQUIRE(g->lo[a] <= g->size[a] && g->hi[a] <= g->size[a],
                 "%s: halo (%d, %d) wider than the tile (%d) on axis %d: strips would "
                 "come from non-adjacent ranks",
                 who, g->lo[a], g->hi[a], g->size[a], a);
  }
  return JG_OK;
}

Geom to_geom(const jg_halo_geom* g) {
  Geom r;
  r.planes = g->planes;
  for (int a = 0; a < 3; ++a) {
    r.n[a] = g->size[a];
    r.lo[a] = g->lo[a];
    r.hi[a] = g->hi[a];
  }
  return r;
}

int grid_for(unsigned long long nvec) {
  unsigned long long blocks = (nvec + 255) / 256;
  // Enough to cover the chip many times over; the kernels grid-stride beyond it.
  const unsigned long long cap = 1u << 20;
  if (blocks > cap) blocks = cap;
  if (blocks == 0) blocks = 1;
  return (int)blocks;
}

void expand9(const void* const in[9], const void* out[27]) {
  for (int i = 0; i < 27; ++i) out[i] = nullptr;
  for (int i = 0; i < 9; ++i) out[9 + i] = in[i];
}

jg_halo_geom geom2d(int64_t planes, int H, int W, int lo_h, int hi_h, int lo_w, int hi_w) {
  jg_halo_geom g;
  g.planes = planes;
  g.size[0] = 1; g.size[1] = H; g.size[2] = W;
  g.lo[0] = 0; g.lo[1] = lo_h; g.lo[2] = lo_w;
  g.hi[0] = 0; g.hi[1] = hi_h; g.hi[2] = hi_w;
  return g;
}

}  // namespace

extern "C" int jg_halo_assemble_3d(void* x_aug, const void* const src[27],
                                   const jg_halo_geom* geom, int elem_size, void* stream) {
  int rc = check_geom(geom, "jg_halo_assemble_3d", true);
  if (rc) return rc;
  JG_REQUIRE(x_aug != nullptr && src != nullptr, "jg_halo_assemble_3d: NULL pointer");
  JG_REQUIRE(src[13] != nullptr, "jg_halo_assemble_3d: slot 13 (own tile) is NULL");
  JG_REQUIRE(elem_size == 2 || elem_size == 4,
             "jg_halo_assemble_3d: elem_size %d not in {2, 4}", elem_size);
  JG_REQUIRE((reinterpret_cast<uintptr_t>(x_aug) & 15) == 0,
             "jg_halo_assemble_3d: x_aug must be 16-byte aligned");
  Table tab;
  for (int i = 0; i < 27; ++i) {
    tab.p[i] = src[i];
    JG_REQUIRE((reinterpret_cast<uintptr_t>(src[i]) & (elem_size - 1)) == 0,
               "jg_halo_assemble_3d: slot %d is not element aligned", i);
  }
  Geom g = to_geom(geom);
  unsigned long long total = (unsigned long long)g.planes;
  for (int a = 0; a < 3; ++a) total *= (unsigned long long)(g.lo[a] + g.n[a] + g.hi[a]);
  if (total == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int Da = g.lo[0] + g.n[0] + g.hi[0], Ha = g.lo[1] + g.n[1] + g.hi[1];
  const int Wa = g.lo[2] + g.n[2] + g.hi[2];
  RowPlan pl;
  const int V = 16 / elem_size;
  if ((Wa * elem_size) % 4 == 0 &&
      make_plan((unsigned long long)g.planes * Da * Ha, (Wa + V - 1) / V, Ha, Da, &pl)) {
    const unsigned blocks = (unsigned)((((unsigned long long)pl.nrows << pl.lpr_log2) + 255) / 256);
    if (elem_size == 2)
      assemble_rows_kernel<uint16_t><<<blocks, 256, 0, s>>>(tab, static_cast<uint16_t*>(x_aug), g, pl);
    else
      assemble_rows_kernel<uint32_t><<<blocks, 256, 0, s>>>(tab, static_cast<uint32_t*>(x_aug), g, pl);
    JG_CHECK_LAUNCH("jg_halo_assemble_3d");
    return JG_OK;
  }
  const bool wide = total >= (1ull << 31);
  if (elem_size == 2) {
    int grid = grid_for((total + 7) / 8);
    if (wide)
      assemble_kernel<uint16_t, unsigned long long><<<grid, 256, 0, s>>>(
          tab, static_cast<uint16_t*>(x_aug), g, total);
    else
      assemble_kernel<uint16_t, uint32_t><<<grid, 256, 0, s>>>(
          tab, static_cast<uint16_t*>(x_aug), g, (uint32_t)total);
  } else {
    int grid = grid_for((total + 3) / 4);
    if (wide)
      assemble_kernel<uint32_t, unsigned long long><<<grid, 256, 0, s>>>(
          tab, static_cast<uint32_t*>(x_aug), g, total);
    else
      assemble_kernel<uint32_t, uint32_t><<<grid, 256, 0, s>>>(
          tab, static_cast<uint32_t*>(x_aug), g, (uint32_t)total);
  }
  JG_CHECK_LAUNCH("jg_halo_assemble_3d");
  return JG_OK;
}

extern "C" int jg_halo_assemble_frame_3d(void* x_aug, const void* const src[27],
                                         const jg_halo_geom* geom, const int32_t band_lo[3],
                                         const int32_t band_hi[3], int elem_size, void* stream) {
  const char* who = "jg_halo_assemble_frame_3d";
  int rc = check_geom(geom, who, true);
  if (rc) return rc;
  JG_REQUIRE(x_aug != nullptr && src != nullptr && band_lo != nullptr && band_hi != nullptr, "%s: NULL pointer", who);
  JG_REQUIRE(src[13] != nullptr, "%s: slot 13 (own tile) is NULL", who);
  JG_REQUIRE(elem_size == 2 || elem_size == 4, "%s: elem_size %d not in {2, 4}", who, elem_size);
  Table tab;
  for (int i = 0; i < 27; ++i) {
    tab.p[i] = src[i];
    JG_REQUIRE((reinterpret_cast<uintptr_t>(src[i]) & (elem_size - 1)) == 0, "%s: slot %d is not element aligned", who, i);
  }
  JG_REQUIRE((reinterpret_cast<uintptr_t>(x_aug) & (elem_size - 1)) == 0, "%s: x_aug is not element aligned", who);
  Geom g = to_geom(geom);
  int ext[3], blo[3], bhi[3];
  for (int a = 0; a < 3; ++a) {
    ext[a] = g.lo[a] + g.n[a] + g.hi[a];
    JG_REQUIRE(band_lo[a] >= 0 && band_hi[a] >= 0, "%s: negative band on axis %d", who, a);
    blo[a] = band_lo[a];
    bhi[a] = band_hi[a];
    if (blo[a] + bhi[a] >= ext[a]) {  // the bands meet: the whole axis
      blo[a] = ext[a];
      bhi[a] = 0;
    }
  }
  if (g.planes == 0 || ext[0] == 0 || ext[1] == 0 || ext[2] == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int V = 16 / elem_size;
  FramePlan fp;
  fp.bd_lo = blo[0]; fp.bd_hi = bhi[0]; fp.bh_lo = blo[1]; fp.bh_hi = bhi[1];
  fp.nbd = blo[0] + bhi[0];
  fp.nbh = blo[1] + bhi[1];
  auto launch = [&](int full_rows, int c_begin, int c_end) -> int {
    if (c_end <= c_begin) return JG_OK;
    fp.full_rows = full_rows;
    fp.c_begin = c_begin;
    fp.c_end = c_end;
    unsigned long long rpp;
    if (full_rows) {
      rpp = (unsigned long long)fp.nbd * ext[1] + (unsigned long long)(ext[0] - fp.nbd) * fp.nbh;
      fp.div_a = make_magic((uint32_t)ext[1]);
      fp.div_b = make_magic((uint32_t)(fp.nbh > 0 ? fp.nbh : 1));
    } else {
      rpp = (unsigned long long)(ext[0] - fp.nbd) * (ext[1] - fp.nbh);
      fp.div_a = make_magic((uint32_t)(ext[1] - fp.nbh > 0 ? ext[1] - fp.nbh : 1));
      fp.div_b = fp.div_a;
    }
    if (rpp == 0) return JG_OK;
    const int nvec = (c_end - c_begin + V - 1) / V + 1;
    int lg = 0;
    while ((1 << lg) * 2 < nvec && lg < 6) ++lg;
    fp.lpr_log2 = lg;
    const unsigned long long rows = (unsigned long long)g.planes * rpp;
    JG_REQUIRE((rows << lg) < (1ull << 32), "%s: too many rows (%llu)", who, rows);
    fp.rows_per_plane = (uint32_t)rpp;
    fp.total_rows = (uint32_t)rows;
    fp.div_rows = make_magic((uint32_t)rpp);
    const unsigned blocks = (unsigned)(((rows << lg) + 255) / 256);
    if (elem_size == 2)
      assemble_frame_kernel<uint16_t><<<blocks, 256, 0, s>>>(tab, static_cast<uint16_t*>(x_aug), g, fp);
    else
      assemble_frame_kernel<uint32_t><<<blocks, 256, 0, s>>>(tab, static_cast<uint32_t*>(x_aug), g, fp);
    JG_CHECK_LAUNCH(who);
    return JG_OK;
  };
  rc = launch(1, 0, ext[2]);                        // rows inside a D or H band, whole
  if (rc) return rc;
  rc = launch(0, 0, blo[2]);                        // other rows: first W band
  if (rc) return rc;
  return launch(0, ext[2] - bhi[2], ext[2]);        // other rows: last W band
}

extern "C" int jg_halo_assemble_2d(void* x_aug, const void* const src[9], int64_t planes,
                                   int H, int W, int lo_h, int hi_h, int lo_w, int hi_w,
                                   int elem_size, void* stream) {
  JG_REQUIRE(src != nullptr, "jg_halo_assemble_2d: src is NULL");
  const void* t[27];
  expand9(src, t);
  jg_halo_geom g = geom2d(planes, H, W, lo_h, hi_h, lo_w, hi_w);
  return jg_halo_assemble_3d(x_aug, t, &g, elem_size, stream);
}

extern "C" int jg_halo_pack_3d(void* const strips[27], const void* src,
                               const jg_halo_geom* geom, int from_padded, int elem_size,
                               void* stream) {
  int rc = check_geom(geom, "jg_halo_pack_3d", true);
  if (rc) return rc;
  JG_REQUIRE(strips != nullptr && src != nullptr, "jg_halo_pack_3d: NULL pointer");
  JG_REQUIRE(elem_size == 2 || elem_size == 4, "jg_halo_pack_3d: elem_size %d not in {2, 4}",
             elem_size);
  Geom g = to_geom(geom);
  PackArgs a;
  long long biggest = 0;
  for (int od = -1; od <= 1; ++od)
    for (int oh = -1; oh <= 1; ++oh)
      for (int ow = -1; ow <= 1; ++ow) {
        const int slot = (od + 1) * 9 + (oh + 1) * 3 + (ow + 1);
        const int o[3] = {od, oh, ow};
        a.dst[slot] = (slot == 13) ? nullptr : strips[slot];
        for (int ax = 0; ax < 3; ++ax) {
          int org, ext;
          if (!from_padded) {
            // forward: the block of my tile that lies in that neighbour's halo
            if (o[ax] < 0) { org = 0; ext = g.hi[ax]; }
            else if (o[ax] == 0) { org = 0; ext = g.n[ax]; }
            else { org = g.n[ax] - g.lo[ax]; ext = g.lo[ax]; }
          } else {
            // backward: the block of my padded gradient that neighbour owns
            if (o[ax] < 0) { org = 0; ext = g.lo[ax]; }
            else if (o[ax] == 0) { org = g.lo[ax]; ext = g.n[ax]; }
            else { org = g.lo[ax] + g.n[ax]; ext = g.hi[ax]; }
          }
          a.box[slot].org[ax] = org;
          a.box[slot].ext[ax] = ext;
        }
        // work items of the slot: 16-byte chunks, whole rows of the strip each
        const int per_vec = 16 / elem_size;
        long long cnt = g.planes * (long long)a.box[slot].ext[0] * a.box[slot].ext[1] *
                        ((a.box[slot].ext[2] + per_vec - 1) / per_vec);
        if (cnt == 0) a.dst[slot] = nullptr;
        if (a.dst[slot] != nullptr && cnt > biggest) biggest = cnt;
      }
  if (biggest == 0) return JG_OK;
  int Sd = g.n[0], Sh = g.n[1], Sw = g.n[2];
  if (from_padded) {
    Sd += g.lo[0] + g.hi[0];
    Sh += g.lo[1] + g.hi[1];
    Sw += g.lo[2] + g.hi[2];
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Both faces across W wanted, at most two cells thick, from rows of more than one cache line,
  // and many of them: one pass that takes both ends of a row (the kernel above says why).
  {
    const Box &lo = a.box[12], &hi = a.box[14];
    const unsigned long long rows = (unsigned long long)g.planes * lo.ext[0] * lo.ext[1];
    if (a.dst[12] != nullptr && a.dst[14] != nullptr && lo.ext[2] <= 2 && hi.ext[2] <= 2 &&
        (long long)Sw * elem_size > 128 && rows >= (1u << 16) && rows < (1ull << 32)) {
      const unsigned blocks = (unsigned)((rows + 1023) / 1024);
      if (elem_size == 2)
        pack_w_faces_kernel<uint16_t><<<blocks, 256, 0, s>>>(static_cast<uint16_t*>(a.dst[12]), static_cast<uint16_t*>(a.dst[14]),
                                                             static_cast<const uint16_t*>(src), lo, hi, (unsigned)rows, Sd, Sh, Sw);
      else
        pack_w_faces_kernel<uint32_t><<<blocks, 256, 0, s>>>(static_cast<uint32_t*>(a.dst[12]), static_cast<uint32_t*>(a.dst[14]),
                                                             static_cast<const uint32_t*>(src), lo, hi, (unsigned)rows, Sd, Sh, Sw);
      JG_CHECK_LAUNCH("jg_halo_pack_3d");
      a.dst[12] = a.dst[14] = nullptr;
      biggest = 0;
      for (int slot = 0; slot < 27; ++slot) {
        const long long cnt = g.planes * (long long)a.box[slot].ext[0] * a.box[slot].ext[1] *
                              ((a.box[slot].ext[2] + 16 / elem_size - 1) / (16 / elem_size));
        if (a.dst[slot] != nullptr && cnt > biggest) biggest = cnt;
      }
      if (biggest == 0) return JG_OK;
    }
  }
  long long bx = (biggest + 255) / 256;
  if (bx > 4096) bx = 4096;
  dim3 grid((unsigned)bx, 27, 1);
  const bool narrow = (unsigned long long)g.planes * Sd * Sh * Sw < (1ull << 31);
  if (elem_size == 2) {
    if (narrow)
      pack_kernel<uint16_t, uint32_t><<<grid, 256, 0, s>>>(a, static_cast<const uint16_t*>(src), g.planes, Sd, Sh, Sw);
    else
      pack_kernel<uint16_t, unsigned long long><<<grid, 256, 0, s>>>(a, static_cast<const uint16_t*>(src), g.planes, Sd,
                                                                     Sh, Sw);
  } else {
    if (narrow)
      pack_kernel<uint32_t, uint32_t><<<grid, 256, 0, s>>>(a, static_cast<const uint32_t*>(src), g.planes, Sd, Sh, Sw);
    else
      pack_kernel<uint32_t, unsigned long long><<<grid, 256, 0, s>>>(a, static_cast<const uint32_t*>(src), g.planes, Sd,
                                                                     Sh, Sw);
  }
  JG_CHECK_LAUNCH("jg_halo_pack_3d");
  return JG_OK;
}

extern "C" int jg_halo_pack_2d(void* const strips[9], const void* src, int64_t planes, int H,
                               int W, int lo_h, int hi_h, int lo_w, int hi_w, int from_padded,
                               int elem_size, void* stream) {
  JG_REQUIRE(strips != nullptr, "jg_halo_pack_2d: strips is NULL");
  void* t[27];
  for (int i = 0; i < 27; ++i) t[i] = nullptr;
  for (int i = 0; i < 9; ++i) t[9 + i] = strips[i];
  jg_halo_geom g = geom2d(planes, H, W, lo_h, hi_h, lo_w, hi_w);
  return jg_halo_pack_3d(t, src, &g, from_padded, elem_size, stream);
}

namespace {
// Plan of the two in-place border kernels; false when the counts do not fit their 32-bit indices.
bool border_plan(const Geom& g, BorderPlan* bp, unsigned long long* row_items, unsigned long long* col_items) {
  const int D = g.n[0], H = g.n[1], W = g.n[2];
  const unsigned long long nrows = (unsigned long long)g.planes * D * H;
  bp->nbd = (g.hi[0] + g.lo[0] >= D) ? D : g.hi[0] + g.lo[0];
  bp->nbh = (g.hi[1] + g.lo[1] >= H) ? H : g.hi[1] + g.lo[1];
  bp->rows_per_plane = (uint32_t)bp->nbd * (uint32_t)H + (uint32_t)(D - bp->nbd) * (uint32_t)bp->nbh;
  const int up0 = W - g.lo[2];
  bp->head = g.hi[2] < up0 ? g.hi[2] : up0;
  bp->n_edge = bp->head + (W - up0);
  bp->div_rows = make_magic(bp->rows_per_plane > 0 ? bp->rows_per_plane : 1);
  bp->div_h = make_magic((uint32_t)H);
  bp->div_nbh = make_magic((uint32_t)(bp->nbh > 0 ? bp->nbh : 1));
  bp->div_edge = make_magic((uint32_t)(bp->n_edge > 0 ? bp->n_edge : 1));
  bp->div_hh = make_magic((uint32_t)H);
  bp->div_d = make_magic((uint32_t)D);
  *row_items = (unsigned long long)g.planes * bp->rows_per_plane;
  *col_items = nrows * (unsigned long long)bp->n_edge;
  return *row_items < (1ull << 31) && *col_items < (1ull << 31) && nrows < (1ull << 31);
}
// The rows a D or H neighbour reaches, summed in full in place; false if there are too many.
template <int DT>
bool launch_border_rows(const Table& tab, void* gx, const Geom& g, BorderPlan bp, unsigned long long row_items, hipStream_t s) {
  typedef typename Arith<DT>::T T;
  if (row_items == 0) return true;
  bp.total = (uint32_t)row_items;
  const int vecs = g.n[2] / (16 / (int)sizeof(T));
  bp.lpr = 1;
  while (bp.lpr < 64 && bp.lpr < vecs) bp.lpr *= 2;
  const unsigned long long threads = row_items * (unsigned long long)bp.lpr;
  if (threads >= (1ull << 32)) return false;
  fold_border_rows_kernel<DT><<<(unsigned)((threads + 255) / 256), 256, 0, s>>>(tab, static_cast<T*>(gx), g, bp);
  return true;
}
}  // namespace

extern "C" int jg_halo_fold_3d(void* gx, const void* gx_aug, const void* const strips[27],
                               const jg_halo_geom* geom, int dtype, void* stream) {
  int rc = check_geom(geom, "jg_halo_fold_3d", true);
  if (rc) return rc;
  JG_REQUIRE(gx != nullptr && gx_aug != nullptr && strips != nullptr,
             "jg_halo_fold_3d: NULL pointer");
  JG_REQUIRE(dtype == JG_F32 || dtype == JG_BF16 || dtype == JG_F16,
             "jg_halo_fold_3d: unknown dtype %d", dtype);
  JG_REQUIRE((reinterpret_cast<uintptr_t>(gx) & 15) == 0,
             "jg_halo_fold_3d: gx must be 16-byte aligned");
  const int es = (int)jg::dtype_size(dtype);
  Table tab;
  for (int i = 0; i < 27; ++i) {
    tab.p[i] = (i == 13) ? nullptr : strips[i];
    JG_REQUIRE((reinterpret_cast<uintptr_t>(tab.p[i]) & (es - 1)) == 0,
               "jg_halo_fold_3d: slot %d is not element aligned", i);
  }
  JG_REQUIRE((reinterpret_cast<uintptr_t>(gx_aug) & (es - 1)) == 0,
             "jg_halo_fold_3d: gx_aug is not element aligned");
  Geom g = to_geom(geom);
  unsigned long long total = (unsigned long long)g.planes * g.n[0] * g.n[1] * g.n[2];
  unsigned long long total_aug = (unsigned long long)g.planes;
  for (int a = 0; a < 3; ++a) total_aug *= (unsigned long long)(g.lo[a] + g.n[a] + g.hi[a]);
  if (total == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int V = 16 / es;
  RowPlan pl;
  if ((g.n[2] * es) % 4 == 0 &&
      make_plan((unsigned long long)g.planes * g.n[0] * g.n[1], (g.n[2] + V - 1) / V, g.n[1], g.n[0], &pl)) {
    const unsigned blocks = (unsigned)((((unsigned long long)pl.nrows << pl.lpr_log2) + 255) / 256);
    // Two launches when the rows a D or H neighbour reaches are many enough to matter (more than one
    // row in 64) and fit the border kernel's indices: the row pass defers them, the border kernel
    // sums them in place from the `0 + own` the row pass left (the same bits: the ordered sum starts
    // from zero, so the sign of a zero in the own term cannot reach the result).
    BorderPlan bp;
    unsigned long long row_items = 0, col_items = 0;
    const bool planned = border_plan(g, &bp, &row_items, &col_items);
    const int vecs = g.n[2] / V;
    int border_lpr = 1;
    while (border_lpr < 64 && border_lpr < vecs) border_lpr *= 2;
    const bool defer = planned && row_items * 64 > (unsigned long long)pl.nrows &&
                       row_items * (unsigned long long)border_lpr < (1ull << 32);
    bool ok = true;
    if (dtype == JG_F32) {
      fold_rows_kernel<JG_F32><<<blocks, 256, 0, s>>>(tab, static_cast<uint32_t*>(gx), static_cast<const uint32_t*>(gx_aug), g, pl, defer);
      if (defer) ok = launch_border_rows<JG_F32>(tab, gx, g, bp, row_items, s);
    } else if (dtype == JG_BF16) {
      fold_rows_kernel<JG_BF16><<<blocks, 256, 0, s>>>(tab, static_cast<uint16_t*>(gx), static_cast<const uint16_t*>(gx_aug), g, pl, defer);
      if (defer) ok = launch_border_rows<JG_BF16>(tab, gx, g, bp, row_items, s);
    } else {
      fold_rows_kernel<JG_F16><<<blocks, 256, 0, s>>>(tab, static_cast<uint16_t*>(gx), static_cast<const uint16_t*>(gx_aug), g, pl, defer);
      if (defer) ok = launch_border_rows<JG_F16>(tab, gx, g, bp, row_items, s);
    }
    JG_REQUIRE(ok, "jg_halo_fold_3d: too many border rows");
    JG_CHECK_LAUNCH("jg_halo_fold_3d");
    return JG_OK;
  }
  const bool wide = total_aug >= (1ull << 31);
  int grid = grid_for((total + V - 1) / V);
#define JG_FOLD(DT)                                                                         \
  do {                                                                                      \
    typedef Arith<DT>::T T;                                                                 \
    if (wide)                                                                               \
      fold_kernel<DT, unsigned long long><<<grid, 256, 0, s>>>(                             \
          static_cast<T*>(gx), static_cast<const T*>(gx_aug), tab, g, total);               \
    else                                                                                    \
      fold_kernel<DT, uint32_t><<<grid, 256, 0, s>>>(                                       \
          static_cast<T*>(gx), static_cast<const T*>(gx_aug), tab, g, (uint32_t)total);     \
  } while (0)
  if (dtype == JG_F32) JG_FOLD(JG_F32);
  else if (dtype == JG_BF16) JG_FOLD(JG_BF16);
  else JG_FOLD(JG_F16);
#undef JG_FOLD
  JG_CHECK_LAUNCH("jg_halo_fold_3d");
  return JG_OK;
}

extern "C" int jg_halo_fold_border_3d(void* gx, const void* const strips[27],
                                      const jg_halo_geom* geom, int dtype, void* stream) {
  int rc = check_geom(geom, "jg_halo_fold_border_3d", true);
  if (rc) return rc;
  JG_REQUIRE(gx != nullptr && strips != nullptr, "jg_halo_fold_border_3d: NULL pointer");
  JG_REQUIRE(dtype == JG_F32 || dtype == JG_BF16 || dtype == JG_F16,
             "jg_halo_fold_border_3d: unknown dtype %d", dtype);
  const int es = (int)jg::dtype_size(dtype);
  JG_REQUIRE((reinterpret_cast<uintptr_t>(gx) & (es - 1)) == 0,
             "jg_halo_fold_border_3d: gx is not element aligned");
  Table tab;
  for (int i = 0; i < 27; ++i) {
    tab.p[i] = (i == 13) ? nullptr : strips[i];
    JG_REQUIRE((reinterpret_cast<uintptr_t>(tab.p[i]) & (es - 1)) == 0,
               "jg_halo_fold_border_3d: slot %d is not element aligned", i);
  }
  Geom g = to_geom(geom);
  const int D = g.n[0], H = g.n[1], W = g.n[2];
  const unsigned long long nrows = (unsigned long long)g.planes * D * H;
  if (nrows == 0 || W == 0) return JG_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  BorderPlan bp;
  unsigned long long row_items = 0, col_items = 0;
  JG_REQUIRE(border_plan(g, &bp, &row_items, &col_items), "jg_halo_fold_border_3d: too many rows (%llu)", nrows);
#define JG_BORDER(DT)                                                                                   \
  do {                                                                                                  \
    typedef Arith<DT>::T T;                                                                             \
    JG_REQUIRE(launch_border_rows<DT>(tab, gx, g, bp, row_items, s),                                    \
               "jg_halo_fold_border_3d: too many border rows (%llu)", row_items);                      \
    if (col_items > 0) {                                                                                \
      bp.total = (uint32_t)col_items;                                                                   \
      fold_border_cols_kernel<DT><<<(unsigned)((col_items + 255) / 256), 256, 0, s>>>(tab, static_cast<T*>(gx), g, bp); \
    }                                                                                                   \
  } while (0)
  if (dtype == JG_F32) JG_BORDER(JG_F32);
  else if (dtype == JG_BF16) JG_BORDER(JG_BF16);
  else JG_BORDER(JG_F16);
#undef JG_BORDER
  JG_CHECK_LAUNCH("jg_halo_fold_border_3d");
  return JG_OK;
}

extern "C" int jg_halo_fold_2d(void* gx, const void* gx_aug, const void* const strips[9],
                               int64_t planes, int H, int W, int lo_h, int hi_h, int lo_w,
                               int hi_w, int dtype, void* stream) {
  JG_REQUIRE(strips != nullptr, "jg_halo_fold_2d: strips is NULL");
  const void* t[27];
  expand9(strips, t);
  jg_halo_geom g = geom2d(planes, H, W, lo_h, hi_h, lo_w, hi_w);
  return jg_halo_fold_3d(gx, gx_aug, t, &g, dtype, stream);
}
