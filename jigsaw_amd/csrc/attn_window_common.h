// Pieces shared by the window-attention kernels (64 queries x 64 keys, head size 32, one
// wavefront per (window, head) entry): fragment layouts, the LDS tile, packing of accumulators.
#pragma once
#include "jg_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int N = 64;         // queries = keys per window
constexpr int D = 32;         // head size
constexpr int WAVES = 4;      // entries per workgroup
constexpr int PITCH = 80;     // bytes per tile row in LDS: 64 + 16, so that the rows 4 apart
                              // that the two lane halves of a transposed read touch fall
                              // into different banks
constexpr int TILE = N * PITCH;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

__device__ inline bf16x8 load_frag(const uint16_t* row_major, int row, int ks, int kg) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(row_major + row * D + ks * 16 + kg * 8));
}

// The fragment registers of a 64 x 32 operand are the whole tile: to LDS, row-major.
__device__ inline void store_tile(unsigned char* tile, const bf16x8 (&f)[2][2], int ln, int kg) {
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
      *reinterpret_cast<u32x4*>(tile + (b * 32 + ln) * PITCH + (ks * 16 + kg * 8) * 2) = __builtin_bit_cast(u32x4, f[b][ks]);
}

// Transposed A fragment of K-step t: slot j = element [16 t + 8 (j / 4) + 4 kg + j % 4][ln].
__device__ inline bf16x8 frag_tr(const unsigned char* tile, int t, int ln, int kg) {
  bf16x8 r;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int row = t * 16 + (j >> 2) * 8 + kg * 4 + (j & 3);
    r[j] = *reinterpret_cast<const __bf16*>(tile + row * PITCH + ln * 2);
  }
  return r;
}

// Slots of K-step h (0 / 1) of a 32-row accumulator block, rounded to bf16.
__device__ inline bf16x8 pack_half(const float (&v)[16], int h) {
  bf16x8 r;
#pragma unroll
  for (int j = 0; j < 8; j += 2) {
    const f32x2 v2 = {v[h * 8 + j], v[h * 8 + j + 1]};
    const bf16x2 h2 = __builtin_convertvector(v2, bf16x2);
    r[j] = h2.x;
    r[j + 1] = h2.y;
  }
  return r;
}

// Rows 8 i4 + 4 kg .. + 3 of a 32 x 32 accumulator as 4 bf16 (one 8-byte store).
__device__ inline u32x2 pack_rows(const f32x16& a, int i4, float mul) {
  const f32x2 lo = {a[i4 * 4 + 0] * mul, a[i4 * 4 + 1] * mul};
  const f32x2 hi = {a[i4 * 4 + 2] * mul, a[i4 * 4 + 3] * mul};
  u32x2 r;
  r.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2));
  r.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2));
  return r;
}

__device__ inline f32x16 zero16() {
  f32x16 z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.0f;
  return z;
}

}  // namespace
