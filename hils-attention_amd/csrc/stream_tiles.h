// Helpers for kernels in which one operand side streams through LDS in 64-row tiles, stored
// row-major (operand of a score product) and/or transposed (operand of a product whose
// contraction runs over the streamed rows).
#pragma once
#include "common.h"

#define LZM_PT 136  // bytes per row of the transposed tile: 64 bf16 + 8 pad

// Rotation of the transposed tile: feature row f keeps its 32 row-pair words rotated by
// (f / 32) * (512 / D) words.  A wavefront of the staging pass holds D/8 feature groups (lane % (D/8))
// times 512/D row pairs; feature groups 4 apart are 4 * 8 * 34 words = a multiple of 64 banks apart, so
// without the rotation the dword stores of a wavefront fell on a quarter (D = 128) or half (D = 64) of
// the banks, four or two lanes each.  The rotation is a compile-time constant for the reader (its
// feature tile index is an unrolled loop variable).
template <int D>
__device__ __forceinline__ constexpr int lzm_rot(int f32_group) { return f32_group * (512 / D); }

// Two adjacent rows of the streamed tile (8 elements each): row-major and element-paired stores.
template <int PITCH>
__device__ __forceinline__ void lzm_stash_pair(unsigned char* rm, unsigned char* tr, int row0,
                                               int seg, const uint4& a, const uint4& b) {
  constexpr int D = (PITCH - 16) / 2;
  *(uint4*)(rm + row0 * PITCH + seg * 16) = a;
  *(uint4*)(rm + (row0 + 1) * PITCH + seg * 16) = b;
  const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
  const int word = (((row0 >> 1) + lzm_rot<D>(seg >> 2)) & 31) * 4;  // byte offset of the row pair
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t lo = __builtin_amdgcn_perm(bw[w], aw[w], 0x05040100u);
    const uint32_t hi = __builtin_amdgcn_perm(bw[w], aw[w], 0x07060302u);
    *(uint32_t*)(tr + (seg * 8 + 2 * w) * LZM_PT + word) = lo;
    *(uint32_t*)(tr + (seg * 8 + 2 * w + 1) * LZM_PT + word) = hi;
  }
}

// Gradient product of one wavefront: acc[rt][dt] += P[rt] (16 owned x 64 streamed) * T (64 x D).
// p[rt][tt] are score-accumulator tiles (lane: owned row = lane & 15, streamed rows 4*(lane>>4)+i
// of tile tt); two tiles form one 32-deep operand, and the transposed tile is read in the same order.
template <int D, int NT>
__device__ __forceinline__ void lzm_grad_product(const unsigned char* tr, const float (&p)[NT][4][4],
                                                 f32x4_t (&acc)[NT][D / 16], int col, int j) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    bf16x8_t a[NT];
#pragma unroll
    for (int rt = 0; rt < NT; ++rt) {
      uint4 u;
      u.x = pack_bf2(p[rt][2 * h][0], p[rt][2 * h][1]);
      u.y = pack_bf2(p[rt][2 * h][2], p[rt][2 * h][3]);
      u.z = pack_bf2(p[rt][2 * h + 1][0], p[rt][2 * h + 1][1]);
      u.w = pack_bf2(p[rt][2 * h + 1][2], p[rt][2 * h + 1][3]);
      a[rt] = *(const bf16x8_t*)&u;
    }
#pragma unroll
    for (int dt = 0; dt < D / 16; ++dt) {
      // rows 32h + 4j .. and 32h + 16 + 4j ..: row-pair words 16h + 2j and 16h + 8 + 2j, rotated
      const unsigned char* row = tr + (dt * 16 + col) * LZM_PT;
      const uint2 b0 = *(const uint2*)(row + ((16 * h + 2 * j + lzm_rot<D>(dt >> 1)) & 31) * 4);
      const uint2 b1 = *(const uint2*)(row + ((16 * h + 8 + 2 * j + lzm_rot<D>(dt >> 1)) & 31) * 4);
      const uint4 bu = {b0.x, b0.y, b1.x, b1.y};
#pragma unroll
      for (int rt = 0; rt < NT; ++rt)
        acc[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt], *(const bf16x8_t*)&bu, acc[rt][dt], 0, 0, 0);
    }
  }
}

