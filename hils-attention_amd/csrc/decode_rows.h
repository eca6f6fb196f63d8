// Helpers for the decode-side kernels, which stream (chunk, head) rows of D bf16 values
// with fully coalesced 16-byte lane loads: LR = D/8 neighbouring lanes cover one row, a
// wavefront load instruction covers 64/LR rows.
#pragma once
#include "common.h"

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

// dot product of 8 bf16 pairs held as 4 packed dwords each, fp32 accumulation
__device__ __forceinline__ float dot8_bf16(const uint4& a, const uint4& b, float acc) {
  acc = __builtin_amdgcn_fdot2_f32_bf16(*(const bf16x2_t*)&a.x, *(const bf16x2_t*)&b.x, acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(*(const bf16x2_t*)&a.y, *(const bf16x2_t*)&b.y, acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(*(const bf16x2_t*)&a.z, *(const bf16x2_t*)&b.z, acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(*(const bf16x2_t*)&a.w, *(const bf16x2_t*)&b.w, acc, false);
  return acc;
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  const int v = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true);
  return x + __int_as_float(v);
}

// all-reduce (sum) over aligned groups of LR = 8 or 16 neighbouring lanes
template <int LR>
__device__ __forceinline__ float row_sum(float x) {
  x = dpp_add<0xB1>(x);   // quad_perm [1,0,3,2]
  x = dpp_add<0x4E>(x);   // quad_perm [2,3,0,1]
  x = dpp_add<0x141>(x);  // row_half_mirror
  if (LR == 16) x = dpp_add<0x140>(x);  // row_mirror
  return x;
}

// wavefront-wide integer sum, result uniform: DPP reduction inside each row of 16 lanes,
// then the four row totals are read out with v_readlane
__device__ __forceinline__ int wave_sum_i(int x) {
  x += __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xF, 0xF, true);
  x += __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xF, 0xF, true);
  x += __builtin_amdgcn_update_dpp(0, x, 0x141, 0xF, 0xF, true);
  x += __builtin_amdgcn_update_dpp(0, x, 0x140, 0xF, 0xF, true);
  return __builtin_amdgcn_readlane(x, 0) + __builtin_amdgcn_readlane(x, 16) +
         __builtin_amdgcn_readlane(x, 32) + __builtin_amdgcn_readlane(x, 48);
}

// wavefront-wide unsigned maximum, result uniform
__device__ __forceinline__ uint32_t wave_max_u(uint32_t v) {
  uint32_t x = v, y;
  y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xF, 0xF, true);  x = x > y ? x : y;
  y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, true);  x = x > y ? x : y;
  y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x141, 0xF, 0xF, true); x = x > y ? x : y;
  y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x140, 0xF, 0xF, true); x = x > y ? x : y;
  const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)x, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)x, 16);
  const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)x, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)x, 48);
  const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
  return ab > cd ? ab : cd;
}

// wavefront-wide bitwise AND / OR, result uniform
__device__ __forceinline__ uint32_t wave_and_u(uint32_t v) {
  int x = (int)v;
  x &= __builtin_amdgcn_update_dpp(-1, x, 0xB1, 0xF, 0xF, false);
  x &= __builtin_amdgcn_update_dpp(-1, x, 0x4E, 0xF, 0xF, false);
  x &= __builtin_amdgcn_update_dpp(-1, x, 0x141, 0xF, 0xF, false);
  x &= __builtin_amdgcn_update_dpp(-1, x, 0x140, 0xF, 0xF, false);
  return (uint32_t)(__builtin_amdgcn_readlane(x, 0) & __builtin_amdgcn_readlane(x, 16) &
                    __builtin_amdgcn_readlane(x, 32) & __builtin_amdgcn_readlane(x, 48));
}
__device__ __forceinline__ uint32_t wave_or_u(uint32_t v) {
  int x = (int)v;
  x |= __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xF, 0xF, true);
  x |= __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xF, 0xF, true);
  x |= __builtin_amdgcn_update_dpp(0, x, 0x141, 0xF, 0xF, true);
  x |= __builtin_amdgcn_update_dpp(0, x, 0x140, 0xF, 0xF, true);
  return (uint32_t)(__builtin_amdgcn_readlane(x, 0) | __builtin_amdgcn_readlane(x, 16) |
                    __builtin_amdgcn_readlane(x, 32) | __builtin_amdgcn_readlane(x, 48));
}
