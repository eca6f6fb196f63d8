// Shared device/host helpers for the gfx950 HiLS kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <math.h>

#define HILS_OK 0
#define HILS_ERR_ARG 1
#define HILS_ERR_LAUNCH 2

// Last-error text, readable through hils_last_error().
void hils_set_error(const char* fmt, ...);

#define HILS_REQUIRE(cond, ...)            \
  do {                                     \
    if (!(cond)) {                         \
      hils_set_error(__VA_ARGS__);         \
      return HILS_ERR_ARG;                 \
    }                                      \
  } while (0)

#define HILS_CHECK_LAUNCH(name)                                            \
  do {                                                                     \
    hipError_t e__ = hipGetLastError();                                    \
    if (e__ != hipSuccess) {                                               \
      hils_set_error("%s: launch failed: %s", name, hipGetErrorString(e__)); \
      return HILS_ERR_LAUNCH;                                              \
    }                                                                      \
  } while (0)

// Compute units of the current device (cached per device; no stream operation, so it is safe
// under HIP graph capture).
int hils_device_cus();

// Raise a kernel's dynamic-LDS limit to `bytes` on the current device if it is not there yet.
// One HilsLdsReserve per kernel instantiation (a function-local static); thread-safe, per device.
#ifdef __cplusplus
#include <atomic>
#define HILS_LDS_RESERVE_DEVICES 64
struct HilsLdsReserve { std::atomic<size_t> bytes[HILS_LDS_RESERVE_DEVICES]; };
int hils_reserve_lds(HilsLdsReserve* state, const void* kernel, size_t bytes, const char* who);
#endif

typedef unsigned short bf16_t;  // raw bfloat16 bits

#define HILS_NEG_INF (-INFINITY)
#define HILS_LOG2E 1.4426950408889634f
#define HILS_LN2 0.6931471805599453f

__device__ __forceinline__ float bf2f(bf16_t x) { return __uint_as_float(((uint32_t)x) << 16); }

// round-to-nearest-even fp32 -> bf16 on the hardware converter (v_cvt_pk_bf16_f32)
typedef __attribute__((ext_vector_type(2))) __bf16 hils_bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float hils_f32x2_t;

__device__ __forceinline__ uint32_t pack_bf2(float lo, float hi) {
  const hils_f32x2_t x = {lo, hi};
  const hils_bf16x2_t y = __builtin_convertvector(x, hils_bf16x2_t);
  return *(const uint32_t*)&y;
}

__device__ __forceinline__ bf16_t f2bf(float f) { return (bf16_t)(pack_bf2(f, 0.f) & 0xffffu); }

// unpack 8 bf16 held in a uint4 into 8 floats
__device__ __forceinline__ void unpack8(const uint4& v, float* f) {
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
  f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Reductions / broadcast across the four 16-lane rows of a wavefront, per column (lane & 15),
// with the gfx950 row-swap instructions: vector-ALU only, no LDS queue involved.
//   permlane16_swap(x, x) = { [r0, r0, r2, r2], [r1, r1, r3, r3] }   (rows of x)
//   permlane32_swap(x, x) = { [lo, lo], [hi, hi] }                   (halves of x)
typedef unsigned hils_uint2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float rows_max(float x) {
  hils_uint2v a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(a.x), __uint_as_float(a.y));
  hils_uint2v b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b.x), __uint_as_float(b.y));
}
__device__ __forceinline__ float rows_sum(float x) {
  hils_uint2v a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(a.x) + __uint_as_float(a.y);
  hils_uint2v b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(b.x) + __uint_as_float(b.y);
}
// value of row 0 (lanes 0..15) in every row
__device__ __forceinline__ unsigned rows_bcast0(unsigned x) {
  hils_uint2v a = __builtin_amdgcn_permlane16_swap(x, x, false, false);
  hils_uint2v b = __builtin_amdgcn_permlane32_swap(a.x, a.x, false, false);
  return b.x;
}

// block-wide reductions for blockDim.x a multiple of 64, <= 1024; `red` holds >= 17 floats
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += red[i];
  return r;
}
// Workgroup barrier that orders LDS accesses only: global stores issued before it stay in
// flight (a __syncthreads() waits for them too).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
// block_max with LDS-only barriers
__device__ __forceinline__ float block_max_lds(float v, float* red) {
  v = wave_max(v);
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  lds_barrier();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  lds_barrier();
  float r = HILS_NEG_INF;
  for (int i = 0; i < nw; ++i) r = fmaxf(r, red[i]);
  return r;
}

__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float r = HILS_NEG_INF;
  for (int i = 0; i < nw; ++i) r = fmaxf(r, red[i]);
  return r;
}

// floor division for possibly negative numerators (b > 0)
__host__ __device__ __forceinline__ int floordiv(int a, int b) {
  int q = a / b;
  return (a % b != 0 && ((a < 0) != (b < 0))) ? q - 1 : q;
}

// number of chunks visible to the query at global position t: chunk c is visible iff c < limit
__host__ __device__ __forceinline__ int visible_limit(int t_global, int window, int block) {
  return window > 0 ? floordiv(t_global - window + 1, block) : floordiv(t_global, block);
}

// Division of a small unsigned number by a divisor that is fixed for a launch: the host passes
// m = hils_udiv_magic(d) = ceil(2^32 / d) and the device takes the high half of n * m, which is
// floor(n / d) whenever n * d < 2^32 (d = 1 has no 32-bit magic and is passed through).  A division by
// a kernel argument otherwise costs about 35 vector instructions.
__host__ __device__ __forceinline__ uint32_t hils_udiv_magic(uint32_t d) {
  return d <= 1u ? 0u : (uint32_t)((0x100000000ull + d - 1u) / d);
}
__device__ __forceinline__ uint32_t hils_udiv(uint32_t n, uint32_t d, uint32_t m) {
  return d == 1u ? n : __umulhi(n, m);
}

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

// Sum of |w| over the K bf16 elements e0 .. e0+K-1 of a tensor of tot_e elements (a weight row may
// start on any element).  The row is read as aligned dwords, a batch of loads in flight together and
// none of them inside a branch (a load inside a branch is waited for inside it): an index is clamped
// to the last even one whose dword lies inside the tensor and a clamped dword counts for nothing; the
// tensor's last element, when its index is even, has no such dword and is read on its own by the
// one thread whose row ends there.
__device__ __forceinline__ float hils_abs_row_sum_bf16(const bf16_t* __restrict__ w, long e0, int K, long tot_e) {
  constexpr int WDW = 17;  // dwords per round: 32 elements + alignment slack
  if (tot_e < 2) return fabsf(bf2f(w[e0]));
  const long e_end = e0 + K;
  const long last_dw = (tot_e - 2) & ~1L;
  float a = 0.f;
  for (long eb = e0 & ~1L; eb < e_end; eb += 2 * WDW) {
    uint32_t wd[WDW];
#pragma unroll
    for (int u = 0; u < WDW; ++u) {
      const long ee = eb + 2 * u;
      wd[u] = *(const uint32_t*)(w + (ee < last_dw ? ee : last_dw));
    }
#pragma unroll
    for (int u = 0; u < WDW; ++u) {
      const long ee = eb + 2 * u;
      const bool here = ee <= last_dw;
      if (here && ee >= e0 && ee < e_end) a += fabsf(__uint_as_float(wd[u] << 16));
      if (here && ee + 1 >= e0 && ee + 1 < e_end) a += fabsf(__uint_as_float(wd[u] & 0xffff0000u));
    }
  }
  if ((tot_e & 1) && e_end == tot_e) a += fabsf(bf2f(w[tot_e - 1]));
  return a;
}
