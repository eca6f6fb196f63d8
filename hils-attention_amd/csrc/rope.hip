// Rotary position embedding in the "rotate half" convention: the two halves of a head vector are
// the real and imaginary parts, out1 = x1*c - x2*s, out2 = x2*c' + x1*s'.  fp32 arithmetic on bf16
// inputs, one rounding to bf16 at the end.  Pure HBM streaming: one thread per 16-byte piece of
// the low half, which also loads the matching piece of the high half.
#include "common.h"
#include "../../include/hils_amd.h"

// cos/sin rows hold D values per position; lo_only: both halves use the first D/2 of them
template <bool TAB_F32>
__global__ void __launch_bounds__(256)
rope_kernel(const bf16_t* __restrict__ x, const void* __restrict__ cos_t, const void* __restrict__ sin_t,
            bf16_t* __restrict__ out, long total, int L, int H, int D, long tab_batch_stride, int lo_only,
            float sin_sign) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;  // piece of 8 elements of the low half
  if (i >= total) return;
  const int pph = D / 16;  // pieces per half
  const int pc = (int)(i % pph);
  const long row = i / pph;  // (b*L + l)*H + h
  const long bl = row / H;
  const long l = bl % L, b = bl / L;
  const long xo = row * D + pc * 8;
  const uint4 lo4 = *(const uint4*)(x + xo);
  const uint4 hi4 = *(const uint4*)(x + xo + D / 2);
  float x1[8], x2[8], c1[8], s1[8], c2[8], s2[8];
  unpack8(lo4, x1);
  unpack8(hi4, x2);
  const long to = b * tab_batch_stride + l * D + pc * 8;
  const long th = lo_only ? to : to + D / 2;
  if (TAB_F32) {
    const float* ct = (const float*)cos_t;
    const float* st = (const float*)sin_t;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      c1[e] = ct[to + e]; s1[e] = st[to + e];
      c2[e] = ct[th + e]; s2[e] = st[th + e];
    }
  } else {
    unpack8(*(const uint4*)((const bf16_t*)cos_t + to), c1);
    unpack8(*(const uint4*)((const bf16_t*)sin_t + to), s1);
    unpack8(*(const uint4*)((const bf16_t*)cos_t + th), c2);
    unpack8(*(const uint4*)((const bf16_t*)sin_t + th), s2);
  }
  float o1[8], o2[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    o1[e] = x1[e] * c1[e] - x2[e] * (s1[e] * sin_sign);
    o2[e] = x2[e] * c2[e] + x1[e] * (s2[e] * sin_sign);
  }
  uint4 w1, w2;
  w1.x = pack_bf2(o1[0], o1[1]); w1.y = pack_bf2(o1[2], o1[3]); w1.z = pack_bf2(o1[4], o1[5]); w1.w = pack_bf2(o1[6], o1[7]);
  w2.x = pack_bf2(o2[0], o2[1]); w2.y = pack_bf2(o2[2], o2[3]); w2.z = pack_bf2(o2[4], o2[5]); w2.w = pack_bf2(o2[6], o2[7]);
  *(uint4*)(out + xo) = w1;
  *(uint4*)(out + xo + D / 2) = w2;
}

extern "C" int hils_rope(const void* x, const void* cos_t, const void* sin_t, void* out, int B, int L,
                         int H, int D, int table_per_batch, int table_f32, int lo_only,
                         float sin_sign, void* stream) {
  HILS_REQUIRE(x && cos_t && sin_t && out, "hils_rope: null pointer");
  HILS_REQUIRE(B > 0 && L > 0 && H > 0 && D > 0, "hils_rope: sizes must be positive");
  HILS_REQUIRE(D % 16 == 0, "hils_rope: D (%d) must be a multiple of 16", D);
  const long total = (long)B * L * H * (D / 16);
  const long nblk = (total + 255) / 256;
  HILS_REQUIRE(nblk <= 2147483647L, "hils_rope: grid too large");
  const long tbs = table_per_batch ? (long)L * D : 0;
  if (table_f32)
    hipLaunchKernelGGL(rope_kernel<true>, dim3((unsigned)nblk), dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t*)x, cos_t, sin_t, (bf16_t*)out, total, L, H, D, tbs, lo_only, sin_sign);
  else
    hipLaunchKernelGGL(rope_kernel<false>, dim3((unsigned)nblk), dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t*)x, cos_t, sin_t, (bf16_t*)out, total, L, H, D, tbs, lo_only, sin_sign);
  HILS_CHECK_LAUNCH("hils_rope");
  return HILS_OK;
}
