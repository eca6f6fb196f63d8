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

// ---------------------------------------------------------------------------
// Key (or query) preparation in one pass over the projected tensor: per-head RMS norm, rotary
// embedding, and the mean over each chunk (the chunk keys) - the layer's sequence
//   k = k_norm(k);  k = k*cos + rotate_half(k)*sin;  lmk = k.view(B,N,S,H,D).mean(2)
// which otherwise reads and writes the (B,L,H,D) tensor once per step.  Roundings follow that
// sequence on bf16 tensors: the normalised value is rounded to bf16 before the weight multiplies it,
// each product and the sum of the rotation are rounded to bf16, and the mean is taken over the
// rounded outputs (fp32 sum, one rounding).  One wavefront owns one (batch, chunk, head): D/8
// neighbouring lanes hold a token row, so the row reductions and the exchange between the two
// halves of a head vector stay inside a group of lanes.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float np_round_bf16(float x) { return bf2f(f2bf(x)); }

template <int LPR>  // lanes per token row = D / 8
__global__ void __launch_bounds__(256)
norm_rope_pool_fwd_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                          const bf16_t* __restrict__ cos_t, const bf16_t* __restrict__ sin_t,
                          bf16_t* __restrict__ out, bf16_t* __restrict__ lmk, int B, int L, int H, int S,
                          int nchunk_all, int nchunk_full, long tab_batch_stride, float eps) {
  constexpr int D = LPR * 8, RPI = 64 / LPR;  // token rows per wavefront and step
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long unit = (long)blockIdx.x * 4 + wave;  // (b * nchunk_all + n) * H + h
  if (unit >= (long)B * nchunk_all * H) return;
  const int h = (int)(unit % H);
  const long bn = unit / H;
  const int n = (int)(bn % nchunk_all);
  const long b = bn / nchunk_all;
  const int p = lane % LPR, rl = lane / LPR;
  float wv[8];
  if (w) unpack8(*(const uint4*)(w + p * 8), wv);
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  for (int tok = rl; tok < S; tok += RPI) {  // uniform trip count over the lanes of a row
    const long t = (long)n * S + tok;
    const bool ok = t < L;
    float f[8];
    if (ok) unpack8(*(const uint4*)(x + ((b * L + t) * H + h) * (long)D + p * 8), f);
    else {
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = 0.f;
    }
    if (w) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(f[e], f[e], ss);
#pragma unroll
      for (int o2 = 1; o2 < LPR; o2 <<= 1) ss += __shfl_xor(ss, o2, 64);
      const float r = rsqrtf(ss * (1.f / D) + eps);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = np_round_bf16(wv[e] * np_round_bf16(f[e] * r));
    }
    if (cos_t) {
      float c[8], s[8];
      const long to = b * tab_batch_stride + (ok ? t : 0) * D + p * 8;
      unpack8(*(const uint4*)(cos_t + to), c);
      unpack8(*(const uint4*)(sin_t + to), s);
      const float sign = p < LPR / 2 ? -1.f : 1.f;  // rotate_half: (-x_hi, x_lo)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float other = __shfl_xor(f[e], LPR / 2, 64);
        f[e] = np_round_bf16(np_round_bf16(f[e] * c[e]) + np_round_bf16(sign * other * s[e]));
      }
    }
    if (ok) {
      uint4 o;
      o.x = pack_bf2(f[0], f[1]); o.y = pack_bf2(f[2], f[3]); o.z = pack_bf2(f[4], f[5]); o.w = pack_bf2(f[6], f[7]);
      *(uint4*)(out + ((b * L + t) * H + h) * (long)D + p * 8) = o;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += f[e];
    }
  }
  if (lmk && n < nchunk_full) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int o2 = LPR; o2 < 64; o2 <<= 1) acc[e] += __shfl_xor(acc[e], o2, 64);
    if (rl == 0) {
      const float inv = 1.f / (float)S;
      uint4 o;
      o.x = pack_bf2(acc[0] * inv, acc[1] * inv); o.y = pack_bf2(acc[2] * inv, acc[3] * inv);
      o.z = pack_bf2(acc[4] * inv, acc[5] * inv); o.w = pack_bf2(acc[6] * inv, acc[7] * inv);
      *(uint4*)(lmk + ((b * nchunk_full + n) * H + h) * (long)D + p * 8) = o;
    }
  }
}

// Backward of the pass above.  g = d_out + d_lmk / S (either may be absent); through the rotation:
// gz = g*cos + rotate_half^T(g*sin); through the weight: d_w += gz * y, gy = gz * w; through the
// norm (y = x r, r = (mean x^2 + eps)^-1/2): dx = r (gy - y mean(gy y)).  d_w (D floats, fp32) is
// added to with one atomic per wavefront and feature.
template <int LPR>
__global__ void __launch_bounds__(256)
norm_rope_pool_bwd_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                          const bf16_t* __restrict__ cos_t, const bf16_t* __restrict__ sin_t,
                          const bf16_t* __restrict__ g_out, const bf16_t* __restrict__ g_lmk,
                          bf16_t* __restrict__ dx, float* __restrict__ dw, int B, int L, int H, int S,
                          int nchunk_all, int nchunk_full, long tab_batch_stride, float eps) {
  constexpr int D = LPR * 8, RPI = 64 / LPR;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long unit = (long)blockIdx.x * 4 + wave;
  if (unit >= (long)B * nchunk_all * H) return;
  const int h = (int)(unit % H);
  const long bn = unit / H;
  const int n = (int)(bn % nchunk_all);
  const long b = bn / nchunk_all;
  const int p = lane % LPR, rl = lane / LPR;
  float wv[8], gl[8], wacc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) { wv[e] = 1.f; gl[e] = 0.f; wacc[e] = 0.f; }
  if (w) unpack8(*(const uint4*)(w + p * 8), wv);
  if (g_lmk && n < nchunk_full) {
    unpack8(*(const uint4*)(g_lmk + ((b * nchunk_full + n) * H + h) * (long)D + p * 8), gl);
    const float inv = 1.f / (float)S;
#pragma unroll
    for (int e = 0; e < 8; ++e) gl[e] *= inv;
  }
  for (int tok = rl; tok < S; tok += RPI) {
    const long t = (long)n * S + tok;
    const bool ok = t < L;
    const long xo = ((b * L + (ok ? t : 0)) * H + h) * (long)D + p * 8;
    float f[8], g[8];
    unpack8(*(const uint4*)(x + xo), f);
    if (g_out) unpack8(*(const uint4*)(g_out + xo), g);
    else {
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = 0.f;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) g[e] = ok ? g[e] + gl[e] : 0.f;
    if (cos_t) {
      float c[8], s[8];
      const long to = b * tab_batch_stride + (ok ? t : 0) * D + p * 8;
      unpack8(*(const uint4*)(cos_t + to), c);
      unpack8(*(const uint4*)(sin_t + to), s);
      const float sign = p < LPR / 2 ? 1.f : -1.f;  // transpose of rotate_half: (u_hi, -u_lo)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float u = g[e] * s[e];
        const float other = __shfl_xor(u, LPR / 2, 64);
        g[e] = fmaf(g[e], c[e], sign * other);
      }
    }
    if (w) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(f[e], f[e], ss);
#pragma unroll
      for (int o2 = 1; o2 < LPR; o2 <<= 1) ss += __shfl_xor(ss, o2, 64);
      const float r = rsqrtf(ss * (1.f / D) + eps);
      float dot = 0.f, y[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        y[e] = f[e] * r;
        wacc[e] = fmaf(g[e], np_round_bf16(y[e]), wacc[e]);
        g[e] *= wv[e];
        dot = fmaf(g[e], y[e], dot);
      }
#pragma unroll
      for (int o2 = 1; o2 < LPR; o2 <<= 1) dot += __shfl_xor(dot, o2, 64);
      dot *= 1.f / D;
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = r * (g[e] - y[e] * dot);
    }
    if (ok) {
      uint4 o;
      o.x = pack_bf2(g[0], g[1]); o.y = pack_bf2(g[2], g[3]); o.z = pack_bf2(g[4], g[5]); o.w = pack_bf2(g[6], g[7]);
      *(uint4*)(dx + xo) = o;
    }
  }
  if (w && dw) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int o2 = LPR; o2 < 64; o2 <<= 1) wacc[e] += __shfl_xor(wacc[e], o2, 64);
    if (rl == 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (wacc[e] != 0.f) unsafeAtomicAdd(dw + p * 8 + e, wacc[e]);
    }
  }
}

static int np_check(const char* who, const void* x, const void* cos_t, const void* sin_t, int B, int L, int H,
                    int D, int S) {
  HILS_REQUIRE(x, "%s: null pointer", who);
  HILS_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "%s: cos and sin come together", who);
  HILS_REQUIRE(B > 0 && L > 0 && H > 0 && S > 0, "%s: sizes must be positive", who);
  HILS_REQUIRE(D == 64 || D == 128 || D == 256, "%s: head dim %d not supported (64, 128 or 256)", who, D);
  HILS_REQUIRE(((long)B * ((L + S - 1) / S) * H + 3) / 4 <= 2147483647L, "%s: grid too large", who);
  return HILS_OK;
}

extern "C" int hils_norm_rope_pool_fwd(const void* x, const void* norm_weight, const void* cos_t,
                                       const void* sin_t, void* out, void* lmk, int B, int L, int H, int D,
                                       int S, int table_per_batch, float eps, void* stream) {
  if (int rc = np_check("hils_norm_rope_pool_fwd", x, cos_t, sin_t, B, L, H, D, S)) return rc;
  HILS_REQUIRE(out, "hils_norm_rope_pool_fwd: null output");
  const int nall = (L + S - 1) / S, nfull = L / S;
  const long units = (long)B * nall * H;
  const dim3 grid((unsigned)((units + 3) / 4));
  const long tbs = table_per_batch ? (long)L * D : 0;
#define NP_FWD(LPR_)                                                                                      \
  hipLaunchKernelGGL(norm_rope_pool_fwd_kernel<LPR_>, grid, dim3(256), 0, (hipStream_t)stream,            \
                     (const bf16_t*)x, (const bf16_t*)norm_weight, (const bf16_t*)cos_t, (const bf16_t*)sin_t, \
                     (bf16_t*)out, (bf16_t*)lmk, B, L, H, S, nall, nfull, tbs, eps)
  if (D == 64) NP_FWD(8); else if (D == 128) NP_FWD(16); else NP_FWD(32);
#undef NP_FWD
  HILS_CHECK_LAUNCH("hils_norm_rope_pool_fwd");
  return HILS_OK;
}

extern "C" int hils_norm_rope_pool_bwd(const void* x, const void* norm_weight, const void* cos_t,
                                       const void* sin_t, const void* d_out, const void* d_lmk, void* dx,
                                       float* d_weight, int B, int L, int H, int D, int S,
                                       int table_per_batch, float eps, void* stream) {
  if (int rc = np_check("hils_norm_rope_pool_bwd", x, cos_t, sin_t, B, L, H, D, S)) return rc;
  HILS_REQUIRE(dx && (d_out || d_lmk), "hils_norm_rope_pool_bwd: null pointer");
  HILS_REQUIRE(!norm_weight || d_weight, "hils_norm_rope_pool_bwd: the norm weight needs d_weight");
  const int nall = (L + S - 1) / S, nfull = L / S;
  const long units = (long)B * nall * H;
  const dim3 grid((unsigned)((units + 3) / 4));
  const long tbs = table_per_batch ? (long)L * D : 0;
#define NP_BWD(LPR_)                                                                                      \
  hipLaunchKernelGGL(norm_rope_pool_bwd_kernel<LPR_>, grid, dim3(256), 0, (hipStream_t)stream,            \
                     (const bf16_t*)x, (const bf16_t*)norm_weight, (const bf16_t*)cos_t, (const bf16_t*)sin_t, \
                     (const bf16_t*)d_out, (const bf16_t*)d_lmk, (bf16_t*)dx, d_weight, B, L, H, S, nall,  \
                     nfull, tbs, eps)
  if (D == 64) NP_BWD(8); else if (D == 128) NP_BWD(16); else NP_BWD(32);
#undef NP_BWD
  HILS_CHECK_LAUNCH("hils_norm_rope_pool_bwd");
  return HILS_OK;
}
