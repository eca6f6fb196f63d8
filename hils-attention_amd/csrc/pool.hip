// Chunk-key pooling kernels (HBM-bandwidth-bound reductions over 64-token chunks).
#include "decode_rows.h"
#include "../../include/hils_amd.h"

// ---------------------------------------------------------------------------
// mean pool
// ---------------------------------------------------------------------------
// One block per (chunk = blockIdx.x, column group = blockIdx.y).  blockDim = (CG, TS): CG lanes
// cover contiguous 16-byte column groups of the flattened (H*D) row, TS token slices
// each own S/TS tokens; the slices are summed through LDS in a fixed order.
template <int TS>
__global__ void mean_pool_fwd_kernel(const uint4* __restrict__ k, uint4* __restrict__ out,
                                     int S, int cols8, float inv_s) {
  extern __shared__ float smem[];  // TS * CG * 8 floats
  const int cg = blockIdx.y * blockDim.x + threadIdx.x;
  const int ts = threadIdx.y;
  const long chunk = blockIdx.x;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (cg < cols8) {
    const uint4* base = k + (chunk * S) * (long)cols8 + cg;
    // four of the slice's rows in flight per lane (one load at a time left the kernel waiting a
    // memory latency per row); rows past the chunk re-read its last row and add nothing
    for (int s0 = ts; s0 < S; s0 += 4 * TS) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int s = s0 + u * TS;
        v[u] = base[(long)(s < S ? s : S - 1) * cols8];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        float f[8];
        unpack8(v[u], f);
        const float on = s0 + u * TS < S ? 1.f : 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = fmaf(f[i], on, acc[i]);
      }
    }
  }
  float* mine = smem + ((size_t)ts * blockDim.x + threadIdx.x) * 8;
#pragma unroll
  for (int i = 0; i < 8; ++i) mine[i] = acc[i];
  __syncthreads();
  if (ts == 0 && cg < cols8) {
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = 0.f;
    for (int t = 0; t < TS; ++t) {
      const float* o = smem + ((size_t)t * blockDim.x + threadIdx.x) * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) r[i] += o[i];
    }
    uint4 w;
    w.x = pack_bf2(r[0] * inv_s, r[1] * inv_s);
    w.y = pack_bf2(r[2] * inv_s, r[3] * inv_s);
    w.z = pack_bf2(r[4] * inv_s, r[5] * inv_s);
    w.w = pack_bf2(r[6] * inv_s, r[7] * inv_s);
    out[chunk * cols8 + cg] = w;
  }
}

__global__ void mean_pool_bwd_kernel(const uint4* __restrict__ g, uint4* __restrict__ dk,
                                     int S, int cols8, float inv_s, long total8) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const long row = i / cols8;  // token row over (B*L)
  const int cg = (int)(i - row * cols8);
  const long chunk = row / S;
  uint4 v = g[chunk * cols8 + cg];
  float f[8];
  unpack8(v, f);
  uint4 w;
  w.x = pack_bf2(f[0] * inv_s, f[1] * inv_s);
  w.y = pack_bf2(f[2] * inv_s, f[3] * inv_s);
  w.z = pack_bf2(f[4] * inv_s, f[5] * inv_s);
  w.w = pack_bf2(f[6] * inv_s, f[7] * inv_s);
  dk[i] = w;
}

extern "C" int hils_mean_pool_fwd(const void* k, void* lmk_k, int B, int L, int H, int D, int S,
                                  void* stream) {
  HILS_REQUIRE(k && lmk_k, "hils_mean_pool_fwd: null pointer");
  HILS_REQUIRE(B > 0 && L > 0 && H > 0 && D > 0 && S > 0, "hils_mean_pool_fwd: sizes must be positive");
  HILS_REQUIRE(L % S == 0, "hils_mean_pool_fwd: L (%d) must be a multiple of S (%d)", L, S);
  HILS_REQUIRE((H * D) % 8 == 0, "hils_mean_pool_fwd: H*D (%d) must be a multiple of 8", H * D);
  const int cols8 = H * D / 8;
  const long chunks = (long)B * (L / S);
  constexpr int TS = 8;
  const int CG = cols8 >= 32 ? 32 : cols8;
  dim3 block(CG, TS);
  HILS_REQUIRE(chunks <= 2147483647L && (cols8 + CG - 1) / CG <= 65535, "hils_mean_pool_fwd: grid too large");
  dim3 grid((unsigned)chunks, (cols8 + CG - 1) / CG);
  size_t smem = (size_t)TS * CG * 8 * sizeof(float);
  hipLaunchKernelGGL(mean_pool_fwd_kernel<TS>, grid, block, smem, (hipStream_t)stream,
                     (const uint4*)k, (uint4*)lmk_k, S, cols8, 1.0f / (float)S);
  HILS_CHECK_LAUNCH("hils_mean_pool_fwd");
  return HILS_OK;
}

extern "C" int hils_mean_pool_bwd(const void* g_lmk, void* dk, int B, int L, int H, int D, int S,
                                  void* stream) {
  HILS_REQUIRE(g_lmk && dk, "hils_mean_pool_bwd: null pointer");
  HILS_REQUIRE(B > 0 && L > 0 && H > 0 && D > 0 && S > 0, "hils_mean_pool_bwd: sizes must be positive");
  HILS_REQUIRE(L % S == 0, "hils_mean_pool_bwd: L (%d) must be a multiple of S (%d)", L, S);
  HILS_REQUIRE((H * D) % 8 == 0, "hils_mean_pool_bwd: H*D (%d) must be a multiple of 8", H * D);
  const int cols8 = H * D / 8;
  const long total8 = (long)B * L * cols8;
  const long nblk = (total8 + 255) / 256;
  HILS_REQUIRE(nblk <= 2147483647L, "hils_mean_pool_bwd: grid too large");
  hipLaunchKernelGGL(mean_pool_bwd_kernel, dim3((unsigned)nblk), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)g_lmk, (uint4*)dk, S, cols8, 1.0f / (float)S, total8);
  HILS_CHECK_LAUNCH("hils_mean_pool_bwd");
  return HILS_OK;
}

// ---------------------------------------------------------------------------
// attention pool: one prior query per (chunk, head) over the chunk's first S-1 keys
// ---------------------------------------------------------------------------
// One block of 256 threads per (chunk bn, head h).  The K tile (S x D, bf16) is staged
// in LDS as fp32 with a padded row so that both the row-wise dot products and the
// column-wise weighted sums are bank-conflict free.
#define POOL_THREADS 256

__global__ void __launch_bounds__(POOL_THREADS)
attn_pool_fwd_kernel(const bf16_t* __restrict__ mu_q, const bf16_t* __restrict__ k,
                     bf16_t* __restrict__ lmk_k, float* __restrict__ lmk_b, float* __restrict__ p_out,
                     int S, int H, int HK, int D, float sm_scale, int compact, int shared_k) {
  extern __shared__ float smem[];
  const int DP = D + 1;
  float* ks = smem;              // S * DP
  float* mu = ks + (size_t)S * DP;  // D
  float* pr = mu + D;            // S
  float* red = pr + S;           // 32
  const long bn = blockIdx.x;
  const int h = blockIdx.y;
  const int kh = shared_k ? 0 : h / (H / HK);  // K has HK heads: H / HK query heads read each
  const int tid = threadIdx.x;

  const int d8 = D / 8;
  for (int i = tid; i < S * d8; i += POOL_THREADS) {
    const int s = i / d8, c = i - s * d8;
    uint4 v = *(const uint4*)(k + ((bn * S + s) * (long)HK + kh) * D + c * 8);
    float f[8];
    unpack8(v, f);
#pragma unroll
    for (int j = 0; j < 8; ++j) ks[s * DP + c * 8 + j] = f[j];
  }
  for (int d = tid; d < D; d += POOL_THREADS) mu[d] = bf2f(mu_q[(bn * H + h) * (long)D + d]);
  __syncthreads();

  // logits, one thread per token
  for (int s = tid; s < S; s += POOL_THREADS) {
    float a = 0.f;
    for (int d = 0; d < D; ++d) a += mu[d] * ks[s * DP + d];
    a *= sm_scale;
    if (s == S - 1) a = HILS_NEG_INF;
    pr[s] = a;
  }
  __syncthreads();
  float m = HILS_NEG_INF;
  for (int s = tid; s < S; s += POOL_THREADS) m = fmaxf(m, pr[s]);
  m = block_max(m, red);
  float e_sum = 0.f;
  for (int s = tid; s < S; s += POOL_THREADS) {
    float e = (pr[s] == HILS_NEG_INF) ? 0.f : expf(pr[s] - m);
    pr[s] = e;
    e_sum += e;
  }
  e_sum = block_sum(e_sum, red);
  const float inv = e_sum > 0.f ? 1.f / e_sum : 0.f;
  float ent = 0.f;
  for (int s = tid; s < S; s += POOL_THREADS) {
    const float pv = pr[s] * inv;
    pr[s] = pv;
    p_out[(bn * S + s) * (long)H + h] = pv;
    if (pv > 0.f) ent += pv * logf(pv);
  }
  ent = block_sum(ent, red);  // also orders the pr[] writes before the reads below
  if (tid == 0) lmk_b[bn * H + h] = -ent;
  for (int d = tid; d < D; d += POOL_THREADS) {
    float a = 0.f;
    if (!compact)
      for (int s = 0; s < S; ++s) a += pr[s] * ks[s * DP + d];
    lmk_k[(bn * H + h) * (long)D + d] = f2bf(a);
  }
}

// Row-streaming variant for 64-token chunks and D = 64 / 128: one wavefront per (chunk, head), the
// K tile is read once with coalesced 16-byte lane loads (LR = D/8 lanes per token row, 64/LR rows
// per instruction) and stays in registers; logits by packed bf16 dot2 + DPP row reduction, the
// softmax over tokens and the weighted sum by in-lane loops plus a reduction over the lanes that
// hold the same 8 columns of different rows.  The four wavefronts of a workgroup take four
// neighbouring heads, i.e. neighbouring 2*D-byte pieces of the same token rows.
template <int LR>
__device__ __forceinline__ float pool_groups_max(float x) {  // over lanes with the same lane % LR
  if (LR == 8) x = fmaxf(x, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(x), __float_as_int(x), 0x128, 0xF, 0xF, false)));
  return rows_max(x);
}
template <int LR>
__device__ __forceinline__ float pool_groups_sum(float x) {
  if (LR == 8) x += __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(x), __float_as_int(x), 0x128, 0xF, 0xF, false));
  return rows_sum(x);
}

template <int D>
__global__ void __launch_bounds__(256)
attn_pool_fwd_rows(const bf16_t* __restrict__ mu_q, const bf16_t* __restrict__ k,
                   bf16_t* __restrict__ lmk_k, float* __restrict__ lmk_b, float* __restrict__ p_out,
                   int H, float sm_scale, int compact, int shared_k) {
  constexpr int S = 64, LR = D / 8, TPI = 64 / LR, NI = S / TPI;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int piece = lane % LR, tsub = lane / LR;
  const int hgroups = (H + 3) / 4;  // neighbouring workgroups: neighbouring heads of one chunk
  const long bn = blockIdx.x / hgroups;
  const int h = (int)(blockIdx.x % hgroups) * 4 + wave;
  if (h >= H) return;
  const int kh = shared_k ? 0 : h;
  const bf16_t* kp = k + ((bn * S + tsub) * (long)H + kh) * D + piece * 8;
  const long step = (long)TPI * H * D;
  uint4 kr[NI];
#pragma unroll
  for (int it = 0; it < NI; ++it) kr[it] = *(const uint4*)(kp + it * step);
  const uint4 mq = *(const uint4*)(mu_q + (bn * H + h) * (long)D + piece * 8);
  float a[NI];
  float m = HILS_NEG_INF;
#pragma unroll
  for (int it = 0; it < NI; ++it) {
    a[it] = row_sum<LR>(dot8_bf16(mq, kr[it], 0.f)) * sm_scale;
    if (it == NI - 1 && tsub == TPI - 1) a[it] = HILS_NEG_INF;  // the chunk's last token is never pooled
    m = fmaxf(m, a[it]);
  }
  m = pool_groups_max<LR>(m);
  float e_sum = 0.f;
#pragma unroll
  for (int it = 0; it < NI; ++it) {
    a[it] = (a[it] == HILS_NEG_INF) ? 0.f : __expf(a[it] - m);
    e_sum += a[it];
  }
  e_sum = pool_groups_sum<LR>(e_sum);
  const float inv = e_sum > 0.f ? 1.f / e_sum : 0.f;
  float ent = 0.f;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int it = 0; it < NI; ++it) {
    const float pv = a[it] * inv;
    if (piece == 0) p_out[(bn * S + it * TPI + tsub) * (long)H + h] = pv;
    if (pv > 0.f) ent += pv * __logf(pv);
    float f[8];
    unpack8(kr[it], f);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = fmaf(pv, f[i], acc[i]);
  }
  ent = pool_groups_sum<LR>(ent);
  if (lane == 0) lmk_b[bn * H + h] = -ent;
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = compact ? 0.f : pool_groups_sum<LR>(acc[i]);
  if (tsub == 0) {
    uint4 w;
    w.x = pack_bf2(acc[0], acc[1]);
    w.y = pack_bf2(acc[2], acc[3]);
    w.z = pack_bf2(acc[4], acc[5]);
    w.w = pack_bf2(acc[6], acc[7]);
    *(uint4*)(lmk_k + (bn * H + h) * (long)D + piece * 8) = w;
  }
}

// Row-streaming backward, same lane layout.  Per (chunk, head):
//   dP_s = <g_k, K_s>,  delta = sum_s p_s dP_s,  dl_s = p_s (dP_s - delta - g_b (log p_s + H)),
//   d_mu = scale * sum_s dl_s K_s,  dK_s = scale * dl_s * mu + p_s * g_k.
// SHARED: K is head 0's tile for every head; a workgroup owns a chunk, its wavefronts walk the
// heads h = wave, wave + 4, ... with the dK sum in registers, the four sums meet in LDS (two
// rounds), head 0 receives the total and heads 1..H-1 are zeroed.
template <int D, bool SHARED>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
attn_pool_bwd_rows(const bf16_t* __restrict__ mu_q, const bf16_t* __restrict__ k,
                   const float* __restrict__ p_saved, const float* __restrict__ lmk_b,
                   const bf16_t* __restrict__ g_k, const float* __restrict__ g_b,
                   bf16_t* __restrict__ d_mu, bf16_t* __restrict__ d_k, int H, float sm_scale,
                   int compact) {
  constexpr int S = 64, LR = D / 8, TPI = 64 / LR, NI = S / TPI;
  extern __shared__ float xch[];  // SHARED: 2 * NI * 8 * 64 floats
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int piece = lane % LR, tsub = lane / LR;
  const int hgroups = SHARED ? 1 : (H + 3) / 4;
  const long bn = blockIdx.x / hgroups;
  const int h_first = SHARED ? wave : (int)(blockIdx.x % hgroups) * 4 + wave;
  const int h_step = SHARED ? 4 : H;  // not SHARED: a single head
  const int kh = SHARED ? 0 : h_first;
  uint4 kr[NI];
  if (SHARED || h_first < H) {
    const bf16_t* kp = k + ((bn * S + tsub) * (long)H + kh) * D + piece * 8;
    const long step = (long)TPI * H * D;
#pragma unroll
    for (int it = 0; it < NI; ++it) kr[it] = *(const uint4*)(kp + it * step);
  }
  float dk_acc[SHARED ? NI : 1][8];
  if (SHARED) {
#pragma unroll
    for (int it = 0; it < NI; ++it)
#pragma unroll
      for (int i = 0; i < 8; ++i) dk_acc[it][i] = 0.f;
  }
  for (int h = h_first; h < H; h += h_step) {
    const uint4 mq = *(const uint4*)(mu_q + (bn * H + h) * (long)D + piece * 8);
    uint4 gq = make_uint4(0, 0, 0, 0);
    if (!compact) gq = *(const uint4*)(g_k + (bn * H + h) * (long)D + piece * 8);
    const float ent = lmk_b[bn * H + h], gb = g_b[bn * H + h];
    float pv[NI], dl[NI];
    float part = 0.f;
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      pv[it] = p_saved[(bn * S + it * TPI + tsub) * (long)H + h];
      dl[it] = row_sum<LR>(dot8_bf16(gq, kr[it], 0.f));
      part += pv[it] * dl[it];
    }
    const float delta = pool_groups_sum<LR>(part);
    float muf[8], gkf[8];
    unpack8(mq, muf);
    unpack8(gq, gkf);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const float x = pv[it] > 0.f ? pv[it] * ((dl[it] - delta) - gb * (__logf(pv[it]) + ent)) : 0.f;
      float f[8];
      unpack8(kr[it], f);
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        acc[i] = fmaf(x, f[i], acc[i]);
        o[i] = sm_scale * x * muf[i] + pv[it] * gkf[i];
      }
      if (SHARED) {
#pragma unroll
        for (int i = 0; i < 8; ++i) dk_acc[it][i] += o[i];
      } else {
        uint4 w;
        w.x = pack_bf2(o[0], o[1]); w.y = pack_bf2(o[2], o[3]);
        w.z = pack_bf2(o[4], o[5]); w.w = pack_bf2(o[6], o[7]);
        *(uint4*)(d_k + ((bn * S + it * TPI + tsub) * (long)H + h) * D + piece * 8) = w;
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = pool_groups_sum<LR>(acc[i]) * sm_scale;
    if (tsub == 0) {
      uint4 w;
      w.x = pack_bf2(acc[0], acc[1]); w.y = pack_bf2(acc[2], acc[3]);
      w.z = pack_bf2(acc[4], acc[5]); w.w = pack_bf2(acc[6], acc[7]);
      *(uint4*)(d_mu + (bn * H + h) * (long)D + piece * 8) = w;
    }
  }
  if (SHARED) {
    // waves 2,3 -> LDS; waves 0,1 add; wave 1 -> LDS; wave 0 adds and writes head 0
    float* slot = xch + (size_t)(wave & 1) * NI * 8 * 64;
    auto put = [&]() {
#pragma unroll
      for (int it = 0; it < NI; ++it)
#pragma unroll
        for (int i = 0; i < 8; ++i) slot[(it * 8 + i) * 64 + lane] = dk_acc[it][i];
    };
    auto add = [&]() {
#pragma unroll
      for (int it = 0; it < NI; ++it)
#pragma unroll
        for (int i = 0; i < 8; ++i) dk_acc[it][i] += slot[(it * 8 + i) * 64 + lane];
    };
    if (wave >= 2) put();
    __syncthreads();
    if (wave < 2) add();
    __syncthreads();
    if (wave == 1) { slot = xch; put(); }
    __syncthreads();
    if (wave == 0) {
      add();
#pragma unroll
      for (int it = 0; it < NI; ++it) {
        uint4 w;
        w.x = pack_bf2(dk_acc[it][0], dk_acc[it][1]); w.y = pack_bf2(dk_acc[it][2], dk_acc[it][3]);
        w.z = pack_bf2(dk_acc[it][4], dk_acc[it][5]); w.w = pack_bf2(dk_acc[it][6], dk_acc[it][7]);
        *(uint4*)(d_k + ((bn * S + it * TPI + tsub) * (long)H) * D + piece * 8) = w;
      }
    }
    // heads 1..H-1 of every token row: (H-1)*D/8 zero pieces per row
    const int zp = (H - 1) * (D / 8);
    for (int i = threadIdx.x; i < S * zp; i += 256) {
      const int srow = i / zp, c = i - srow * zp;
      *(uint4*)(d_k + ((bn * S + srow) * (long)H + 1) * D + (long)c * 8) = make_uint4(0, 0, 0, 0);
    }
  }
}

// Grouped query heads (K with HK = H / G heads, the model's own KV head count): one wavefront per
// (chunk, KV head) keeps that head's K tile in registers and runs its G prior queries over it, so K
// is read once instead of G times and nothing is repeated in memory beforehand.  Same lane layout
// and arithmetic as the per-head kernels above.
template <int D>
__global__ void __launch_bounds__(256)
attn_pool_fwd_rows_gqa(const bf16_t* __restrict__ mu_q, const bf16_t* __restrict__ k,
                       bf16_t* __restrict__ lmk_k, float* __restrict__ lmk_b, float* __restrict__ p_out,
                       int H, int HK, float sm_scale, int compact) {
  constexpr int S = 64, LR = D / 8, TPI = 64 / LR, NI = S / TPI;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int piece = lane % LR, tsub = lane / LR;
  const int hgroups = (HK + 3) / 4;
  const long bn = blockIdx.x / hgroups;
  const int kh = (int)(blockIdx.x % hgroups) * 4 + wave;
  if (kh >= HK) return;
  const int G = H / HK;
  const bf16_t* kp = k + ((bn * S + tsub) * (long)HK + kh) * D + piece * 8;
  const long step = (long)TPI * HK * D;
  uint4 kr[NI];
#pragma unroll
  for (int it = 0; it < NI; ++it) kr[it] = *(const uint4*)(kp + it * step);
  for (int g = 0; g < G; ++g) {
    const int h = kh * G + g;
    const uint4 mq = *(const uint4*)(mu_q + (bn * H + h) * (long)D + piece * 8);
    float a[NI];
    float m = HILS_NEG_INF;
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      a[it] = row_sum<LR>(dot8_bf16(mq, kr[it], 0.f)) * sm_scale;
      if (it == NI - 1 && tsub == TPI - 1) a[it] = HILS_NEG_INF;  // the chunk's last token is never pooled
      m = fmaxf(m, a[it]);
    }
    m = pool_groups_max<LR>(m);
    float e_sum = 0.f;
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      a[it] = (a[it] == HILS_NEG_INF) ? 0.f : __expf(a[it] - m);
      e_sum += a[it];
    }
    e_sum = pool_groups_sum<LR>(e_sum);
    const float inv = e_sum > 0.f ? 1.f / e_sum : 0.f;
    float ent = 0.f;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const float pv = a[it] * inv;
      if (piece == 0) p_out[(bn * S + it * TPI + tsub) * (long)H + h] = pv;
      if (pv > 0.f) ent += pv * __logf(pv);
      float f[8];
      unpack8(kr[it], f);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(pv, f[i], acc[i]);
    }
    ent = pool_groups_sum<LR>(ent);
    if (lane == 0) lmk_b[bn * H + h] = -ent;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = compact ? 0.f : pool_groups_sum<LR>(acc[i]);
    if (tsub == 0) {
      uint4 w;
      w.x = pack_bf2(acc[0], acc[1]);
      w.y = pack_bf2(acc[2], acc[3]);
      w.z = pack_bf2(acc[4], acc[5]);
      w.w = pack_bf2(acc[6], acc[7]);
      *(uint4*)(lmk_k + (bn * H + h) * (long)D + piece * 8) = w;
    }
  }
}

// The same forward with the logits on the matrix cores, for G <= 16.  A wavefront takes a (chunk, KV
// head) tile; its K (read once, coalesced, into registers for the weighted sum) is also laid in
// the wavefront's LDS and read back as the A operand of S^T = K mu^T (tokens x heads, the G heads
// padded to 16 columns); a lane then holds 16 tokens of one head's column, so the softmax of all
// heads runs at once, and P goes back through LDS (over the K tile, no longer needed there) to the
// lanes that hold the token rows.  The vector ALU is left with the weighted sum.
// (Tried and slower at 512 chunks x 8 KV heads, D = 128, where this takes 22.5 us: K read straight into
// A-operand order instead of through LDS, 24.6 us; wavefronts that walk two tiles and touch the next
// tile's lines ahead of the arithmetic, 25.5 us.)
template <int D>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
attn_pool_fwd_gqa_mfma(const bf16_t* __restrict__ mu_q, const bf16_t* __restrict__ k,
                       bf16_t* __restrict__ lmk_k, float* __restrict__ lmk_b, float* __restrict__ p_out,
                       long tiles, int H, int HK, float sm_scale, int compact) {
  constexpr int S = 64, LR = D / 8, TPI = 64 / LR, NI = S / TPI, KS = D / 32;
  constexpr int PITCH = D * 2 + 16;  // bytes of a token row in LDS: 16-byte reads of 16 rows spread over the banks
  static_assert(S * PITCH >= 16 * S * 4, "P of 16 heads fits over the K tile");
  extern __shared__ __align__(16) unsigned char pool_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int piece = lane % LR, tsub = lane / LR;
  const int col = lane & 15, j = lane >> 4;
  const int G = H / HK;
  unsigned char* kl = pool_lds + (size_t)wave * (S * PITCH);
  float* ps = (float*)kl;  // P, [head][token % TPI][token / TPI], once S is formed
  const long step = (long)TPI * HK * D;
  // tile = chunk * HK + KV head: neighbouring wavefronts read neighbouring pieces of the same token rows
  auto load = [&](uint4 (&kr)[NI], long tile) {
    const bf16_t* kp = k + (tile / HK * S + tsub) * (long)HK * D + (tile % HK) * (long)D + piece * 8;
#pragma unroll
    for (int it = 0; it < NI; ++it) kr[it] = *(const uint4*)(kp + it * step);
  };
  auto process = [&](const uint4 (&kr)[NI], long tile) {
    const long bn = tile / HK;
    const int kh = (int)(tile - bn * HK);
    // B operand: column `col` is head kh * G + col (zero past G), lane group j holds k = 8j .. 8j+7 of a step
    bf16x8_t mub[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (col < G) v = *(const uint4*)(mu_q + (bn * H + kh * G + col) * (long)D + ks * 32 + j * 8);
      mub[ks] = *(bf16x8_t*)&v;
    }
#pragma unroll
    for (int it = 0; it < NI; ++it) *(uint4*)(kl + (it * TPI + tsub) * PITCH + piece * 16) = kr[it];
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_wave_barrier();
    f32x4_t st[4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      st[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const uint4 a = *(const uint4*)(kl + (mt * 16 + col) * PITCH + ks * 64 + j * 16);
        st[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&a, mub[ks], st[mt], 0, 0, 0);
      }
    }
    // st[mt][i] = <K[token mt*16 + 4j + i], mu[head col]>: softmax over the tokens of a column
    float m = HILS_NEG_INF;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float x = st[mt][i] * sm_scale;
        if (mt == 3 && i == 3 && j == 3) x = HILS_NEG_INF;  // the chunk's last token is never pooled
        st[mt][i] = x;
        m = fmaxf(m, x);
      }
    m = rows_max(m);
    float e_sum = 0.f;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float e = (st[mt][i] == HILS_NEG_INF) ? 0.f : __expf(st[mt][i] - m);
        st[mt][i] = e;
        e_sum += e;
      }
    e_sum = rows_sum(e_sum);
    const float inv = e_sum > 0.f ? 1.f / e_sum : 0.f;
    const int h = kh * G + col;  // (a head only where col < G)
    float ent = 0.f;
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_wave_barrier();  // every lane's reads of the K tile are issued: P may overwrite it
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = st[mt][i] * inv;
        const int t = mt * 16 + 4 * j + i;
        if (pv > 0.f) ent += pv * __logf(pv);
        ps[col * S + (t % TPI) * NI + t / TPI] = pv;  // columns past G hold the softmax of zeros: finite, unused
      }
    ent = rows_sum(ent);
    if (col < G && j == 0) lmk_b[bn * H + h] = -ent;
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_wave_barrier();
    // the saved P, (chunk, token, head): lane t writes token t's G heads, contiguous in memory (from the
    // accumulator layout it would be 16 stores of 4 bytes per lane)
    {
      float* dst = p_out + (bn * S + lane) * (long)H + kh * G;
      const float* src = ps + (lane % TPI) * NI + lane / TPI;
      if ((G & 3) == 0) {
        for (int g = 0; g < G; g += 4)
          *(float4*)(dst + g) = make_float4(src[g * S], src[(g + 1) * S], src[(g + 2) * S], src[(g + 3) * S]);
      } else {
        for (int g = 0; g < G; ++g) dst[g] = src[g * S];
      }
    }
    // lmk_k = P K, four heads at a time over the token rows in registers
    for (int g0 = 0; g0 < G; g0 += 4) {
      float acc[4][8];
#pragma unroll
      for (int gg = 0; gg < 4; ++gg)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[gg][i] = 0.f;
      if (!compact) {
#pragma unroll
        for (int i4 = 0; i4 < NI; i4 += 4) {
          __builtin_amdgcn_sched_barrier(0);  // (keeps the unpacked rows of later steps out of the registers of this one)
          float4 pq[4];
#pragma unroll
          for (int gg = 0; gg < 4; ++gg) pq[gg] = *(const float4*)(ps + (g0 + gg) * S + tsub * NI + i4);  // g0 + gg < 16
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float f[8];
            unpack8(kr[i4 + e], f);
#pragma unroll
            for (int gg = 0; gg < 4; ++gg) {
              const float pv = e == 0 ? pq[gg].x : (e == 1 ? pq[gg].y : (e == 2 ? pq[gg].z : pq[gg].w));
#pragma unroll
              for (int i = 0; i < 8; ++i) acc[gg][i] = fmaf(pv, f[i], acc[gg][i]);
            }
          }
        }
      }
#pragma unroll
      for (int gg = 0; gg < 4; ++gg) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[gg][i] = pool_groups_sum<LR>(acc[gg][i]);
        if (tsub == 0 && g0 + gg < G) {
          uint4 w;
          w.x = pack_bf2(acc[gg][0], acc[gg][1]);
          w.y = pack_bf2(acc[gg][2], acc[gg][3]);
          w.z = pack_bf2(acc[gg][4], acc[gg][5]);
          w.w = pack_bf2(acc[gg][6], acc[gg][7]);
          *(uint4*)(lmk_k + (bn * H + kh * G + g0 + gg) * (long)D + piece * 8) = w;
        }
      }
    }
  };
  const long tile = (long)blockIdx.x * 4 + wave;
  if (tile >= tiles) return;  // (the wavefronts of a workgroup never synchronise)
  uint4 kr[NI];
  load(kr, tile);
  process(kr, tile);
}

// Its backward: dK of a KV head is the sum over its G query heads, kept in registers (fp32) and
// rounded once.
template <int D>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(D > 64 ? 1 : 2)))
attn_pool_bwd_rows_gqa(const bf16_t* __restrict__ mu_q, const bf16_t* __restrict__ k,
                       const float* __restrict__ p_saved, const float* __restrict__ lmk_b,
                       const bf16_t* __restrict__ g_k, const float* __restrict__ g_b,
                       bf16_t* __restrict__ d_mu, bf16_t* __restrict__ d_k, int H, int HK, float sm_scale,
                       int compact) {
  constexpr int S = 64, LR = D / 8, TPI = 64 / LR, NI = S / TPI;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int piece = lane % LR, tsub = lane / LR;
  const int hgroups = (HK + 3) / 4;
  const long bn = blockIdx.x / hgroups;
  const int kh = (int)(blockIdx.x % hgroups) * 4 + wave;
  if (kh >= HK) return;
  const int G = H / HK;
  const bf16_t* kp = k + ((bn * S + tsub) * (long)HK + kh) * D + piece * 8;
  const long step = (long)TPI * HK * D;
  uint4 kr[NI];
#pragma unroll
  for (int it = 0; it < NI; ++it) kr[it] = *(const uint4*)(kp + it * step);
  float dk_acc[NI][8];
#pragma unroll
  for (int it = 0; it < NI; ++it)
#pragma unroll
    for (int i = 0; i < 8; ++i) dk_acc[it][i] = 0.f;
  for (int g = 0; g < G; ++g) {
    const int h = kh * G + g;
    const uint4 mq = *(const uint4*)(mu_q + (bn * H + h) * (long)D + piece * 8);
    uint4 gq = make_uint4(0, 0, 0, 0);
    if (!compact) gq = *(const uint4*)(g_k + (bn * H + h) * (long)D + piece * 8);
    const float ent = lmk_b[bn * H + h], gb = g_b[bn * H + h];
    float pv[NI], dl[NI];
    float part = 0.f;
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      pv[it] = p_saved[(bn * S + it * TPI + tsub) * (long)H + h];
      dl[it] = row_sum<LR>(dot8_bf16(gq, kr[it], 0.f));
      part += pv[it] * dl[it];
    }
    const float delta = pool_groups_sum<LR>(part);
    float muf[8], gkf[8];
    unpack8(mq, muf);
    unpack8(gq, gkf);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const float x = pv[it] > 0.f ? pv[it] * ((dl[it] - delta) - gb * (__logf(pv[it]) + ent)) : 0.f;
      float f[8];
      unpack8(kr[it], f);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        acc[i] = fmaf(x, f[i], acc[i]);
        dk_acc[it][i] += sm_scale * x * muf[i] + pv[it] * gkf[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = pool_groups_sum<LR>(acc[i]) * sm_scale;
    if (tsub == 0) {
      uint4 w;
      w.x = pack_bf2(acc[0], acc[1]); w.y = pack_bf2(acc[2], acc[3]);
      w.z = pack_bf2(acc[4], acc[5]); w.w = pack_bf2(acc[6], acc[7]);
      *(uint4*)(d_mu + (bn * H + h) * (long)D + piece * 8) = w;
    }
  }
#pragma unroll
  for (int it = 0; it < NI; ++it) {
    uint4 w;
    w.x = pack_bf2(dk_acc[it][0], dk_acc[it][1]); w.y = pack_bf2(dk_acc[it][2], dk_acc[it][3]);
    w.z = pack_bf2(dk_acc[it][4], dk_acc[it][5]); w.w = pack_bf2(dk_acc[it][6], dk_acc[it][7]);
    *(uint4*)(d_k + ((bn * S + it * TPI + tsub) * (long)HK + kh) * D + piece * 8) = w;
  }
}

// Backward.  Block per (bn, h); per bn looping over all heads when K is shared, per (bn, KV head)
// looping over its query heads when K has fewer heads than mu_q, so that the per-head dK can be
// summed without atomics.
__global__ void __launch_bounds__(POOL_THREADS)
attn_pool_bwd_kernel(const bf16_t* __restrict__ mu_q, const bf16_t* __restrict__ k,
                     const float* __restrict__ p_saved, const float* __restrict__ lmk_b,
                     const bf16_t* __restrict__ g_k, const float* __restrict__ g_b,
                     bf16_t* __restrict__ d_mu, bf16_t* __restrict__ d_k,
                     int S, int H, int HK, int D, float sm_scale, int compact, int shared_k) {
  extern __shared__ float smem[];
  const int DP = D + 1;
  float* ks = smem;                 // S * DP
  float* mu = ks + (size_t)S * DP;  // D
  float* gk = mu + D;               // D
  float* pr = gk + D;               // S
  float* dl = pr + S;               // S  (dP, then dlogits)
  float* red = dl + S;              // 32
  float* dk_acc = red + 32;         // S * D, only when several heads share a K tile
  const long bn = blockIdx.x;
  const int tid = threadIdx.x;
  const int d8 = D / 8;
  const int G = H / HK;             // query heads per K head (1 unless K has fewer heads)
  const bool summed = shared_k || G > 1;
  const int h_begin = shared_k ? 0 : blockIdx.y * G;
  const int h_end = shared_k ? H : h_begin + G;
  const int kh = shared_k ? 0 : blockIdx.y;

  if (summed)
    for (int i = tid; i < S * D; i += POOL_THREADS) dk_acc[i] = 0.f;

  for (int h = h_begin; h < h_end; ++h) {
    __syncthreads();
    if (h == h_begin) {
      for (int i = tid; i < S * d8; i += POOL_THREADS) {
        const int s = i / d8, c = i - s * d8;
        uint4 v = *(const uint4*)(k + ((bn * S + s) * (long)HK + kh) * D + c * 8);
        float f[8];
        unpack8(v, f);
#pragma unroll
        for (int j = 0; j < 8; ++j) ks[s * DP + c * 8 + j] = f[j];
      }
    }
    for (int d = tid; d < D; d += POOL_THREADS) {
      mu[d] = bf2f(mu_q[(bn * H + h) * (long)D + d]);
      gk[d] = compact ? 0.f : bf2f(g_k[(bn * H + h) * (long)D + d]);
    }
    for (int s = tid; s < S; s += POOL_THREADS) pr[s] = p_saved[(bn * S + s) * (long)H + h];
    __syncthreads();
    float part = 0.f;
    for (int s = tid; s < S; s += POOL_THREADS) {
      float a = 0.f;
      for (int d = 0; d < D; ++d) a += gk[d] * ks[s * DP + d];
      dl[s] = a;
      part += pr[s] * a;
    }
    const float delta = block_sum(part, red);
    const float ent = lmk_b[bn * H + h];
    const float gb = g_b[bn * H + h];
    for (int s = tid; s < S; s += POOL_THREADS) {
      const float pv = pr[s];
      dl[s] = pv > 0.f ? pv * ((dl[s] - delta) - gb * (logf(pv) + ent)) : 0.f;
    }
    __syncthreads();
    for (int d = tid; d < D; d += POOL_THREADS) {
      float a = 0.f;
      for (int s = 0; s < S; ++s) a += dl[s] * ks[s * DP + d];
      d_mu[(bn * H + h) * (long)D + d] = f2bf(a * sm_scale);
    }
    if (summed) {
      for (int i = tid; i < S * D; i += POOL_THREADS) {
        const int s = i / D, d = i - s * D;
        dk_acc[i] += sm_scale * dl[s] * mu[d] + pr[s] * gk[d];
      }
    } else {
      for (int i = tid; i < S * D; i += POOL_THREADS) {
        const int s = i / D, d = i - s * D;
        d_k[((bn * S + s) * (long)H + h) * D + d] = f2bf(sm_scale * dl[s] * mu[d] + pr[s] * gk[d]);
      }
    }
  }
  if (summed) {
    __syncthreads();
    for (int i = tid; i < S * D; i += POOL_THREADS) {
      const int s = i / D, d = i - s * D;
      d_k[((bn * S + s) * (long)HK + kh) * D + d] = f2bf(dk_acc[i]);
    }
  }
  if (shared_k) {
    for (long i = tid; i < (long)S * (H - 1) * D; i += POOL_THREADS) {
      const int s = (int)(i / ((long)(H - 1) * D));
      const long r = i - (long)s * (H - 1) * D;
      d_k[((bn * S + s) * (long)H + 1) * D + r] = 0;
    }
  }
}

static int pool_check(const char* name, int BN, int S, int H, int HK, int D, int shared_k) {
  HILS_REQUIRE(BN > 0 && S > 1 && H > 0 && D > 0, "%s: sizes must be positive (S > 1)", name);
  HILS_REQUIRE(D % 8 == 0, "%s: D (%d) must be a multiple of 8", name, D);
  HILS_REQUIRE(H <= 65535, "%s: H (%d) too large", name, H);
  HILS_REQUIRE(HK > 0 && H % HK == 0, "%s: the heads of mu_q (%d) must be a multiple of the heads of k (%d)", name, H, HK);
  HILS_REQUIRE(!shared_k || HK == H, "%s: shared_k reads head 0 of a k with as many heads as mu_q (%d), got %d", name,
               H, HK);
  return HILS_OK;
}

extern "C" int hils_attn_pool_fwd(const void* mu_q, const void* k, void* lmk_k, float* lmk_b,
                                  float* p, int BN, int S, int H, int h_kv, int D, float sm_scale,
                                  int compact, int shared_k, void* stream) {
  HILS_REQUIRE(mu_q && k && lmk_k && lmk_b && p, "hils_attn_pool_fwd: null pointer");
  if (int rc = pool_check("hils_attn_pool_fwd", BN, S, H, h_kv, D, shared_k)) return rc;
  const int HK = h_kv;
  if (S == 64 && (D == 64 || D == 128) && HK < H && H / HK <= 16) {
    const long tiles = (long)BN * HK;
    const long nblk = (tiles + 3) / 4;
    HILS_REQUIRE(nblk <= 2147483647L, "hils_attn_pool_fwd: grid too large");
    const dim3 grid((unsigned)nblk);
    const size_t smem = (size_t)4 * S * (D * 2 + 16);  // a padded K tile per wavefront
    if (D == 64) {
      static HilsLdsReserve reserved;
      if (int rc = hils_reserve_lds(&reserved, (const void*)attn_pool_fwd_gqa_mfma<64>, smem, "hils_attn_pool_fwd")) return rc;
      hipLaunchKernelGGL(attn_pool_fwd_gqa_mfma<64>, grid, dim3(256), smem, (hipStream_t)stream,
                         (const bf16_t*)mu_q, (const bf16_t*)k, (bf16_t*)lmk_k, lmk_b, p, tiles, H, HK, sm_scale, compact);
    } else {
      static HilsLdsReserve reserved;
      if (int rc = hils_reserve_lds(&reserved, (const void*)attn_pool_fwd_gqa_mfma<128>, smem, "hils_attn_pool_fwd")) return rc;
      hipLaunchKernelGGL(attn_pool_fwd_gqa_mfma<128>, grid, dim3(256), smem, (hipStream_t)stream,
                         (const bf16_t*)mu_q, (const bf16_t*)k, (bf16_t*)lmk_k, lmk_b, p, tiles, H, HK, sm_scale, compact);
    }
    HILS_CHECK_LAUNCH("hils_attn_pool_fwd");
    return HILS_OK;
  }
  if (S == 64 && (D == 64 || D == 128) && HK < H && (long)BN * ((HK + 3) / 4) <= 2147483647L) {  // more than 16 heads a group
    const dim3 grid((unsigned)((long)BN * ((HK + 3) / 4)));
    if (D == 64)
      hipLaunchKernelGGL(attn_pool_fwd_rows_gqa<64>, grid, dim3(256), 0, (hipStream_t)stream,
                         (const bf16_t*)mu_q, (const bf16_t*)k, (bf16_t*)lmk_k, lmk_b, p, H, HK, sm_scale, compact);
    else
      hipLaunchKernelGGL(attn_pool_fwd_rows_gqa<128>, grid, dim3(256), 0, (hipStream_t)stream,
                         (const bf16_t*)mu_q, (const bf16_t*)k, (bf16_t*)lmk_k, lmk_b, p, H, HK, sm_scale, compact);
    HILS_CHECK_LAUNCH("hils_attn_pool_fwd");
    return HILS_OK;
  }
  if (S == 64 && (D == 64 || D == 128) && HK == H && (long)BN * ((H + 3) / 4) <= 2147483647L) {
    const dim3 grid((unsigned)((long)BN * ((H + 3) / 4)));
    if (D == 64)
      hipLaunchKernelGGL(attn_pool_fwd_rows<64>, grid, dim3(256), 0, (hipStream_t)stream,
                         (const bf16_t*)mu_q, (const bf16_t*)k, (bf16_t*)lmk_k, lmk_b, p, H, sm_scale,
                         compact, shared_k);
    else
      hipLaunchKernelGGL(attn_pool_fwd_rows<128>, grid, dim3(256), 0, (hipStream_t)stream,
                         (const bf16_t*)mu_q, (const bf16_t*)k, (bf16_t*)lmk_k, lmk_b, p, H, sm_scale,
                         compact, shared_k);
    HILS_CHECK_LAUNCH("hils_attn_pool_fwd");
    return HILS_OK;
  }
  size_t smem = ((size_t)S * (D + 1) + D + S + 32) * sizeof(float);
  HILS_REQUIRE(smem <= 160 * 1024, "hils_attn_pool_fwd: S*D (%d x %d) tile does not fit in LDS", S, D);
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)attn_pool_fwd_kernel,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  hipLaunchKernelGGL(attn_pool_fwd_kernel, dim3(BN, H), dim3(POOL_THREADS), smem,
                     (hipStream_t)stream, (const bf16_t*)mu_q, (const bf16_t*)k, (bf16_t*)lmk_k,
                     lmk_b, p, S, H, HK, D, sm_scale, compact, shared_k);
  HILS_CHECK_LAUNCH("hils_attn_pool_fwd");
  return HILS_OK;
}

extern "C" int hils_attn_pool_bwd(const void* mu_q, const void* k, const float* p,
                                  const float* lmk_b, const void* g_k, const float* g_b,
                                  void* d_mu, void* d_k, int BN, int S, int H, int h_kv, int D,
                                  float sm_scale, int compact, int shared_k, void* stream) {
  HILS_REQUIRE(mu_q && k && p && lmk_b && g_k && g_b && d_mu && d_k, "hils_attn_pool_bwd: null pointer");
  if (int rc = pool_check("hils_attn_pool_bwd", BN, S, H, h_kv, D, shared_k)) return rc;
  const int HK = h_kv;
  if (S == 64 && (D == 64 || D == 128) && HK < H && (long)BN * ((HK + 3) / 4) <= 2147483647L) {
    const dim3 grid((unsigned)((long)BN * ((HK + 3) / 4)));
    if (D == 64)
      hipLaunchKernelGGL(attn_pool_bwd_rows_gqa<64>, grid, dim3(256), 0, (hipStream_t)stream,
                         (const bf16_t*)mu_q, (const bf16_t*)k, p, lmk_b, (const bf16_t*)g_k, g_b,
                         (bf16_t*)d_mu, (bf16_t*)d_k, H, HK, sm_scale, compact);
    else
      hipLaunchKernelGGL(attn_pool_bwd_rows_gqa<128>, grid, dim3(256), 0, (hipStream_t)stream,
                         (const bf16_t*)mu_q, (const bf16_t*)k, p, lmk_b, (const bf16_t*)g_k, g_b,
                         (bf16_t*)d_mu, (bf16_t*)d_k, H, HK, sm_scale, compact);
    HILS_CHECK_LAUNCH("hils_attn_pool_bwd");
    return HILS_OK;
  }
  if (S == 64 && (D == 64 || D == 128) && HK == H && (long)BN * ((H + 3) / 4) <= 2147483647L) {
    const dim3 grid((unsigned)((long)BN * (shared_k ? 1 : (H + 3) / 4)));
    const size_t xch = shared_k ? (size_t)2 * S * D * sizeof(float) : 0;
#define POOL_BWD_ROWS(D_, SH_)                                                                      \
  hipLaunchKernelGGL((attn_pool_bwd_rows<D_, SH_>), grid, dim3(256), xch, (hipStream_t)stream,      \
                     (const bf16_t*)mu_q, (const bf16_t*)k, p, lmk_b, (const bf16_t*)g_k, g_b,      \
                     (bf16_t*)d_mu, (bf16_t*)d_k, H, sm_scale, compact)
    if (D == 64) {
      if (shared_k) POOL_BWD_ROWS(64, true); else POOL_BWD_ROWS(64, false);
    } else {
      if (shared_k) POOL_BWD_ROWS(128, true); else POOL_BWD_ROWS(128, false);
    }
#undef POOL_BWD_ROWS
    HILS_CHECK_LAUNCH("hils_attn_pool_bwd");
    return HILS_OK;
  }
  const bool summed = shared_k || HK < H;
  size_t smem = ((size_t)S * (D + 1) + 2 * D + 2 * S + 32 + (summed ? (size_t)S * D : 0)) * sizeof(float);
  HILS_REQUIRE(smem <= 160 * 1024, "hils_attn_pool_bwd: S*D (%d x %d) tile does not fit in LDS", S, D);
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)attn_pool_bwd_kernel,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  dim3 grid(BN, shared_k ? 1 : HK);
  hipLaunchKernelGGL(attn_pool_bwd_kernel, grid, dim3(POOL_THREADS), smem, (hipStream_t)stream,
                     (const bf16_t*)mu_q, (const bf16_t*)k, p, lmk_b, (const bf16_t*)g_k, g_b,
                     (bf16_t*)d_mu, (bf16_t*)d_k, S, H, HK, D, sm_scale, compact, shared_k);
  HILS_CHECK_LAUNCH("hils_attn_pool_bwd");
  return HILS_OK;
}
