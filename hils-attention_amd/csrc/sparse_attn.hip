// Sparse attention over selected chunks: shape-generic kernels (any D, Dv, G, chunk size).
//
// One workgroup owns one (batch, query, KV head): its G query heads share the K/V
// chunks of the K selected slots.  These kernels do their arithmetic on the vector
// ALU in fp32; they are the path for shapes the MFMA kernels do not cover and for
// decode-sized query counts, and they also implement the q-block-shared index /
// `sm_n` denominator variant of the older HSA operator.
#include "common.h"
#include "../../include/hils_amd.h"

#define SA_THREADS 256
#define SA_MAX_OUT 16  // outputs (g, dv) per thread

size_t hils_ga_workspace_bytes(int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K, int S,
                               int q_block, int WH, float sm_n);
int hils_sparse_attn_fwd_mfma(const void* q, const void* k, const void* v, const void* weights,
                              const int32_t* indices, const float* slope, const void* swa_o, int merge_col,
                              void* o, float* lse, void* workspace, int workspace_ready, int B, int L,
                              int Lkv, int HQ, int H, int D, int Dv, int K, int NW, int S, float sm_scale,
                              int mask_last, int q_block, int WH, float sm_n, void* stream,
                              int* handled);

bool hils_decode_covers(int L, int HQ, int H, int D, int Dv, int S, int q_block, int WH, float sm_n,
                        const float* slope, const float* lse);
size_t hils_decode_workspace_bytes(int B, int L, int HQ, int H, int Dv, int K);
int hils_sparse_attn_decode(const void* q, const void* k, const void* v, const void* weights,
                            const int32_t* indices, void* o, void* workspace, int B, int L, int Lkv,
                            int HQ, int H, int D, int Dv, int K, int NW, float sm_scale,
                            int mask_last, void* stream);

struct SaDims {
  int L, Lkv, HQ, H, G, D, Dv, K, NW, WH, q_block, S, mask_last;
  float sm_scale, sm_n;
  int skip_dkdv;  // backward: dK and dV come from the chunk-major kernel
};

// element access of the shape-generic kernels: bf16 tensors, or fp32 tensors (the fp32 mode)
__device__ __forceinline__ float sa_ld(const bf16_t* p) { return bf2f(*p); }
__device__ __forceinline__ float sa_ld(const float* p) { return *p; }
__device__ __forceinline__ void sa_ld8(const bf16_t* p, float* f) { unpack8(*(const uint4*)p, f); }
__device__ __forceinline__ void sa_ld8(const float* p, float* f) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void sa_st(bf16_t* p, float x) { *p = f2bf(x); }
__device__ __forceinline__ void sa_st(float* p, float x) { *p = x; }

// scores of slot chunk c for all (g, s): sc[g*S+s] = (q_g . K_s - slope_g*dist_s) * sm_scale,
// -inf for the masked last token.  q_s holds the G query rows in fp32.
template <class T>
__device__ __forceinline__ void sa_scores(const SaDims& dm, const float* q_s, const T* kbase,
                                          const float* slope_s, float* sc) {
  const int GS = dm.G * dm.S;
  for (int p = threadIdx.x; p < GS; p += SA_THREADS) {
    const int g = p / dm.S, s = p - g * dm.S;
    const T* kr = kbase + (long)s * dm.H * dm.D;
    const float* qr = q_s + g * dm.D;
    float a = 0.f;
    for (int d8 = 0; d8 < dm.D / 8; ++d8) {
      float f[8];
      sa_ld8(kr + d8 * 8, f);
#pragma unroll
      for (int j = 0; j < 8; ++j) a = fmaf(qr[d8 * 8 + j], f[j], a);
    }
    if (slope_s) {
      const int dist = dm.S - 2 - s;
      a -= slope_s[g] * (float)(dist > 0 ? dist : 0);
    }
    a *= dm.sm_scale;
    if (dm.mask_last && s == dm.S - 1) a = HILS_NEG_INF;
    sc[p] = a;
  }
}

template <class T>
__global__ void __launch_bounds__(SA_THREADS)
sparse_attn_fwd_simple(const T* __restrict__ q, const T* __restrict__ k,
                       const T* __restrict__ v, const T* __restrict__ weights,
                       const int32_t* __restrict__ indices, const float* __restrict__ slope,
                       T* __restrict__ o, float* __restrict__ lse, SaDims dm) {
  extern __shared__ float smem[];
  float* q_s = smem;                       // G*D
  float* sc = q_s + dm.G * dm.D;           // G*S
  float* w_s = sc + dm.G * dm.S;           // G
  float* slope_s = w_s + dm.G;             // G
  const int G = dm.G, S = dm.S, D = dm.D, Dv = dm.Dv;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long row = blockIdx.x;  // (b*L + t)*H + hk
  const int hk = (int)(row % dm.H);
  const long bt = row / dm.H;
  const int t = (int)(bt % dm.L);
  const long b = bt / dm.L;
  const long LB = dm.L / dm.q_block;
  const long irow = (b * LB + t / dm.q_block) * dm.H + hk;
  const int nchunk = dm.Lkv / S;

  for (int i = tid; i < G * D; i += SA_THREADS)
    q_s[i] = sa_ld(q + (bt * dm.HQ + hk * G) * (long)D + i);
  if (tid < G) slope_s[tid] = slope ? slope[hk * G + tid] : 0.f;

  float acc[SA_MAX_OUT];
#pragma unroll
  for (int j = 0; j < SA_MAX_OUT; ++j) acc[j] = 0.f;
  const int nout = G * Dv;

  for (int kk = 0; kk < dm.K; ++kk) {
    const int c = indices[irow * dm.K + kk];
    __syncthreads();
    if (c < 0 || c >= nchunk) {
      if (lse)  // empty or out-of-range slot
        for (int g = tid; g < G; g += SA_THREADS) lse[(bt * dm.HQ + hk * G + g) * (long)dm.K + kk] = HILS_NEG_INF;
      continue;
    }
    if (tid < G) {
      const long wrow = (b * LB + t / dm.q_block) * dm.WH + (dm.WH == dm.HQ ? hk * G + tid : hk);
      w_s[tid] = sa_ld(weights + wrow * dm.NW + kk);
    }
    const T* kbase = k + ((b * dm.Lkv + (long)c * S) * dm.H + hk) * D;
    const T* vbase = v + ((b * dm.Lkv + (long)c * S) * dm.H + hk) * Dv;
    sa_scores(dm, q_s, kbase, slope ? slope_s : nullptr, sc);
    __syncthreads();
    for (int g = wave; g < G; g += SA_THREADS / 64) {
      float m = HILS_NEG_INF;
      for (int s = lane; s < S; s += 64) m = fmaxf(m, sc[g * S + s]);
      m = wave_max(m);
      float sum = 0.f;
      for (int s = lane; s < S; s += 64) {
        const float x = sc[g * S + s];
        const float e = (x == HILS_NEG_INF) ? 0.f : __expf(x - m);
        sc[g * S + s] = e;
        sum += e;
      }
      sum = wave_sum(sum);
      const float den = (m > HILS_NEG_INF) ? sum + dm.sm_n * __expf(-m) : 0.f;
      const float f = den > 0.f ? w_s[g] / den : 0.f;
      for (int s = lane; s < S; s += 64) sc[g * S + s] *= f;
      if (lse && lane == 0)
        lse[(bt * dm.HQ + hk * G + g) * (long)dm.K + kk] =
            den > 0.f ? m * HILS_LOG2E + log2f(den) : HILS_NEG_INF;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < SA_MAX_OUT; ++j) {
      const int oi = tid + j * SA_THREADS;
      if (oi < nout) {
        const int g = oi / Dv, dv = oi - g * Dv;
        float a = acc[j];
        for (int s = 0; s < S; ++s) a = fmaf(sc[g * S + s], sa_ld(vbase + (long)s * dm.H * Dv + dv), a);
        acc[j] = a;
      }
    }
  }
#pragma unroll
  for (int j = 0; j < SA_MAX_OUT; ++j) {
    const int oi = tid + j * SA_THREADS;
    if (oi < nout) sa_st(o + (bt * dm.HQ + hk * G) * (long)Dv + oi, acc[j]);
  }
}

template <class T>
__global__ void __launch_bounds__(SA_THREADS)
sparse_attn_bwd_simple(const T* __restrict__ q, const T* __restrict__ k,
                       const T* __restrict__ v, const T* __restrict__ weights,
                       const int32_t* __restrict__ indices, const float* __restrict__ slope,
                       const float* __restrict__ lse, const T* __restrict__ d_o,
                       T* __restrict__ dq, float* __restrict__ dk, float* __restrict__ dv,
                       float* __restrict__ dw, SaDims dm) {
  extern __shared__ float smem[];
  const int G = dm.G, S = dm.S, D = dm.D, Dv = dm.Dv;
  float* q_s = smem;               // G*D
  float* do_s = q_s + G * D;       // G*Dv
  float* p_s = do_s + G * Dv;      // G*S  probabilities
  float* ds_s = p_s + G * S;       // G*S  dPV, then dS
  float* w_s = ds_s + G * S;       // G
  float* slope_s = w_s + G;        // G
  float* dwk = slope_s + G;        // G
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long row = blockIdx.x;
  const int hk = (int)(row % dm.H);
  const long bt = row / dm.H;
  const int t = (int)(bt % dm.L);
  const long b = bt / dm.L;
  const long LB = dm.L / dm.q_block;
  const long irow = (b * LB + t / dm.q_block) * dm.H + hk;
  const int nchunk = dm.Lkv / S;
  const bool dw_atomic = dm.q_block > 1 || dm.WH != dm.HQ;

  for (int i = tid; i < G * D; i += SA_THREADS) q_s[i] = sa_ld(q + (bt * dm.HQ + hk * G) * (long)D + i);
  for (int i = tid; i < G * Dv; i += SA_THREADS) do_s[i] = sa_ld(d_o + (bt * dm.HQ + hk * G) * (long)Dv + i);
  if (tid < G) slope_s[tid] = slope ? slope[hk * G + tid] : 0.f;

  float dq_acc[SA_MAX_OUT];
#pragma unroll
  for (int j = 0; j < SA_MAX_OUT; ++j) dq_acc[j] = 0.f;
  const int nq = G * D;

  for (int kk = 0; kk < dm.K; ++kk) {
    const int c = indices[irow * dm.K + kk];
    __syncthreads();
    if (c < 0 || c >= nchunk) continue;
    if (tid < G) {
      const long wrow = (b * LB + t / dm.q_block) * dm.WH + (dm.WH == dm.HQ ? hk * G + tid : hk);
      w_s[tid] = sa_ld(weights + wrow * dm.NW + kk);
    }
    const T* kbase = k + ((b * dm.Lkv + (long)c * S) * dm.H + hk) * D;
    const T* vbase = v + ((b * dm.Lkv + (long)c * S) * dm.H + hk) * Dv;
    sa_scores(dm, q_s, kbase, slope ? slope_s : nullptr, p_s);
    // dPV[g][s] = dO_g . V_s
    for (int p = tid; p < G * S; p += SA_THREADS) {
      const int g = p / S, s = p - g * S;
      const T* vr = vbase + (long)s * dm.H * Dv;
      float a = 0.f;
      for (int d8 = 0; d8 < Dv / 8; ++d8) {
        float f[8];
        sa_ld8(vr + d8 * 8, f);
#pragma unroll
        for (int j = 0; j < 8; ++j) a = fmaf(do_s[g * Dv + d8 * 8 + j], f[j], a);
      }
      ds_s[p] = a;
    }
    __syncthreads();
    for (int g = wave; g < G; g += SA_THREADS / 64) {
      const float l2 = lse[(bt * dm.HQ + hk * G + g) * (long)dm.K + kk];
      float part = 0.f;
      for (int s = lane; s < S; s += 64) {
        const float x = p_s[g * S + s];
        const float pv = (x == HILS_NEG_INF || l2 == HILS_NEG_INF) ? 0.f : exp2f(x * HILS_LOG2E - l2);
        p_s[g * S + s] = pv;
        part += pv * ds_s[g * S + s];
      }
      part = wave_sum(part);
      if (lane == 0) dwk[g] = part;
      const float wg = w_s[g];
      for (int s = lane; s < S; s += 64)
        ds_s[g * S + s] = dm.sm_scale * wg * p_s[g * S + s] * (ds_s[g * S + s] - part);
    }
    __syncthreads();
    if (tid < G) {
      const long wrow = (b * LB + t / dm.q_block) * dm.WH + (dm.WH == dm.HQ ? hk * G + tid : hk);
      if (dw_atomic) atomicAdd(dw + wrow * dm.NW + kk, dwk[tid]);
      else dw[wrow * dm.NW + kk] = dwk[tid];
    }
    // dV[s][dv] += sum_g w_g P[g][s] dO[g][dv]
    float* dvb = dv + ((b * dm.Lkv + (long)c * S) * dm.H + hk) * Dv;
    for (int p = tid; p < (dm.skip_dkdv ? 0 : S * Dv); p += SA_THREADS) {
      const int s = p / Dv, d = p - s * Dv;
      float a = 0.f;
      for (int g = 0; g < G; ++g) a = fmaf(w_s[g] * p_s[g * S + s], do_s[g * Dv + d], a);
      if (a != 0.f) atomicAdd(dvb + (long)s * dm.H * Dv + d, a);
    }
    // dK[s][d] += sum_g dS[g][s] q[g][d]
    float* dkb = dk + ((b * dm.Lkv + (long)c * S) * dm.H + hk) * D;
    for (int p = tid; p < (dm.skip_dkdv ? 0 : S * D); p += SA_THREADS) {
      const int s = p / D, d = p - s * D;
      float a = 0.f;
      for (int g = 0; g < G; ++g) a = fmaf(ds_s[g * S + s], q_s[g * D + d], a);
      if (a != 0.f) atomicAdd(dkb + (long)s * dm.H * D + d, a);
    }
    // dQ[g][d] += sum_s dS[g][s] K[s][d]
#pragma unroll
    for (int j = 0; j < SA_MAX_OUT; ++j) {
      const int oi = tid + j * SA_THREADS;
      if (oi < nq) {
        const int g = oi / D, d = oi - g * D;
        float a = dq_acc[j];
        for (int s = 0; s < S; ++s) a = fmaf(ds_s[g * S + s], sa_ld(kbase + (long)s * dm.H * D + d), a);
        dq_acc[j] = a;
      }
    }
  }
#pragma unroll
  for (int j = 0; j < SA_MAX_OUT; ++j) {
    const int oi = tid + j * SA_THREADS;
    if (oi < nq) sa_st(dq + (bt * dm.HQ + hk * G) * (long)D + oi, dq_acc[j]);
  }
}

static int sa_check(const char* name, int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K,
                    int NW, int WH, int q_block, int S) {
  HILS_REQUIRE(B > 0 && L > 0 && Lkv > 0 && HQ > 0 && H > 0 && D > 0 && Dv > 0 && K > 0 && S > 0,
               "%s: sizes must be positive", name);
  HILS_REQUIRE(HQ % H == 0, "%s: HQ (%d) must be a multiple of H (%d)", name, HQ, H);
  HILS_REQUIRE(D % 8 == 0 && Dv % 8 == 0, "%s: D (%d) and Dv (%d) must be multiples of 8", name, D, Dv);
  HILS_REQUIRE(NW >= K, "%s: weights hold %d columns, need at least K = %d", name, NW, K);
  HILS_REQUIRE(WH == HQ || WH == H, "%s: weights head count %d must be HQ or H", name, WH);
  HILS_REQUIRE(q_block >= 1 && L % q_block == 0, "%s: L (%d) must be a multiple of q_block (%d)", name, L, q_block);
  const int G = HQ / H;
  HILS_REQUIRE(G * Dv <= SA_MAX_OUT * SA_THREADS && G * D <= SA_MAX_OUT * SA_THREADS,
               "%s: G*D (%d) or G*Dv (%d) too large", name, G * D, G * Dv);
  HILS_REQUIRE((long)B * L * H <= 2147483647L, "%s: grid too large", name);
  return HILS_OK;
}

extern "C" size_t hils_sparse_attn_fwd_workspace(int B, int L, int Lkv, int HQ, int H, int D,
                                                 int Dv, int K, int WH, int q_block, int S,
                                                 float sm_n) {
  if (hils_decode_covers(L, HQ, H, D, Dv, S, q_block, WH, sm_n, nullptr, nullptr))
    return hils_decode_workspace_bytes(B, L, HQ, H, Dv, K);
  return hils_ga_workspace_bytes(B, L, Lkv, HQ, H, D, Dv, K, S, q_block, WH, sm_n);
}

// o += swa_o * weights[..., col] for the paths that do not merge in their own epilogue:
// one thread per 8 output elements.
__global__ void __launch_bounds__(256)
merge_local_kernel(bf16_t* __restrict__ o, const bf16_t* __restrict__ swa_o, const bf16_t* __restrict__ weights,
                   long n8, int L, int HQ, int G, int Dv, int NW, int WH, int q_block, int col) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  const int c8n = Dv / 8;
  const long row = i / c8n;          // (b*L + t)*HQ + hq
  const int hq = (int)(row % HQ);
  const long bt = row / HQ;
  const int t = (int)(bt % L);
  const long b = bt / L;
  const long wrow = (b * (L / q_block) + t / q_block) * WH + (WH == HQ ? hq : hq / G);
  const float wl = bf2f(weights[wrow * NW + col]);
  float a[8], c[8];
  unpack8(*(const uint4*)(o + i * 8), a);
  unpack8(*(const uint4*)(swa_o + i * 8), c);
  uint4 x;
  x.x = pack_bf2(fmaf(c[0], wl, a[0]), fmaf(c[1], wl, a[1]));
  x.y = pack_bf2(fmaf(c[2], wl, a[2]), fmaf(c[3], wl, a[3]));
  x.z = pack_bf2(fmaf(c[4], wl, a[4]), fmaf(c[5], wl, a[5]));
  x.w = pack_bf2(fmaf(c[6], wl, a[6]), fmaf(c[7], wl, a[7]));
  *(uint4*)(o + i * 8) = x;
}

static int sa_merge_local(void* o, const void* swa_o, const void* weights, int B, int L, int HQ, int H,
                          int Dv, int NW, int WH, int q_block, int col, void* stream) {
  const long n8 = (long)B * L * HQ * (Dv / 8);
  HILS_REQUIRE((n8 + 255) / 256 <= 2147483647L, "hils_sparse_attn_fwd: grid too large");
  hipLaunchKernelGGL(merge_local_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (bf16_t*)o, (const bf16_t*)swa_o, (const bf16_t*)weights, n8, L, HQ, HQ / H, Dv, NW, WH,
                     q_block, col);
  return HILS_OK;
}

extern "C" int hils_sparse_attn_fwd(const void* q, const void* k, const void* v,
                                    const void* weights, const int32_t* indices,
                                    const float* slope, const void* swa_o, void* o, float* lse,
                                    void* workspace, size_t workspace_bytes, int workspace_ready, int B, int L,
                                    int Lkv, int HQ, int H, int D, int Dv, int K, int NW, int WH, int q_block,
                                    int S, float sm_scale, int mask_last, float sm_n, int merge_col,
                                    void* stream) {
  HILS_REQUIRE(q && k && v && weights && indices && o, "hils_sparse_attn_fwd: null pointer");
  if (int rc = sa_check("hils_sparse_attn_fwd", B, L, Lkv, HQ, H, D, Dv, K, NW, WH, q_block, S)) return rc;
  {
    const size_t need = hils_sparse_attn_fwd_workspace(B, L, Lkv, HQ, H, D, Dv, K, WH, q_block, S, sm_n);
    HILS_REQUIRE(!workspace || workspace_bytes >= need,
                 "hils_sparse_attn_fwd: workspace of %zu bytes is shorter than the %zu bytes "
                 "hils_sparse_attn_fwd_workspace returns for this shape (a workspace packed for another "
                 "shape cannot be reused)", workspace_bytes, need);
  }
  HILS_REQUIRE(!swa_o || (merge_col >= 0 && merge_col < NW),
               "hils_sparse_attn_fwd: merge_col (%d) must be a weight column (0..%d)", merge_col, NW - 1);
  if (hils_decode_covers(L, HQ, H, D, Dv, S, q_block, WH, sm_n, slope, lse) && Lkv >= S) {
    if (int rc = hils_sparse_attn_decode(q, k, v, weights, indices, o, workspace, B, L, Lkv, HQ, H, D,
                                         Dv, K, NW, sm_scale, mask_last, stream))
      return rc;
    if (swa_o)
      if (int rc = sa_merge_local(o, swa_o, weights, B, L, HQ, H, Dv, NW, WH, q_block, merge_col, stream)) return rc;
    HILS_CHECK_LAUNCH("hils_sparse_attn_fwd");
    return HILS_OK;
  }
  if (workspace && hils_ga_workspace_bytes(B, L, Lkv, HQ, H, D, Dv, K, S, q_block, WH, sm_n) > 0) {
    int handled = 0;
    if (int rc = hils_sparse_attn_fwd_mfma(q, k, v, weights, indices, slope, swa_o, merge_col, o, lse,
                                           workspace, workspace_ready, B, L, Lkv, HQ, H, D, Dv, K, NW, S,
                                           sm_scale, mask_last, q_block, WH, sm_n, stream, &handled))
      return rc;
    if (handled) {
      HILS_CHECK_LAUNCH("hils_sparse_attn_fwd");
      return HILS_OK;
    }
  }
  SaDims dm{L, Lkv, HQ, H, HQ / H, D, Dv, K, NW, WH, q_block, S, mask_last, sm_scale, sm_n, 0};
  size_t smem = ((size_t)dm.G * D + (size_t)dm.G * S + 2 * dm.G) * sizeof(float);
  HILS_REQUIRE(smem <= 64 * 1024, "hils_sparse_attn_fwd: G*(D+S) too large for LDS");
  hipLaunchKernelGGL(sparse_attn_fwd_simple<bf16_t>, dim3((unsigned)((long)B * L * H)), dim3(SA_THREADS),
                     smem, (hipStream_t)stream, (const bf16_t*)q, (const bf16_t*)k,
                     (const bf16_t*)v, (const bf16_t*)weights, indices, slope, (bf16_t*)o, lse, dm);
  if (swa_o)
    if (int rc = sa_merge_local(o, swa_o, weights, B, L, HQ, H, Dv, NW, WH, q_block, merge_col, stream)) return rc;
  HILS_CHECK_LAUNCH("hils_sparse_attn_fwd");
  return HILS_OK;
}

bool hils_bw_covers(int L, int Lkv, int HQ, int H, int D, int Dv, int K, int S, int q_block, int WH,
                    float sm_n, const float* slope);
size_t hils_bw_workspace_bytes(int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K, int S,
                               int q_block, int WH, float sm_n);
int hils_bw_run(const void* q, const void* k, const void* v, const void* weights, const int32_t* indices,
                const float* slope, const float* lse, const void* d_o, void* dq, void* dk, void* dv,
                float* dw, void* workspace, int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K, int NW,
                float sm_scale, int mask_last, int kv16, void* stream);

extern "C" size_t hils_sparse_attn_bwd_workspace(int B, int L, int Lkv, int HQ, int H, int D, int Dv,
                                                 int K, int WH, int q_block, int S, float sm_n) {
  return hils_bw_workspace_bytes(B, L, Lkv, HQ, H, D, Dv, K, S, q_block, WH, sm_n);
}

// Backward of the merge o = o_remote + swa_o * w[col]: d_swa_o = d_o * w[col], dw[col] = <d_o, swa_o>.
// Dv/8 neighbouring lanes own one (query, head) row.
__global__ void __launch_bounds__(256)
merge_local_bwd_kernel(const bf16_t* __restrict__ d_o, const bf16_t* __restrict__ swa_o,
                       const bf16_t* __restrict__ weights, bf16_t* __restrict__ d_swa_o, float* __restrict__ dw,
                       long n8, int lpr, int NW, int col) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  const bool ok = i < n8;
  const long row = (ok ? i : n8 - 1) / lpr;
  const float wl = bf2f(weights[row * NW + col]);
  float g[8], c[8];
  float dot = 0.f;
  if (ok) {
    unpack8(*(const uint4*)(d_o + i * 8), g);
    unpack8(*(const uint4*)(swa_o + i * 8), c);
#pragma unroll
    for (int e = 0; e < 8; ++e) dot = fmaf(g[e], c[e], dot);
    uint4 x;
    x.x = pack_bf2(g[0] * wl, g[1] * wl);
    x.y = pack_bf2(g[2] * wl, g[3] * wl);
    x.z = pack_bf2(g[4] * wl, g[5] * wl);
    x.w = pack_bf2(g[6] * wl, g[7] * wl);
    *(uint4*)(d_swa_o + i * 8) = x;
  }
  for (int o2 = 1; o2 < lpr; o2 <<= 1) dot += __shfl_xor(dot, o2, 64);
  if (ok && (i % lpr) == 0) dw[row * NW + col] = dot;
}

extern "C" int hils_sparse_attn_bwd(const void* q, const void* k, const void* v,
                                    const void* weights, const int32_t* indices,
                                    const float* slope, const float* lse, const void* d_o,
                                    void* dq, void* dk, void* dv, float* dw, void* workspace,
                                    size_t workspace_bytes, int B,
                                    int L, int Lkv, int HQ, int H, int D, int Dv, int K, int NW, int WH,
                                    int q_block, int S, float sm_scale, int mask_last, float sm_n,
                                    const void* swa_o, void* d_swa_o, int merge_col, int kv_grad_bf16,
                                    void* stream) {
  HILS_REQUIRE(q && k && v && weights && indices && lse && d_o && dq && dk && dv && dw,
               "hils_sparse_attn_bwd: null pointer");
  if (int rc = sa_check("hils_sparse_attn_bwd", B, L, Lkv, HQ, H, D, Dv, K, NW, WH, q_block, S)) return rc;
  {
    const size_t need = hils_bw_workspace_bytes(B, L, Lkv, HQ, H, D, Dv, K, S, q_block, WH, sm_n);
    HILS_REQUIRE(!workspace || workspace_bytes >= need,
                 "hils_sparse_attn_bwd: workspace of %zu bytes is shorter than the %zu bytes "
                 "hils_sparse_attn_bwd_workspace returns for this shape", workspace_bytes, need);
  }
  if (swa_o) {  // the forward merged the local branch: its gradient and that of its weight column
    const int lpr = Dv / 8;
    HILS_REQUIRE(d_swa_o && merge_col >= K && merge_col < NW && q_block == 1 && WH == HQ && lpr <= 64 &&
                     (lpr & (lpr - 1)) == 0,
                 "hils_sparse_attn_bwd: the merged local branch needs d_swa_o, a weight column in K..NW-1, "
                 "per-query-head weights and Dv/8 a power of two");
    const long n8 = (long)B * L * HQ * lpr;
    HILS_REQUIRE((n8 + 255) / 256 <= 2147483647L, "hils_sparse_attn_bwd: grid too large");
    hipLaunchKernelGGL(merge_local_bwd_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (const bf16_t*)d_o, (const bf16_t*)swa_o, (const bf16_t*)weights,
                       (bf16_t*)d_swa_o, dw, n8, lpr, NW, merge_col);
  }
  if (workspace && hils_bw_workspace_bytes(B, L, Lkv, HQ, H, D, Dv, K, S, q_block, WH, sm_n) > 0 &&
      hils_bw_covers(L, Lkv, HQ, H, D, Dv, K, S, q_block, WH, sm_n, slope)) {
    const int rc = hils_bw_run(q, k, v, weights, indices, slope, lse, d_o, dq, dk, dv, dw, workspace, B, L, Lkv, HQ,
                               H, D, Dv, K, NW, sm_scale, mask_last, kv_grad_bf16 ? 1 : 0, stream);
    if (rc > 0) return rc;
    if (rc == HILS_OK) {
      HILS_CHECK_LAUNCH("hils_sparse_attn_bwd");
      return HILS_OK;
    }
  }
  HILS_REQUIRE(!kv_grad_bf16, "hils_sparse_attn_bwd: bf16 dk / dv need the workspace kernels (a workspace of "
                              "hils_sparse_attn_bwd_workspace bytes > 0)");
  SaDims dm{L, Lkv, HQ, H, HQ / H, D, Dv, K, NW, WH, q_block, S, mask_last, sm_scale, sm_n, 0};
  size_t smem = ((size_t)dm.G * (D + Dv) + 2 * (size_t)dm.G * S + 3 * dm.G) * sizeof(float);
  HILS_REQUIRE(smem <= 64 * 1024, "hils_sparse_attn_bwd: G*(D+Dv+2S) too large for LDS");
  hipLaunchKernelGGL(sparse_attn_bwd_simple<bf16_t>, dim3((unsigned)((long)B * L * H)), dim3(SA_THREADS),
                     smem, (hipStream_t)stream, (const bf16_t*)q, (const bf16_t*)k,
                     (const bf16_t*)v, (const bf16_t*)weights, indices, slope, lse,
                     (const bf16_t*)d_o, (bf16_t*)dq, (float*)dk, (float*)dv, dw, dm);
  HILS_CHECK_LAUNCH("hils_sparse_attn_bwd");
  return HILS_OK;
}


// ---- fp32 tensors (the reference's dtype="float32" mode): the shape-generic kernels on fp32 q, k,
// v, weights, d_o; fp32 o and dq; everything computed in fp32 (no bf16 rounding of P) ----
extern "C" int hils_sparse_attn_fwd_f32(const float* q, const float* k, const float* v, const float* weights,
                                        const int32_t* indices, const float* slope, float* o, float* lse,
                                        int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K, int NW,
                                        int WH, int q_block, int S, float sm_scale, int mask_last, float sm_n,
                                        void* stream) {
  HILS_REQUIRE(q && k && v && weights && indices && o, "hils_sparse_attn_fwd_f32: null pointer");
  if (int rc = sa_check("hils_sparse_attn_fwd_f32", B, L, Lkv, HQ, H, D, Dv, K, NW, WH, q_block, S)) return rc;
  HILS_REQUIRE(Lkv >= S, "hils_sparse_attn_fwd_f32: Lkv (%d) is shorter than one chunk (%d)", Lkv, S);
  SaDims dm{L, Lkv, HQ, H, HQ / H, D, Dv, K, NW, WH, q_block, S, mask_last, sm_scale, sm_n, 0};
  const size_t smem = ((size_t)dm.G * D + (size_t)dm.G * S + 2 * dm.G) * sizeof(float);
  HILS_REQUIRE(smem <= 64 * 1024, "hils_sparse_attn_fwd_f32: G*(D+S) too large for LDS");
  hipLaunchKernelGGL(sparse_attn_fwd_simple<float>, dim3((unsigned)((long)B * L * H)), dim3(SA_THREADS), smem,
                     (hipStream_t)stream, q, k, v, weights, indices, slope, o, lse, dm);
  HILS_CHECK_LAUNCH("hils_sparse_attn_fwd_f32");
  return HILS_OK;
}

extern "C" int hils_sparse_attn_bwd_f32(const float* q, const float* k, const float* v, const float* weights,
                                        const int32_t* indices, const float* slope, const float* lse,
                                        const float* d_o, float* dq, float* dk, float* dv, float* dw, int B,
                                        int L, int Lkv, int HQ, int H, int D, int Dv, int K, int NW, int WH,
                                        int q_block, int S, float sm_scale, int mask_last, float sm_n,
                                        void* stream) {
  HILS_REQUIRE(q && k && v && weights && indices && lse && d_o && dq && dk && dv && dw,
               "hils_sparse_attn_bwd_f32: null pointer");
  if (int rc = sa_check("hils_sparse_attn_bwd_f32", B, L, Lkv, HQ, H, D, Dv, K, NW, WH, q_block, S)) return rc;
  SaDims dm{L, Lkv, HQ, H, HQ / H, D, Dv, K, NW, WH, q_block, S, mask_last, sm_scale, sm_n, 0};
  const size_t smem = ((size_t)dm.G * (D + Dv) + 2 * (size_t)dm.G * S + 3 * dm.G) * sizeof(float);
  HILS_REQUIRE(smem <= 64 * 1024, "hils_sparse_attn_bwd_f32: G*(D+Dv+2S) too large for LDS");
  hipLaunchKernelGGL(sparse_attn_bwd_simple<float>, dim3((unsigned)((long)B * L * H)), dim3(SA_THREADS), smem,
                     (hipStream_t)stream, q, k, v, weights, indices, slope, lse, d_o, dq, dk, dv, dw, dm);
  HILS_CHECK_LAUNCH("hils_sparse_attn_bwd_f32");
  return HILS_OK;
}
