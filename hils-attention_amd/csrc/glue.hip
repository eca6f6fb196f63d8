// Inter-chunk softmax of the HiLS layer, fused: prior-bias gather + concatenation with the
// local-branch LSE (+ the optional "softmax-1" zero logit) + softmax, one pass, bf16 out.
#include "common.h"
#include "../../include/hils_amd.h"

#define GL_MAXK 64

// One thread per (batch, query, query head) row.
__global__ void __launch_bounds__(256)
chunk_weights_kernel(const bf16_t* __restrict__ scores, const void* __restrict__ lse_ptr,
                     int lse_bf16, const float* __restrict__ prior_b, const int32_t* __restrict__ indices,
                     bf16_t* __restrict__ weights, long rows, int L, int HQ, int H, int N, int K,
                     int softmax1) {
  const long row = (long)blockIdx.x * blockDim.x + threadIdx.x;  // (b*L + t)*HQ + hq
  if (row >= rows) return;
  const int hq = (int)(row % HQ);
  const long bt = row / HQ;
  const long b = bt / L;
  const int G = HQ / H;
  const bf16_t* srow = scores + row * K;
  float x[GL_MAXK];
  const float lse_v = lse_bf16 ? bf2f(((const bf16_t*)lse_ptr)[row]) : ((const float*)lse_ptr)[row];
  float m = lse_v;
  if (softmax1) m = fmaxf(m, 0.f);
#pragma unroll
  for (int k = 0; k < GL_MAXK; ++k) {
    if (k < K) {
      float s = bf2f(srow[k]);
      if (prior_b) {
        int c = indices[(bt * H + hq / G) * (long)K + k];
        c = c < 0 ? 0 : c;
        // the layer adds the gathered bias after casting it to the scores' dtype
        s = bf2f(f2bf(s + bf2f(f2bf(prior_b[(b * N + c) * (long)HQ + hq]))));
      }
      x[k] = s;
      m = fmaxf(m, s);
    }
  }
  const int NW = K + 1 + (softmax1 ? 1 : 0);
  bf16_t* wrow = weights + row * NW;
  if (m == HILS_NEG_INF) {  // every logit is -inf: softmax of that row is NaN in the reference
    for (int k = 0; k < NW; ++k) wrow[k] = 0x7fc0;
    return;
  }
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < GL_MAXK; ++k)
    if (k < K) { x[k] = __expf(x[k] - m); sum += x[k]; }
  const float el = __expf(lse_v - m);
  sum += el;
  const float e0 = softmax1 ? __expf(0.f - m) : 0.f;
  sum += e0;
  const float inv = 1.f / sum;
#pragma unroll
  for (int k = 0; k < GL_MAXK; ++k)
    if (k < K) wrow[k] = f2bf(x[k] * inv);
  wrow[K] = f2bf(el * inv);
  if (softmax1) wrow[K + 1] = f2bf(e0 * inv);
}

// Cooperative variant for K in {8, 16, 32, 64}: K/8 neighbouring lanes own one row (one
// 16-byte load each), reductions run over those lanes with DPP, and the (K+1(+1))-wide output
// rows of a wavefront, contiguous in memory, are staged in LDS and stored coalesced.
template <int LPR>
__global__ void __launch_bounds__(256)
chunk_weights_rows_kernel(const bf16_t* __restrict__ scores, const void* __restrict__ lse_swa,
                          int lse_bf16, const float* __restrict__ prior_b,
                          const int32_t* __restrict__ indices, bf16_t* __restrict__ weights, long rows,
                          int L, int HQ, int H, int N, int softmax1) {
  constexpr int K = LPR * 8, RPW = 64 / LPR;
  __shared__ bf16_t stage[4][RPW * (K + 2)];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPR, rl = lane / LPR;
  const long row0 = ((long)blockIdx.x * 4 + wave) * RPW;
  const long row = row0 + rl;
  const int NW = K + 1 + (softmax1 ? 1 : 0);
  const bool valid = row < rows;
  float x[8];
  float lse = HILS_NEG_INF;
  if (valid) {
    const uint4 v = *(const uint4*)(scores + row * K + sub * 8);
    unpack8(v, x);
    lse = lse_bf16 ? bf2f(((const bf16_t*)lse_swa)[row]) : ((const float*)lse_swa)[row];
    if (prior_b) {
      const int hq = (int)(row % HQ);
      const long bt = row / HQ;
      const long b = bt / L;
      const int G = HQ / H;
      const int32_t* ip = indices + (bt * H + hq / G) * (long)K + sub * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        int c = ip[e];
        c = c < 0 ? 0 : c;
        x[e] = bf2f(f2bf(x[e] + bf2f(f2bf(prior_b[(b * N + c) * (long)HQ + hq]))));
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = HILS_NEG_INF;
  }
  float m = softmax1 ? fmaxf(lse, 0.f) : lse;
#pragma unroll
  for (int e = 0; e < 8; ++e) m = fmaxf(m, x[e]);
  if (LPR >= 2) m = fmaxf(m, __shfl_xor(m, 1, 64));
  if (LPR >= 4) m = fmaxf(m, __shfl_xor(m, 2, 64));
  if (LPR >= 8) m = fmaxf(m, __shfl_xor(m, 4, 64));
  const bool dead = !(m > HILS_NEG_INF);  // all logits -inf: the reference's softmax gives NaN
  float sum = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) { x[e] = dead ? 0.f : __expf(x[e] - m); sum += x[e]; }
  if (LPR >= 2) sum += __shfl_xor(sum, 1, 64);
  if (LPR >= 4) sum += __shfl_xor(sum, 2, 64);
  if (LPR >= 8) sum += __shfl_xor(sum, 4, 64);
  const float el = dead ? 0.f : __expf(lse - m);
  const float e0 = (softmax1 && !dead) ? __expf(0.f - m) : 0.f;
  const float inv = dead ? __uint_as_float(0x7fc00000u) : 1.f / (sum + el + e0);
  bf16_t* st = stage[wave] + rl * NW;
#pragma unroll
  for (int e = 0; e < 8; ++e) st[sub * 8 + e] = f2bf(dead ? inv : x[e] * inv);
  if (sub == 0) {
    st[K] = f2bf(dead ? inv : el * inv);
    if (softmax1) st[K + 1] = f2bf(dead ? inv : e0 * inv);
  }
  // same wavefront wrote the slice: stores and loads of one wavefront stay in program order
  long nrow = rows - row0;
  if (nrow > RPW) nrow = RPW;
  if (nrow <= 0) return;
  const int total = (int)nrow * NW;
  bf16_t* dst = weights + row0 * NW;
  for (int i = lane; i < total; i += 64) dst[i] = stage[wave][i];
}

extern "C" int hils_chunk_weights(const void* scores, const void* lse_swa, int lse_bf16,
                                  const float* prior_b, const int32_t* indices, void* weights, int B,
                                  int L, int HQ, int H, int N, int K, int softmax1, void* stream) {
  HILS_REQUIRE(scores && lse_swa && weights, "hils_chunk_weights: null pointer");
  HILS_REQUIRE(!prior_b || indices, "hils_chunk_weights: prior_b needs indices");
  HILS_REQUIRE(B > 0 && L > 0 && HQ > 0 && H > 0 && HQ % H == 0, "hils_chunk_weights: bad head counts");
  HILS_REQUIRE(K >= 1 && K <= GL_MAXK, "hils_chunk_weights: K (%d) must be in 1..%d", K, GL_MAXK);
  const long rows = (long)B * L * HQ;
  const long nblk = (rows + 255) / 256;
  HILS_REQUIRE(nblk <= 2147483647L, "hils_chunk_weights: grid too large");
  if (K == 8 || K == 16 || K == 32 || K == 64) {
    const int rpw = 64 / (K / 8);
    const long nb = (rows + 4 * rpw - 1) / (4 * rpw);
    HILS_REQUIRE(nb <= 2147483647L, "hils_chunk_weights: grid too large");
#define GL_CALL(LPR_)                                                                              \
  hipLaunchKernelGGL(chunk_weights_rows_kernel<LPR_>, dim3((unsigned)nb), dim3(256), 0,            \
                     (hipStream_t)stream, (const bf16_t*)scores, lse_swa, lse_bf16, prior_b, indices, \
                     (bf16_t*)weights, rows, L, HQ, H, N, softmax1)
    if (K == 8) GL_CALL(1); else if (K == 16) GL_CALL(2); else if (K == 32) GL_CALL(4); else GL_CALL(8);
#undef GL_CALL
    HILS_CHECK_LAUNCH("hils_chunk_weights");
    return HILS_OK;
  }
  hipLaunchKernelGGL(chunk_weights_kernel, dim3((unsigned)nblk), dim3(256), 0, (hipStream_t)stream,
                     (const bf16_t*)scores, lse_swa, lse_bf16, prior_b, indices, (bf16_t*)weights, rows, L, HQ, H,
                     N, K, softmax1);
  HILS_CHECK_LAUNCH("hils_chunk_weights");
  return HILS_OK;
}

// Backward of the inter-chunk softmax.  One thread per (batch, query, query head) row: the logits
// are rebuilt from the forward's inputs (so the probabilities are the unrounded fp32 ones the
// reference's autograd uses), then d_logit_j = y_j * (d_w_j - sum_i y_i d_w_i).  Columns: K chunk
// scores, the local-branch LSE, and with softmax1 a constant zero logit (no gradient).
__global__ void __launch_bounds__(256)
chunk_weights_bwd_kernel(const bf16_t* __restrict__ scores, const void* __restrict__ lse_ptr, int lse_bf16,
                         const float* __restrict__ prior_b, const int32_t* __restrict__ indices,
                         const bf16_t* __restrict__ d_weights, bf16_t* __restrict__ d_scores,
                         float* __restrict__ d_lse, float* __restrict__ d_prior_b, long rows, int L, int HQ,
                         int H, int N, int K, int softmax1) {
  const long row = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= rows) return;
  const int hq = (int)(row % HQ);
  const long bt = row / HQ;
  const long b = bt / L;
  const int G = HQ / H;
  const bf16_t* srow = scores + row * K;
  const int NW = K + 1 + (softmax1 ? 1 : 0);
  const bf16_t* grow = d_weights + row * NW;
  const int32_t* irow = indices ? indices + (bt * H + hq / G) * (long)K : nullptr;
  float x[GL_MAXK];
  const float lse_v = lse_bf16 ? bf2f(((const bf16_t*)lse_ptr)[row]) : ((const float*)lse_ptr)[row];
  float m = softmax1 ? fmaxf(lse_v, 0.f) : lse_v;
#pragma unroll
  for (int k = 0; k < GL_MAXK; ++k) {
    if (k < K) {
      float s = bf2f(srow[k]);
      if (prior_b) {
        int c = irow[k];
        c = c < 0 ? 0 : c;
        s = bf2f(f2bf(s + bf2f(f2bf(prior_b[(b * N + c) * (long)HQ + hq]))));
      }
      x[k] = s;
      m = fmaxf(m, s);
    }
  }
  bf16_t* drow = d_scores + row * K;
  if (m == HILS_NEG_INF) {  // forward gave NaN weights for this row
    for (int k = 0; k < K; ++k) drow[k] = 0x7fc0;
    if (d_lse) d_lse[row] = __uint_as_float(0x7fc00000u);
    return;
  }
  float sum = 0.f, dot = 0.f;
#pragma unroll
  for (int k = 0; k < GL_MAXK; ++k)
    if (k < K) {
      x[k] = __expf(x[k] - m);
      sum += x[k];
      dot += x[k] * bf2f(grow[k]);
    }
  const float el = __expf(lse_v - m);
  const float gl = bf2f(grow[K]);
  sum += el;
  dot += el * gl;
  if (softmax1) {
    const float e0 = __expf(0.f - m);
    sum += e0;
    dot += e0 * bf2f(grow[K + 1]);
  }
  const float inv = 1.f / sum;
  dot *= inv;  // sum_i y_i d_w_i
#pragma unroll
  for (int k = 0; k < GL_MAXK; ++k)
    if (k < K) {
      const float dl = x[k] * inv * (bf2f(grow[k]) - dot);
      drow[k] = f2bf(dl);
      if (d_prior_b && dl != 0.f) {  // empty slots gather chunk 0, as the forward does (their dl is 0 when the score is -inf)
        const int c = irow[k] < 0 ? 0 : irow[k];
        atomicAdd(d_prior_b + (b * N + c) * (long)HQ + hq, dl);
      }
    }
  if (d_lse) d_lse[row] = el * inv * (gl - dot);
}

// Cooperative variant for K in {8, 16, 32, 64}, laid out like the forward's: K/8 neighbouring
// lanes own one row (one 16-byte load of scores and one 16-byte store of d_scores each).  The
// (K+1(+1))-wide d_weights rows of a wavefront are contiguous in memory but not 16-byte aligned:
// they are loaded coalesced into LDS and read from there.
// TAB (with d_prior_b): a workgroup walks a run of consecutive rows of one batch element and adds the bias
// gradients into a table (N x HQ) in LDS, which it adds to d_prior_b once at the end.  One global
// atomic per element has every query of a batch element adding into the same N x HQ words: 33 M adds into
// 16 K words took 0.51 ms at B8 L8192 h16 K32.  The table is 64-bit fixed point (2^-40): integer LDS adds
// run at several times the rate of float ones, and a run's sum does not depend on the order of its adds.
// (TAB: 16 wavefronts a workgroup, two workgroups a compute unit: the rows of a run are walked one tile after
// the other, and with four wavefronts a workgroup too few loads were in flight)
template <int LPR, bool TAB>
__global__ void __launch_bounds__(TAB ? 1024 : 256)
chunk_weights_bwd_rows_kernel(const bf16_t* __restrict__ scores, const void* __restrict__ lse_swa,
                              int lse_bf16, const float* __restrict__ prior_b,
                              const int32_t* __restrict__ indices, const bf16_t* __restrict__ d_weights,
                              bf16_t* __restrict__ d_scores, float* __restrict__ d_lse,
                              float* __restrict__ d_prior_b, long rows, int L, int HQ, int H, int N,
                              int softmax1, int tiles_per_wg) {
  constexpr int K = LPR * 8, RPW = 64 / LPR;
  constexpr int NWV = TAB ? 16 : 4;  // wavefronts of a workgroup
  __shared__ bf16_t stage[NWV][RPW * (K + 2)];
  extern __shared__ unsigned long long cwb_tab[];  // TAB: N x HQ, two's complement fixed point
  constexpr float TAB_SCALE = 1099511627776.f;  // 2^40: |sums| below 2^23, steps far below an fp32 gradient's own
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPR, rl = lane / LPR;
  const int NW = K + 1 + (softmax1 ? 1 : 0);
  // rows of this workgroup: [first, last); TAB: a run inside batch element blockIdx.y
  long first = (long)blockIdx.x * NWV * RPW, last = rows;
  int ntile = 1;
  if (TAB) {
    const long per_b = (long)L * HQ;
    first = blockIdx.y * per_b + (long)blockIdx.x * tiles_per_wg * NWV * RPW;
    last = (blockIdx.y + 1) * per_b;
    ntile = tiles_per_wg;
    for (int i = threadIdx.x; i < N * HQ; i += NWV * 64) cwb_tab[i] = 0ull;
    __syncthreads();
  }
  for (int tile = 0; tile < ntile; ++tile) {
    const long row0 = first + ((long)tile * NWV + wave) * RPW;
    const long row = row0 + rl;
    long nrow = last - row0;
    if (nrow > RPW) nrow = RPW;
    if (nrow <= 0) break;  // (the wavefront's rows only grow: nothing is left for it)
    {
      const int total = (int)nrow * NW;
      const bf16_t* src = d_weights + row0 * NW;
      for (int i = lane; i < total; i += 64) stage[wave][i] = src[i];
    }
    // same wavefront wrote the slice: stores and loads of one wavefront stay in program order
    const bool valid = row < last;
    float x[8], g[8];
    int cidx[8];
    float lse = HILS_NEG_INF, gl = 0.f, g0 = 0.f;
    int hq = 0;
    long b = 0;
    if (valid) {
      const uint4 v = *(const uint4*)(scores + row * K + sub * 8);
      unpack8(v, x);
      lse = lse_bf16 ? bf2f(((const bf16_t*)lse_swa)[row]) : ((const float*)lse_swa)[row];
      const bf16_t* st = stage[wave] + rl * NW;
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = bf2f(st[sub * 8 + e]);
      gl = bf2f(st[K]);
      if (softmax1) g0 = bf2f(st[K + 1]);
      if (prior_b) {
        hq = (int)(row % HQ);
        const long bt = row / HQ;
        b = bt / L;
        const int G = HQ / H;
        const int32_t* ip = indices + (bt * H + hq / G) * (long)K + sub * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          int c = ip[e];
          c = c < 0 ? 0 : c;
          cidx[e] = c;
          x[e] = bf2f(f2bf(x[e] + bf2f(f2bf(prior_b[(b * N + c) * (long)HQ + hq]))));
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) { x[e] = HILS_NEG_INF; g[e] = 0.f; }
    }
    float m = softmax1 ? fmaxf(lse, 0.f) : lse;
#pragma unroll
    for (int e = 0; e < 8; ++e) m = fmaxf(m, x[e]);
    if (LPR >= 2) m = fmaxf(m, __shfl_xor(m, 1, 64));
    if (LPR >= 4) m = fmaxf(m, __shfl_xor(m, 2, 64));
    if (LPR >= 8) m = fmaxf(m, __shfl_xor(m, 4, 64));
    const bool dead = !(m > HILS_NEG_INF);  // the forward gave NaN weights for this row
    float sum = 0.f, dot = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      x[e] = dead ? 0.f : __expf(x[e] - m);
      sum += x[e];
      dot += x[e] * g[e];
    }
    if (LPR >= 2) { sum += __shfl_xor(sum, 1, 64); dot += __shfl_xor(dot, 1, 64); }
    if (LPR >= 4) { sum += __shfl_xor(sum, 2, 64); dot += __shfl_xor(dot, 2, 64); }
    if (LPR >= 8) { sum += __shfl_xor(sum, 4, 64); dot += __shfl_xor(dot, 4, 64); }
    const float el = dead ? 0.f : __expf(lse - m);
    const float e0 = (softmax1 && !dead) ? __expf(0.f - m) : 0.f;
    sum += el + e0;
    dot += el * gl + e0 * g0;
    const float nan = __uint_as_float(0x7fc00000u);
    const float inv = dead ? nan : 1.f / sum;
    dot *= inv;  // sum_i y_i d_w_i
    if (valid) {
      float dl[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) dl[e] = dead ? nan : x[e] * inv * (g[e] - dot);
      uint4 out;
      out.x = pack_bf2(dl[0], dl[1]);
      out.y = pack_bf2(dl[2], dl[3]);
      out.z = pack_bf2(dl[4], dl[5]);
      out.w = pack_bf2(dl[6], dl[7]);
      *(uint4*)(d_scores + row * K + sub * 8) = out;
      if (d_prior_b && !dead) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (dl[e] != 0.f) {
            if (TAB) atomicAdd(&cwb_tab[cidx[e] * HQ + hq], (unsigned long long)(long long)(dl[e] * TAB_SCALE));
            else atomicAdd(d_prior_b + (b * N + cidx[e]) * (long)HQ + hq, dl[e]);
          }
      }
      if (d_lse && sub == 0) d_lse[row] = dead ? nan : el * inv * (gl - dot);
    }
  }
  if (TAB) {
    __syncthreads();
    float* dst = d_prior_b + (long)blockIdx.y * N * HQ;
    for (int i = threadIdx.x; i < N * HQ; i += NWV * 64) {
      const long long t = (long long)cwb_tab[i];
      if (t != 0) atomicAdd(dst + i, (float)((double)t * (1.0 / 1099511627776.0)));
    }
  }
}

extern "C" int hils_chunk_weights_bwd(const void* scores, const void* lse_swa, int lse_bf16,
                                      const float* prior_b, const int32_t* indices, const void* d_weights,
                                      void* d_scores, float* d_lse, float* d_prior_b, int B, int L, int HQ,
                                      int H, int N, int K, int softmax1, void* stream) {
  HILS_REQUIRE(scores && lse_swa && d_weights && d_scores, "hils_chunk_weights_bwd: null pointer");
  HILS_REQUIRE(!prior_b || indices, "hils_chunk_weights_bwd: prior_b needs indices");
  HILS_REQUIRE(!d_prior_b || prior_b, "hils_chunk_weights_bwd: d_prior_b needs prior_b");
  HILS_REQUIRE(B > 0 && L > 0 && HQ > 0 && H > 0 && HQ % H == 0, "hils_chunk_weights_bwd: bad head counts");
  HILS_REQUIRE(K >= 1 && K <= GL_MAXK, "hils_chunk_weights_bwd: K (%d) must be in 1..%d", K, GL_MAXK);
  const long rows = (long)B * L * HQ;
  const long nblk = (rows + 255) / 256;
  HILS_REQUIRE(nblk <= 2147483647L, "hils_chunk_weights_bwd: grid too large");
  if (K == 8 || K == 16 || K == 32 || K == 64) {
    const int rpw = 64 / (K / 8);
    const long nb = (rows + 4 * rpw - 1) / (4 * rpw);
    HILS_REQUIRE(nb <= 2147483647L, "hils_chunk_weights_bwd: grid too large");
    // with a bias gradient whose table fits the LDS: runs of rows per workgroup, about two workgroups a
    // compute unit, each run long enough that its adds outnumber the table it flushes
    const size_t tab_b = (size_t)N * HQ * sizeof(unsigned long long);
    if (d_prior_b && tab_b <= 48 * 1024) {
      const long tiles_b = ((long)L * HQ + 16 * rpw - 1) / (16 * rpw);  // 16-wavefront tiles of a batch element
      long segs = 2L * hils_device_cus() / B;
      if (segs < 1) segs = 1;
      if (segs > tiles_b) segs = tiles_b;
      const int tiles_per_wg = (int)((tiles_b + segs - 1) / segs);
      const dim3 grid((unsigned)((tiles_b + tiles_per_wg - 1) / tiles_per_wg), (unsigned)B);
      HILS_REQUIRE(B <= 65535, "hils_chunk_weights_bwd: batch too large for the grid");
#define GL_CALL_T(LPR_)                                                                                \
  hipLaunchKernelGGL((chunk_weights_bwd_rows_kernel<LPR_, true>), grid, dim3(1024), tab_b,             \
                     (hipStream_t)stream, (const bf16_t*)scores, lse_swa, lse_bf16, prior_b, indices,  \
                     (const bf16_t*)d_weights, (bf16_t*)d_scores, d_lse, d_prior_b, rows, L, HQ, H, N, \
                     softmax1, tiles_per_wg)
      if (K == 8) GL_CALL_T(1); else if (K == 16) GL_CALL_T(2); else if (K == 32) GL_CALL_T(4); else GL_CALL_T(8);
#undef GL_CALL_T
      HILS_CHECK_LAUNCH("hils_chunk_weights_bwd");
      return HILS_OK;
    }
#define GL_CALL(LPR_)                                                                                  \
  hipLaunchKernelGGL((chunk_weights_bwd_rows_kernel<LPR_, false>), dim3((unsigned)nb), dim3(256), 0,   \
                     (hipStream_t)stream, (const bf16_t*)scores, lse_swa, lse_bf16, prior_b, indices,  \
                     (const bf16_t*)d_weights, (bf16_t*)d_scores, d_lse, d_prior_b, rows, L, HQ, H, N, \
                     softmax1, 1)
    if (K == 8) GL_CALL(1); else if (K == 16) GL_CALL(2); else if (K == 32) GL_CALL(4); else GL_CALL(8);
#undef GL_CALL
    HILS_CHECK_LAUNCH("hils_chunk_weights_bwd");
    return HILS_OK;
  }
  hipLaunchKernelGGL(chunk_weights_bwd_kernel, dim3((unsigned)nblk), dim3(256), 0, (hipStream_t)stream,
                     (const bf16_t*)scores, lse_swa, lse_bf16, prior_b, indices, (const bf16_t*)d_weights,
                     (bf16_t*)d_scores, d_lse, d_prior_b, rows, L, HQ, H, N, K, softmax1);
  HILS_CHECK_LAUNCH("hils_chunk_weights_bwd");
  return HILS_OK;
}
