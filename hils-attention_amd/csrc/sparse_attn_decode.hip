// Sparse attention forward for decode-sized query counts (HBM-bandwidth-bound gather).
//
// A (batch, query, KV head) reads K*64 tokens of K and V exactly once; nothing is reused,
// so the kernel is organised for memory-level parallelism: the K selected slots of a row
// are split over `nsplit` workgroups of 8 wavefronts, one slot (chunk) per wavefront at a
// time, every load a 16-byte lane load along a token row.  Scores S^T = K q^T use one
// 16x16x32 bf16 MFMA chain per 16 tokens (the G query heads are the first G columns), the
// per-chunk softmax runs in the accumulator registers, and P V is a vector-ALU pass over
// the row-major V chunk.  Partial outputs of the splits go to an fp32 scratch and are
// summed by a second small kernel (skipped when nsplit == 1).
#include "common.h"
#include "../../include/hils_amd.h"

#define DE_THREADS 512
#define DE_WAVES (DE_THREADS / 64)
#define DE_S 64

struct DeDims {
  int L, Lkv, HQ, H, G, K, NW, nchunk, nsplit, mask_last;
  float sm_scale;
};

template <int D, int DV>
__global__ void __launch_bounds__(DE_THREADS)
sparse_attn_decode_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                          const bf16_t* __restrict__ v, const bf16_t* __restrict__ weights,
                          const int32_t* __restrict__ indices, bf16_t* __restrict__ o,
                          float* __restrict__ partial, DeDims dm) {
  constexpr int KS = D / 32;
  constexpr int LR = DV / 8;        // lanes that cover one V row with 16-byte loads
  constexpr int TPI = 64 / LR;      // tokens per load instruction
  extern __shared__ float de_smem[];
  float(*p_s)[DE_S][16] = (float(*)[DE_S][16])de_smem;  // [wave][token][g padded to 16]
  float* o_s = de_smem + DE_WAVES * DE_S * 16;          // [wave][G][DV] partial outputs

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int split = blockIdx.x, hk = blockIdx.y;
  const long bt = blockIdx.z;  // b * L + t
  const long b = bt / dm.L;
  const int G = dm.G, K = dm.K;

  // B operand: the G query rows of this KV head (columns r < G), zero elsewhere
  bf16x8_t bq[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    uint4 x = make_uint4(0, 0, 0, 0);
    if (r < G) x = *(const uint4*)(q + (bt * dm.HQ + hk * G + r) * (long)D + ks * 32 + j * 8);
    bq[ks] = *(bf16x8_t*)&x;
  }
  const float c2 = dm.sm_scale * HILS_LOG2E;
  float oacc[16][8];  // [g][8 dv of this lane's column group] over this lane's tokens
#pragma unroll
  for (int g = 0; g < 16; ++g)
#pragma unroll
    for (int e = 0; e < 8; ++e) oacc[g][e] = 0.f;

  const int per_split = (K + dm.nsplit - 1) / dm.nsplit;
  const int s_begin = split * per_split;
  const int s_end = (s_begin + per_split < K) ? s_begin + per_split : K;
  for (int slot = s_begin + wave; slot < s_end; slot += DE_WAVES) {
    const int c = indices[(bt * dm.H + hk) * (long)K + slot];
    if (c < 0 || c >= dm.nchunk) continue;
    const bf16_t* kbase = k + ((b * dm.Lkv + (long)c * DE_S + r) * dm.H + hk) * D + j * 8;
    f32x4_t st[4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      st[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const uint4 x = *(const uint4*)(kbase + (long)mt * 16 * dm.H * D + ks * 32);
        st[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&x, bq[ks], st[mt], 0, 0, 0);
      }
    }
    // V rows of the chunk: issue the loads before the softmax arithmetic
    const bf16_t* vbase = v + ((b * dm.Lkv + (long)c * DE_S) * dm.H + hk) * DV;
    uint4 vr[DE_S / TPI];
#pragma unroll
    for (int it = 0; it < DE_S / TPI; ++it) {
      const int tok = it * TPI + lane / LR;
      vr[it] = *(const uint4*)(vbase + (long)tok * dm.H * DV + (lane % LR) * 8);
    }
    float wr = 0.f;
    if (r < G) wr = bf2f(weights[(bt * dm.HQ + hk * G + r) * (long)dm.NW + slot]);
    float m = HILS_NEG_INF;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int tok = mt * 16 + j * 4 + i;
        if (dm.mask_last && tok == DE_S - 1) st[mt][i] = HILS_NEG_INF;
        m = fmaxf(m, st[mt][i]);
      }
    m = fmaxf(m, __shfl_xor(m, 16, 64));
    m = fmaxf(m, __shfl_xor(m, 32, 64));
    const float mc = m * c2;
    float sum = 0.f;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float e = __builtin_amdgcn_exp2f(st[mt][i] * c2 - mc);
        st[mt][i] = e;
        sum += e;
      }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    const float f = wr / sum;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) p_s[wave][mt * 16 + j * 4 + i][r] = st[mt][i] * f;
    // P V on the vector ALU: this lane owns 8 output columns and every TPI-th token
#pragma unroll
    for (int it = 0; it < DE_S / TPI; ++it) {
      const int tok = it * TPI + lane / LR;
      float vf[8];
      unpack8(vr[it], vf);
      const float* pr = p_s[wave][tok];
#pragma unroll
      for (int g = 0; g < 16; ++g) {
        if (g < G) {
          const float pg = pr[g];
#pragma unroll
          for (int e = 0; e < 8; ++e) oacc[g][e] = fmaf(pg, vf[e], oacc[g][e]);
        }
      }
    }
  }
  // sum over the token groups of the wavefront, then over the wavefronts of the workgroup
#pragma unroll
  for (int g = 0; g < 16; ++g) {
    if (g < G) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float x = oacc[g][e];
#pragma unroll
        for (int off = LR; off < 64; off <<= 1) x += __shfl_xor(x, off, 64);
        if (lane < LR) o_s[((size_t)wave * dm.G + g) * DV + lane * 8 + e] = x;
      }
    }
  }
  __syncthreads();
  for (int i = tid; i < G * DV; i += DE_THREADS) {
    const int g = i / DV, dv = i - g * DV;
    float x = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < DE_WAVES; ++w2) x += o_s[((size_t)w2 * dm.G + g) * DV + dv];
    if (dm.nsplit == 1) o[(bt * dm.HQ + hk * G + g) * (long)DV + dv] = f2bf(x);
    else partial[((bt * dm.HQ + hk * G + g) * (long)dm.nsplit + split) * DV + dv] = x;
  }
}

__global__ void decode_reduce_kernel(const float* __restrict__ partial, bf16_t* __restrict__ o,
                                     long rows, int Dv, int nsplit) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * Dv) return;
  const long row = i / Dv;
  const int dv = (int)(i - row * Dv);
  float x = 0.f;
  for (int s = 0; s < nsplit; ++s) x += partial[(row * nsplit + s) * Dv + dv];
  o[i] = f2bf(x);
}

static int de_pick_nsplit(int B, int L, int H, int K) {
  const int cus = hils_device_cus();
  const long rows = (long)B * L * H;
  // one workgroup per row and whole rounds of rows over the compute units: no split, no partial sums
  if (K >= 16 && rows >= cus && (rows % cus == 0 || rows >= 8L * cus)) return 1;
  int nsplit = 1;
  // aim for >= 4 workgroups per CU, at least one slot per wavefront
  while (rows * nsplit < 4L * cus && (K + nsplit * 2 - 1) / (nsplit * 2) >= DE_WAVES / 2 && nsplit < 16) nsplit *= 2;
  return nsplit;
}

bool hils_decode_covers(int L, int HQ, int H, int D, int Dv, int S, int q_block, int WH, float sm_n,
                        const float* slope, const float* lse) {
  if (H <= 0 || HQ % H != 0) return false;
  const int G = HQ / H;
  return S == DE_S && (D == 64 || D == 128) && (Dv == 64 || Dv == 128) && G <= 16 && q_block == 1 &&
         WH == HQ && sm_n == 0.f && slope == nullptr && lse == nullptr && L < 64;
}

size_t hils_decode_workspace_bytes(int B, int L, int HQ, int H, int Dv, int K) {
  const int nsplit = de_pick_nsplit(B, L, H, K);
  return nsplit == 1 ? 0 : (size_t)B * L * HQ * nsplit * Dv * sizeof(float);
}

bool hils_decode_rows_covers(int D, int Dv, int G, int K);
int hils_sparse_attn_decode_rows(const void* q, const void* k, const void* v, const void* weights,
                                  const int32_t* indices, void* o, void* workspace, int nsplit,
                                  int B, int L, int Lkv, int HQ, int H, int D, int K, int NW,
                                  float sm_scale, int mask_last, const int32_t* page_table, int max_pages,
                                  int num_pages, hipStream_t st);

int hils_sparse_attn_decode(const void* q, const void* k, const void* v, const void* weights,
                            const int32_t* indices, void* o, void* workspace, int B, int L, int Lkv,
                            int HQ, int H, int D, int Dv, int K, int NW, float sm_scale,
                            int mask_last, void* stream) {
  int nsplit = workspace ? de_pick_nsplit(B, L, H, K) : 1;
  if ((long)B * L > 65535L * 32768L || H > 65535) {
    hils_set_error("hils_sparse_attn_fwd: grid too large");
    return HILS_ERR_ARG;
  }
  DeDims dm{L, Lkv, HQ, H, HQ / H, K, NW, Lkv / DE_S, nsplit, mask_last, sm_scale};
  dim3 grid(nsplit, H, (unsigned)((long)B * L));
  hipStream_t st = (hipStream_t)stream;
  if (hils_decode_rows_covers(D, Dv, HQ / H, K)) {
    if (int rc = hils_sparse_attn_decode_rows(q, k, v, weights, indices, o, workspace, nsplit, B, L, Lkv, HQ, H, D,
                                              K, NW, sm_scale, mask_last, nullptr, 0, 0, st))
      return rc;
  } else {
  const size_t smem = ((size_t)DE_WAVES * DE_S * 16 + (size_t)DE_WAVES * dm.G * Dv) * sizeof(float);
#define DE_CALL(D_, DV_)                                                                           \
  do {                                                                                             \
    auto kern = sparse_attn_decode_kernel<D_, DV_>;                                                \
    if (smem > 64 * 1024)                                                                          \
      (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,     \
                                (int)smem);                                                        \
    hipLaunchKernelGGL(kern, grid, dim3(DE_THREADS), smem, st, (const bf16_t*)q, (const bf16_t*)k, \
                       (const bf16_t*)v, (const bf16_t*)weights, indices, (bf16_t*)o,              \
                       (float*)workspace, dm);                                                     \
  } while (0)
  if (D == 64 && Dv == 64) DE_CALL(64, 64);
  else if (D == 128 && Dv == 128) DE_CALL(128, 128);
  else if (D == 64 && Dv == 128) DE_CALL(64, 128);
  else DE_CALL(128, 64);
#undef DE_CALL
  }
  if (nsplit > 1) {
    const long rows = (long)B * L * HQ;
    const long n = rows * Dv;
    hipLaunchKernelGGL(decode_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                       (const float*)workspace, (bf16_t*)o, rows, Dv, nsplit);
  }
  return HILS_OK;
}

// Decode over a paged cache (page = chunk = 64 tokens): k_pages, v_pages (num_pages, H, 64, D) bf16;
// page_table (B, max_pages) int32, chunk c of batch element b -> page id (negative = unmapped).
extern "C" size_t hils_sparse_attn_decode_paged_workspace(int B, int L, int HQ, int H, int D, int K) {
  return hils_decode_workspace_bytes(B, L, HQ, H, D, K);
}

extern "C" int hils_sparse_attn_decode_paged(const void* q, const void* k_pages, const void* v_pages,
                                             const int32_t* page_table, const void* weights,
                                             const int32_t* indices, void* o, void* workspace,
                                             size_t workspace_bytes, int B, int L,
                                             int HQ, int H, int D, int K, int NW, int max_pages, int num_pages,
                                             float sm_scale, int mask_last, void* stream) {
  HILS_REQUIRE(q && k_pages && v_pages && page_table && weights && indices && o,
               "hils_sparse_attn_decode_paged: null pointer");
  HILS_REQUIRE(!workspace || workspace_bytes >= hils_decode_workspace_bytes(B, L, HQ, H, D, K),
               "hils_sparse_attn_decode_paged: workspace of %zu bytes is shorter than the %zu bytes "
               "hils_sparse_attn_decode_paged_workspace returns for this shape", workspace_bytes,
               hils_decode_workspace_bytes(B, L, HQ, H, D, K));
  HILS_REQUIRE(B > 0 && L > 0 && HQ > 0 && H > 0 && HQ % H == 0 && K > 0 && NW >= K && max_pages > 0 && num_pages > 0,
               "hils_sparse_attn_decode_paged: bad sizes");
  HILS_REQUIRE(hils_decode_rows_covers(D, D, HQ / H, K),
               "hils_sparse_attn_decode_paged: needs D = Dv in {64, 128}, at most 16 query heads per KV head, K <= 128");
  HILS_REQUIRE((long)B * L <= 65535L * 32768L && H <= 65535, "hils_sparse_attn_decode_paged: grid too large");
  const int nsplit = workspace ? de_pick_nsplit(B, L, H, K) : 1;
  hipStream_t st = (hipStream_t)stream;
  if (int rc = hils_sparse_attn_decode_rows(q, k_pages, v_pages, weights, indices, o, workspace, nsplit, B, L, 0, HQ,
                                            H, D, K, NW, sm_scale, mask_last, page_table, max_pages, num_pages, st))
    return rc;
  if (nsplit > 1) {
    const long rows = (long)B * L * HQ;
    const long n = rows * D;
    hipLaunchKernelGGL(decode_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                       (const float*)workspace, (bf16_t*)o, rows, D, nsplit);
  }
  HILS_CHECK_LAUNCH("hils_sparse_attn_decode_paged");
  return HILS_OK;
}
