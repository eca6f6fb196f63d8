// Decode sparse attention, one workgroup per (query, KV head) row and slot share: the kernel and its
// launcher around decode_rows_body (decode_rows_body.h).
#include "decode_rows_body.h"

template <int D, int NWAVE>
__global__ void __launch_bounds__(NWAVE * 64) __attribute__((amdgpu_waves_per_eu(2)))
sparse_attn_decode_rows_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                               const bf16_t* __restrict__ v, const bf16_t* __restrict__ weights,
                               const int32_t* __restrict__ indices, bf16_t* __restrict__ o,
                               float* __restrict__ partial, DrDims dm) {
  extern __shared__ __align__(16) char dr_dyn[];
  decode_rows_body<D, NWAVE>(q, k, v, weights, indices, o, partial, dm, dr_dyn, (int)blockIdx.x, (int)blockIdx.y,
                             (long)blockIdx.z);
}

// A workgroup of 8 (no split) or 4 wavefronts, DR_MAXSLOT slots per wavefront: K <= 128 covers
// every split the launcher picks.
bool hils_decode_rows_covers(int D, int Dv, int G, int K) {
  return D == Dv && (D == 64 || D == 128) && G >= 1 && G <= DR_NH && K <= 4 * DR_MAXSLOT;
}

template <int D, int NWAVE>
static int dr_launch(dim3 grid, hipStream_t st, const void* q, const void* k, const void* v, const void* weights,
                     const int32_t* indices, void* o, void* workspace, const DrDims& dm) {
  const size_t smem = dr_smem_bytes(D, dm.G, NWAVE);
  auto kern = sparse_attn_decode_rows_kernel<D, NWAVE>;
  static HilsLdsReserve reserved;  // per instantiation
  if (int rc = hils_reserve_lds(&reserved, (const void*)kern, smem, "hils_sparse_attn_fwd (decode)")) return rc;
  hipLaunchKernelGGL(kern, grid, dim3(NWAVE * 64), smem, st, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v,
                     (const bf16_t*)weights, indices, (bf16_t*)o, (float*)workspace, dm);
  return HILS_OK;
}

int hils_sparse_attn_decode_rows(const void* q, const void* k, const void* v, const void* weights,
                                 const int32_t* indices, void* o, void* workspace, int nsplit,
                                 int B, int L, int Lkv, int HQ, int H, int D, int K, int NW,
                                 float sm_scale, int mask_last, const int32_t* page_table, int max_pages,
                                 int num_pages, hipStream_t st) {
  const int G = HQ / H;
  DrDims dm{L, Lkv, HQ, H, G, K, NW, page_table ? max_pages : Lkv / DR_S, nsplit, mask_last, sm_scale,
            page_table, max_pages, num_pages};
  dim3 grid(nsplit, H, (unsigned)((long)B * L));
  // no split and many slots: one workgroup of 8 wavefronts per (query, KV head)
  const bool wide = nsplit == 1 && K >= 16;
  if (D == 64) {
    return wide ? dr_launch<64, 8>(grid, st, q, k, v, weights, indices, o, workspace, dm)
                : dr_launch<64, 4>(grid, st, q, k, v, weights, indices, o, workspace, dm);
  }
  return wide ? dr_launch<128, 8>(grid, st, q, k, v, weights, indices, o, workspace, dm)
              : dr_launch<128, 4>(grid, st, q, k, v, weights, indices, o, workspace, dm);
}
