// Measurement aid: what a kernel that only loads reaches on this GPU, for the access patterns the
// decode kernels have.  The roofline fractions of the HBM-bound kernels are quoted against the
// published peak; these figures say how much of it any kernel can get.
#include "common.h"
#include "../../include/hils_amd.h"

typedef unsigned pr_u4 __attribute__((ext_vector_type(4)));

// pattern 0: every workgroup streams a contiguous share, four 16-byte loads per lane in flight
__global__ void __launch_bounds__(1024) probe_contiguous(const pr_u4* __restrict__ p, size_t n16, unsigned* sink) {
  const size_t per = n16 / gridDim.x;
  const pr_u4* b = p + per * blockIdx.x;
  pr_u4 acc = {0u, 0u, 0u, 0u};
  for (size_t i = threadIdx.x; i + 3 * 1024 < per; i += 4 * 1024) {
    pr_u4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(&b[i + (size_t)u * 1024]);
#pragma unroll
    for (int u = 0; u < 4; ++u) acc ^= v[u];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = 1u;  // keeps the loads alive
}

// pattern 1: the tensor as (tokens, 8 heads, 128) bf16; a workgroup reads one head's 256-byte rows
// (a 2 KiB stride) of its share of the tokens; all heads together read everything
__global__ void __launch_bounds__(1024) probe_rows(const pr_u4* __restrict__ p, size_t ntok, unsigned* sink) {
  const int h = blockIdx.x & 7;
  const size_t share = blockIdx.x >> 3, nshare = gridDim.x >> 3;
  const size_t per = ntok / nshare;
  const int sub = threadIdx.x >> 4, piece = threadIdx.x & 15;
  pr_u4 acc = {0u, 0u, 0u, 0u};
  for (size_t t = share * per + sub; t + 7 * 64 < (share + 1) * per; t += 8 * 64) {
    pr_u4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = p[((t + u * 64) * 8 + h) * 16 + piece];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = 1u;
}

extern "C" int hils_stream_probe(const void* buf, size_t bytes, int pattern, void* sink, void* stream) {
  HILS_REQUIRE(buf && sink, "hils_stream_probe: null pointer");
  HILS_REQUIRE(bytes >= ((size_t)64 << 20) && bytes % ((size_t)1 << 20) == 0,
               "hils_stream_probe: the buffer must be a multiple of 1 MiB, 64 MiB at least");
  HILS_REQUIRE(pattern == 0 || pattern == 1, "hils_stream_probe: pattern must be 0 or 1");
  const int wgs = 2 * hils_device_cus();
  if (pattern == 0)
    hipLaunchKernelGGL(probe_contiguous, dim3(wgs), dim3(1024), 0, (hipStream_t)stream, (const pr_u4*)buf, bytes / 16,
                       (unsigned*)sink);
  else
    hipLaunchKernelGGL(probe_rows, dim3(wgs & ~7), dim3(1024), 0, (hipStream_t)stream, (const pr_u4*)buf, bytes / 2048,
                       (unsigned*)sink);
  HILS_CHECK_LAUNCH("hils_stream_probe");
  return HILS_OK;
}
