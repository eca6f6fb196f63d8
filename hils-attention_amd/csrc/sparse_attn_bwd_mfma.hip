// Sparse attention backward on bf16 MFMA (chunk size 64, D and Dv in {64, 128}).
//
// dK and dV of a chunk are sums over every (query, head) row that selected the chunk, so
// that side is computed chunk-major: an inverse index (for each (batch, KV head, chunk) the
// list of (query, slot) pairs that hold it) is built by a counting sort, then one workgroup
// per chunk streams its rows in tiles of 16, recomputes P and dS with the scores in the
// orientation rows x tokens, and keeps dK, dV of the chunk in MFMA accumulators: no atomics,
// one write per element.
//
//   S  = Q K^T            (16 rows x 16 tokens per wavefront, 16x16x32 MFMA over d)
//   dP = dO V^T           (same shape, 16x16x32 MFMA over dv)
//   P  = exp2(S c2 - lse2),  delta = sum_tokens P dP,  dS = w P (dP - delta)
//   dV += (w P)^T dO      (16 tokens x Dv, 16x16x16 MFMA over the 16 rows)
//   dK += scale dS^T Q    (16 tokens x D,  16x16x16 MFMA over the 16 rows)
//
// An accumulator-layout tile (lane: column = token, registers = rows 4j..4j+3) is, two row tiles
// side by side, exactly the A operand of the 16x16x32 MFMA with the roles (row m = token, k = 32
// rows), so P and dS feed the second pair of products without leaving registers.  Their B operands
// (k = rows, n = feature) are columns of the gathered Q and dO rows: the workgroup stages the rows
// row-major in LDS once per round for all four wavefronts (16 tokens each), and the column reads
// are the hardware's transposing LDS loads (a 16-lane group fetches a 4 x 16 block and every lane
// receives one column of it).
#include "decode_rows.h"
#include "../../include/hils_amd.h"

#define BW_S 64
typedef short bw_s4 __attribute__((ext_vector_type(4)));
typedef unsigned bw_u4 __attribute__((ext_vector_type(4)));  // a 16-byte piece as a register value

__global__ void bw_fill_int_kernel(int* p, int value, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = value;
}

// ---------------------------------------------------------------------------
// Inverse index: pairs (query << 8 | slot) grouped by (batch, KV head, chunk).
// ---------------------------------------------------------------------------
// The index entries (query t_lo + r, slot s) of one KV head for the queries of a segment, walked by a
// workgroup of 1024: thread tid takes entries tid, tid + 1024, ... of the segment's rows x K entries
// (consecutive threads read consecutive slots of a row).  (r, s) advance by (1024 / K, 1024 % K) per
// step, so that nothing is divided inside the loop, and four loads are in flight per thread (a
// clamped row is loaded for a step past the end and skipped).  f(t, slot, chunk).
template <class F>
__device__ __forceinline__ void bw_walk_indices(const int32_t* __restrict__ seg0, int t_lo, int rows, int H, int K,
                                                F f) {
  const int qK = 1024 / K, rK = 1024 % K;
  int r = (int)threadIdx.x / K, sl = (int)threadIdx.x - r * K;
  const long rstride = (long)H * K;
  while (r < rows) {
    int rr[4], ss[4], cc[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      rr[u] = r;
      ss[u] = sl;
      sl += rK;
      r += qK;
      if (sl >= K) { sl -= K; ++r; }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) cc[u] = seg0[(long)(rr[u] < rows ? rr[u] : rows - 1) * rstride + ss[u]];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (rr[u] < rows) f(t_lo + rr[u], ss[u], cc[u]);
  }
}

// counts[(b*H + h) * nchunk + c] = number of valid entries equal to c; one workgroup per
// (batch, KV head, segment of queries), LDS histogram first.
__global__ void __launch_bounds__(1024)
bw_count_kernel(const int32_t* __restrict__ indices, int* __restrict__ counts, int L, int H, int K,
                int nchunk, int seg_len) {
  extern __shared__ int hist[];
  const int h = blockIdx.y;
  const long b = blockIdx.z;
  const int t_lo = blockIdx.x * seg_len;
  const int t_hi = (t_lo + seg_len < L) ? t_lo + seg_len : L;
  for (int i = threadIdx.x; i < nchunk; i += 1024) hist[i] = 0;
  __syncthreads();
  const int32_t* seg0 = indices + ((b * L + t_lo) * H + h) * (long)K;
  bw_walk_indices(seg0, t_lo, t_hi - t_lo, H, K, [&](int, int, int c) {
    if (c >= 0 && c < nchunk) atomicAdd(&hist[c], 1);
  });
  __syncthreads();
  int* out = counts + (b * H + h) * (long)nchunk;
  for (int i = threadIdx.x; i < nchunk; i += 1024)
    if (hist[i]) atomicAdd(&out[i], hist[i]);
}

// exclusive scan of n counts into offsets[0..n] (offsets[n] = total); one workgroup
__global__ void __launch_bounds__(1024)
bw_scan_kernel(const int* __restrict__ counts, int* __restrict__ offsets, int* __restrict__ cursor, long n) {
  __shared__ int wsum[16];
  __shared__ int carry_s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (long base = 0; base < n; base += 1024) {
    const long i = base + tid;
    const int x = (i < n) ? counts[i] : 0;
    int incl = x;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int y = __shfl_up(incl, o, 64);
      if (lane >= o) incl += y;
    }
    if (lane == 63) wsum[wave] = incl;
    __syncthreads();
    int pre = carry_s;
    for (int w = 0; w < wave; ++w) pre += wsum[w];
    if (i < n) {
      offsets[i] = pre + incl - x;
      cursor[i] = pre + incl - x;
    }
    __syncthreads();
    if (tid == 1023) carry_s = pre + incl;
    __syncthreads();
  }
  if (tid == 0) offsets[n] = carry_s;
}

// pairs grouped by (b,h,c): a workgroup histograms its segment of queries in LDS, reserves one
// range per chunk with a single global atomic, and scatters (t << 8 | slot) inside its ranges
__global__ void __launch_bounds__(1024)
bw_scatter_kernel(const int32_t* __restrict__ indices, int* __restrict__ cursor,
                  uint32_t* __restrict__ pairs, int L, int H, int K, int nchunk, int seg_len) {
  extern __shared__ int pos[];  // nchunk: count -> next free position
  const int h = blockIdx.y;
  const long b = blockIdx.z;
  const int t_lo = blockIdx.x * seg_len;
  const int t_hi = (t_lo + seg_len < L) ? t_lo + seg_len : L;
  int* cur = cursor + (b * H + h) * (long)nchunk;
  for (int i = threadIdx.x; i < nchunk; i += 1024) pos[i] = 0;
  __syncthreads();
  const int32_t* seg0 = indices + ((b * L + t_lo) * H + h) * (long)K;
  bw_walk_indices(seg0, t_lo, t_hi - t_lo, H, K, [&](int, int, int c) {
    if (c >= 0 && c < nchunk) atomicAdd(&pos[c], 1);
  });
  __syncthreads();
  for (int i = threadIdx.x; i < nchunk; i += 1024) {
    const int cnt = pos[i];
    pos[i] = cnt ? atomicAdd(&cur[i], cnt) : 0;
  }
  __syncthreads();
  bw_walk_indices(seg0, t_lo, t_hi - t_lo, H, K, [&](int t, int slot, int c) {
    if (c >= 0 && c < nchunk) pairs[atomicAdd(&pos[c], 1)] = ((uint32_t)t << 8) | (uint32_t)slot;
  });
}

// ---------------------------------------------------------------------------
// dK, dV: one workgroup of four wavefronts per (batch, KV head, chunk)
// ---------------------------------------------------------------------------
struct BwDims {
  int L, Lkv, HQ, H, K, NW, nchunk, mask_last;
  float sm_scale;
  int out16;  // dk, dv are bf16 tensors that this kernel overwrites (else fp32, added to)
  int B;
  const float* slope;  // per query head, or null: scores lose slope * max(0, 62 - token) before the softmax
};

template <int D, int DV, int G>
// (64-wide heads fit the register budget of four wavefronts per SIMD: four workgroups per compute
// unit, whose two 19 KiB staging buffers each just fit the LDS)
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((D <= 64 && DV <= 64) ? 4 : 2)))
bw_dkdv_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
               const bf16_t* __restrict__ weights, const float* __restrict__ lse,
               const float* __restrict__ delta, const bf16_t* __restrict__ d_o,
               const int* __restrict__ offsets, const uint32_t* __restrict__ pairs,
               void* __restrict__ dk_out, void* __restrict__ dv_out, BwDims dm) {
  // delta (B,L,HQ,NW) fp32: sum_tokens P dP of every (row, slot), written by the dQ kernel
  constexpr int KS = D / 32, VS = DV / 32;    // k-steps of the two 16x16x32 products
  constexpr int DT = D / 16, VT = DV / 16;    // 16-wide column tiles of dK, dV
  constexpr int DMAX = D > DV ? D : DV;
  constexpr int NSUB = 256 / DMAX;            // 16-row tiles staged per round (4 or 2)
  constexpr int ROWS = 16 * NSUB;             // rows per round
  constexpr int PPR = ROWS / G;               // pairs per round
  constexpr int QROW = D * 2 + 16;            // staging: padded row (bytes)
  constexpr int OROW = DV * 2 + 16;
  constexpr int BUF = ROWS * (QROW + OROW) + 3 * ROWS * 4;  // one staging buffer (bytes)
  extern __shared__ __attribute__((aligned(16))) char bw_smem[];  // two staging buffers
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, j = lane >> 4;
  // XCD-aware order: hardware hands consecutive workgroup ids to the 8 XCDs in turn; an XCD works
  // through the chunks of one (batch, KV head) at a time, so the query and dO rows that its
  // workgroups gather (the same L rows for every chunk of the head) stay in its L2.
  const int units = dm.H * dm.B;
  const int slot = (int)(blockIdx.x / 8);
  const int unit = (slot / dm.nchunk) * 8 + (int)(blockIdx.x % 8);
  if (unit >= units) return;
  const int c = slot % dm.nchunk, hk = unit % dm.H;
  const long b = unit / dm.H;
  const long cell = (b * dm.H + hk) * (long)dm.nchunk + c;
  const int p_lo = offsets[cell], p_hi = offsets[cell + 1];
  if (p_lo == p_hi) {
    if (dm.out16) {  // nobody selected the chunk: its gradients are zero
      bf16_t* dk16 = (bf16_t*)dk_out + ((b * dm.Lkv + (long)c * BW_S) * dm.H + hk) * D;
      bf16_t* dv16 = (bf16_t*)dv_out + ((b * dm.Lkv + (long)c * BW_S) * dm.H + hk) * DV;
      for (int i = tid; i < BW_S * (D / 8); i += 256)
        *(uint4*)(dk16 + (long)(i / (D / 8)) * dm.H * D + (i % (D / 8)) * 8) = make_uint4(0, 0, 0, 0);
      for (int i = tid; i < BW_S * (DV / 8); i += 256)
        *(uint4*)(dv16 + (long)(i / (DV / 8)) * dm.H * DV + (i % (DV / 8)) * 8) = make_uint4(0, 0, 0, 0);
    }
    return;
  }

  // this wavefront's 16 tokens of the chunk as B operands (k = feature, n = token)
  const long tok = (long)c * BW_S + wave * 16 + col;
  uint4 kb[KS], vb[VS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    kb[ks] = *(const uint4*)(k + ((b * dm.Lkv + tok) * dm.H + hk) * D + ks * 32 + j * 8);
#pragma unroll
  for (int ks = 0; ks < VS; ++ks)
    vb[ks] = *(const uint4*)(v + ((b * dm.Lkv + tok) * dm.H + hk) * DV + ks * 32 + j * 8);
  const bool masked_col = dm.mask_last && wave == 3 && col == 15;  // token 63 of the chunk
  // distance penalty of this lane's token for its four accumulator rows (16 % G == 0: the head of
  // row 4j + i is the same in every 16-row tile)
  float pen[4] = {0.f, 0.f, 0.f, 0.f};
  if (dm.slope) {
    const int dist = BW_S - 2 - (wave * 16 + col);
#pragma unroll
    for (int i = 0; i < 4; ++i) pen[i] = dm.slope[hk * G + (4 * j + i) % G] * (float)(dist > 0 ? dist : 0);
  }

  f32x4_t acc_k[DT], acc_v[VT];
#pragma unroll
  for (int t = 0; t < DT; ++t) acc_k[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t = 0; t < VT; ++t) acc_v[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  const float c2 = dm.sm_scale * HILS_LOG2E;

  // Staging roles: thread -> (row, 16-byte piece), NQ (NO) items per thread and round.
  constexpr int QPP = D / 8, OPP = DV / 8;
  constexpr int NQ = ROWS * QPP / 256, NO = ROWS * OPP / 256;
  constexpr int QRS = 256 / QPP, ORS = 256 / OPP;  // row step between a thread's items
  const int q_row0 = tid / QPP, q_pc = tid % QPP;
  const int o_row0 = tid / OPP, o_pc = tid % OPP;
  const int npair = p_hi - p_lo;
  const int nround = (npair + PPR - 1) / PPR;

  // Loads below are unconditional from clamped addresses, the pair entries as relaxed atomic
  // loads: a load inside a branch is waited for inside it, and a plain load may be moved next to
  // its use; either way the gathers of a round would queue up behind one another's latency.
  auto pair_ok = [&](int round, int row) __attribute__((always_inline)) -> bool {  // false for padding rows
    return row < ROWS && round * PPR + row / G < npair;
  };
  auto pair_of = [&](int round, int row) __attribute__((always_inline)) -> uint32_t {  // pair of a round's row (pair 0 of the chunk for padding rows)
    const int pi = round * PPR + row / G;
    return __hip_atomic_load(pairs + p_lo + (pair_ok(round, row) ? pi : 0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  uint32_t pk_q[NQ], pk_o[NO], pk_r;
  bw_u4 xq[NQ], xo[NO];
  float r_l2 = INFINITY, r_dl = 0.f;
  bf16_t r_wb = 0;
  bool r_ok = false;
  auto load_pairs = [&](int round) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < NQ; ++u) pk_q[u] = pair_of(round, q_row0 + u * QRS);
#pragma unroll
    for (int u = 0; u < NO; ++u) pk_o[u] = pair_of(round, o_row0 + u * ORS);
    pk_r = pair_of(round, tid);
  };
  auto fetch = [&](int round) __attribute__((always_inline)) {  // gathers of `round`, whose pairs load_pairs(round) fetched
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      // padding rows read the row of the chunk's first pair (finite values): their P is 0, so they add nothing
      xq[u] = *(const bw_u4*)(q + ((b * dm.L + (pk_q[u] >> 8)) * (long)dm.HQ + hk * G + (q_row0 + u * QRS) % G) * D + q_pc * 8);
    }
#pragma unroll
    for (int u = 0; u < NO; ++u) {
      xo[u] = *(const bw_u4*)(d_o + ((b * dm.L + (pk_o[u] >> 8)) * (long)dm.HQ + hk * G + (o_row0 + u * ORS) % G) * DV + o_pc * 8);
    }
    {
      // raw values; what a padding row gets instead is decided where they are staged, so that
      // nothing here has to wait for a load
      r_ok = pair_ok(round, tid);
      const uint32_t pk = pk_r;
      const long rowi = (b * dm.L + (pk >> 8)) * (long)dm.HQ + hk * G + tid % G;
      r_l2 = lse[rowi * dm.K + (pk & 255)];
      r_wb = weights[rowi * dm.NW + (pk & 255)];
      r_dl = delta[rowi * dm.NW + (pk & 255)];
    }
  };
  // staging of the gathered rows of a round (in registers since fetch(round)) into buffer `buf`
  auto stage = [&](int buf) __attribute__((always_inline)) {
    char* q_rm = bw_smem + buf * BUF;       // ROWS x QROW
    char* o_rm = q_rm + ROWS * QROW;        // ROWS x OROW
    float* row_lse = (float*)(o_rm + ROWS * OROW);
    float* row_w = row_lse + ROWS;
    float* row_delta = row_w + ROWS;
#pragma unroll
    for (int u = 0; u < NQ; ++u) *(bw_u4*)(q_rm + (q_row0 + u * QRS) * QROW + q_pc * 16) = xq[u];
#pragma unroll
    for (int u = 0; u < NO; ++u) *(bw_u4*)(o_rm + (o_row0 + u * ORS) * OROW + o_pc * 16) = xo[u];
    if (tid < ROWS) {  // padding rows and empty slots: P = 0
      row_lse[tid] = (r_ok && r_l2 != HILS_NEG_INF) ? r_l2 : INFINITY;
      row_w[tid] = r_ok ? bf2f(r_wb) : 0.f;
      row_delta[tid] = r_ok ? r_dl : 0.f;
    }
  };
  // one column-read of a staged tile: rows r0 + 4j .. r0 + 4j + 3 of columns c0 .. c0 + 15, this
  // lane's column.  (Transposing load: lane l of a 16-lane group addresses row l/4, columns
  // 4*(l%4) .. +3 of the 4 x 16 block and receives column l of it.)
  typedef short bw_tr4 __attribute__((ext_vector_type(4)));
  auto col_read = [&](const char* base, int rowb, int r0, int c0) __attribute__((always_inline)) -> uint2 {
    const char* p = base + (r0 + 4 * j + (col >> 2)) * rowb + (c0 + 4 * (col & 3)) * 2;
    const bw_tr4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) bw_tr4*)p);
    return __builtin_bit_cast(uint2, v);
  };
  load_pairs(0);
  fetch(0);
  load_pairs(1);
  stage(0);
  if (nround > 1) {
    fetch(1);
    load_pairs(2);
  }
  lds_barrier();

  for (int round = 0; round < nround; ++round) {
    const char* q_rm = bw_smem + (round & 1) * BUF;
    const char* o_rm = q_rm + ROWS * QROW;
    const float* row_lse = (const float*)(o_rm + ROWS * OROW);
    const float* row_w = row_lse + ROWS;
    const float* row_delta = row_w + ROWS;
    const int rows_here = ((npair - round * PPR < PPR) ? npair - round * PPR : PPR) * G;
    // two 16-row tiles at a time: their P and dS, side by side, are the A operands (m = token,
    // k = 32 rows) of one 16x16x32 product per column tile; k index 8j + e stands for row
    // 4j + e of the first tile (e < 4) or row 4j + e - 4 of the second
#pragma unroll
    for (int sub = 0; sub < NSUB; sub += 2) {
      if (sub * 16 < rows_here) {
        uint2 xp[2], xds[2];
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          const int sb = sub + h2;
          // ---- S and dP of 16 rows x this wavefront's 16 tokens
          f32x4_t s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const uint4 a = *(const uint4*)(q_rm + (sb * 16 + col) * QROW + (ks * 32 + j * 8) * 2);
            s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&a, *(const bf16x8_t*)&kb[ks], s, 0, 0, 0);
          }
#pragma unroll
          for (int ks = 0; ks < VS; ++ks) {
            const uint4 a = *(const uint4*)(o_rm + (sb * 16 + col) * OROW + (ks * 32 + j * 8) * 2);
            dp = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&a, *(const bf16x8_t*)&vb[ks], dp, 0, 0, 0);
          }
          // accumulator layout: column = token `col`, registers = rows 4j..4j+3
          float pw[4], ds[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int r = sb * 16 + 4 * j + i;
            float pv = __builtin_amdgcn_exp2f((s[i] - pen[i]) * c2 - row_lse[r]);
            if (masked_col) pv = 0.f;
            pw[i] = row_w[r] * pv;
            ds[i] = pw[i] * (dp[i] - row_delta[r]);
          }
          xp[h2].x = pack_bf2(pw[0], pw[1]);
          xp[h2].y = pack_bf2(pw[2], pw[3]);
          xds[h2].x = pack_bf2(ds[0], ds[1]);
          xds[h2].y = pack_bf2(ds[2], ds[3]);
        }
        const uint4 a_p = make_uint4(xp[0].x, xp[0].y, xp[1].x, xp[1].y);
        const uint4 a_ds = make_uint4(xds[0].x, xds[0].y, xds[1].x, xds[1].y);
        // ---- dK += dS^T Q, dV += (wP)^T dO: contraction over the 32 rows
#pragma unroll
        for (int t = 0; t < DT; ++t) {
          const uint2 b0 = col_read(q_rm, QROW, sub * 16, t * 16);
          const uint2 b1 = col_read(q_rm, QROW, (sub + 1) * 16, t * 16);
          const uint4 bq = make_uint4(b0.x, b0.y, b1.x, b1.y);
          acc_k[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&a_ds, *(const bf16x8_t*)&bq, acc_k[t], 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < VT; ++t) {
          const uint2 b0 = col_read(o_rm, OROW, sub * 16, t * 16);
          const uint2 b1 = col_read(o_rm, OROW, (sub + 1) * 16, t * 16);
          const uint4 bo = make_uint4(b0.x, b0.y, b1.x, b1.y);
          acc_v[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&a_p, *(const bf16x8_t*)&bo, acc_v[t], 0, 0, 0);
        }
      }
    }
    // the next round's rows (gathered while this round computed) go to the other buffer, which
    // was last read a round ago (before the previous barrier); its gathers follow
    if (round + 1 < nround) {
      stage((round + 1) & 1);
      if (round + 2 < nround) {
        fetch(round + 2);
        load_pairs(round + 3);
      }
    }
    lds_barrier();
  }
  // accumulators: column = feature t*16 + col, rows = tokens wave*16 + 4j + i
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long tk = (long)c * BW_S + wave * 16 + 4 * j + i;
    const long rk = ((b * dm.Lkv + tk) * dm.H + hk) * D, rv = ((b * dm.Lkv + tk) * dm.H + hk) * DV;
    if (dm.out16) {
      bf16_t* dkr = (bf16_t*)dk_out + rk;
      bf16_t* dvr = (bf16_t*)dv_out + rv;
#pragma unroll
      for (int t = 0; t < DT; ++t) dkr[t * 16 + col] = f2bf(acc_k[t][i] * dm.sm_scale);
#pragma unroll
      for (int t = 0; t < VT; ++t) dvr[t * 16 + col] = f2bf(acc_v[t][i]);
    } else {
      float* dkr = (float*)dk_out + rk;
      float* dvr = (float*)dv_out + rv;
#pragma unroll
      for (int t = 0; t < DT; ++t) dkr[t * 16 + col] += acc_k[t][i] * dm.sm_scale;
#pragma unroll
      for (int t = 0; t < VT; ++t) dvr[t * 16 + col] += acc_v[t][i];
    }
  }
}

// ---------------------------------------------------------------------------
// dQ, dW: query-block-major, like the forward kernel.  One workgroup owns T consecutive
// queries of a (batch, KV head), sorts the T*K (query, slot) pairs by chunk in LDS, and its
// wavefronts take chunks from a shared counter.  Per 16-row tile of a visit, with the scores
// in the orientation tokens x rows:
//   S^T  = K Q^T,  dP^T = V dO^T      (16x16x32 MFMAs, K and V of the chunk as A operands)
//   P = exp2(S c2 - lse2), delta = sum_tokens P dP (= dW of the pair), dS = w P (dP - delta)
//   dQ  += scale dS K                 (dS^T in accumulator layout is the A operand; K of the chunk
//                                      pre-transposed as B operand)
// dQ tiles are added into an LDS tile of the block as 32-bit fixed point (integer LDS atomics),
// scaled by a power of two from the bound  scale * 2 * max_row(sum_k|w| * |dO|_1) * max|V| * max|K|.
// ---------------------------------------------------------------------------
#define BQ_THREADS 512
#define BQ_MAXP 16  // (query, slot) pairs of a block per thread
#define BQ_WAVES (BQ_THREADS / 64)

struct BqDims {
  int L, Lkv, HQ, H, B, K, NW, T, nblk, nchunk, mask_last;
  float sm_scale;
  const float* slope;  // as in BwDims
  uint32_t k_magic;    // hils_udiv_magic(K)
};

// STAGE: the block's own query and dO rows are copied into LDS once (coalesced) and every tile
// takes its row operands from there instead of gathering them from global memory once per (row,
// slot) pair; chosen by the launcher when those rows fit beside the output tile without shrinking
// the block much (narrow heads without grouping).
template <int D, int DV, int G, bool STAGE>
__global__ void __launch_bounds__(BQ_THREADS)
bw_dq_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ d_o, const bf16_t* __restrict__ ka,
             const bf16_t* __restrict__ va, const bf16_t* __restrict__ kt, const float* __restrict__ vmax,
             const float* __restrict__ kmax, const bf16_t* __restrict__ weights,
             const int32_t* __restrict__ indices, const float* __restrict__ lse, bf16_t* __restrict__ dq,
             float* __restrict__ dw, BqDims dm) {
  constexpr int KS = D / 32, VS = DV / 32;
  constexpr int DT = D / 16;
  constexpr int QT = 16 / G;
  constexpr int MAXP = BQ_MAXP;
  extern __shared__ int smem_i[];
  const int R = dm.T * G;
  int* q_acc = smem_i;                       // (R + 1) x D fixed point; row R takes padding rows
  int* cur = q_acc + (size_t)(R + 1) * D;    // nchunk: histogram -> running ends
  unsigned short* pairs = (unsigned short*)(cur + dm.nchunk);  // T*K pairs (query << 8 | slot) grouped by chunk (T, K <= 256)
  constexpr int QROWB = D * 2 + 16, OROWB = DV * 2 + 16;       // staged rows, padded (bytes)
  char* rows_q = (char*)pairs + (((size_t)dm.T * dm.K * 2 + 15) & ~(size_t)15);  // STAGE: R x QROWB
  char* rows_o = rows_q + (size_t)R * QROWB;                                     //        R x OROWB
  __shared__ float red[32];
  __shared__ int scan_s[BQ_WAVES];
  __shared__ int next_s;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int total = dm.nblk * dm.H * dm.B;
  const int per_xcd = (total + 7) / 8;
  const int vid = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
  if (vid >= total) return;
  const int unit = vid / dm.nblk;
  const int blk = dm.nblk - 1 - (vid - unit * dm.nblk);
  const int hk = unit % dm.H;
  const long b = unit / dm.H;
  const int t0 = blk * dm.T;
  const int K = dm.K;
  const int npair = dm.T * K;

  // selected chunk of every (query, slot) pair of the block
  int creg[MAXP], preg[MAXP];
#pragma unroll
  for (int e = 0; e < MAXP; ++e) {
    const int i = tid + e * BQ_THREADS;
    int c = -1;
    preg[e] = 0;
    if (i < npair) {
      const int ql = (int)hils_udiv((uint32_t)i, (uint32_t)K, dm.k_magic), slot = i - ql * K;
      preg[e] = (ql << 8) | slot;
      if (t0 + ql < dm.L) c = indices[((b * dm.L + t0 + ql) * dm.H + hk) * (long)K + slot];
    }
    if (c < 0 || c >= dm.nchunk) c = -1;
    creg[e] = c;
  }
  // row bound: sum_k |w| * |dO|_1
  float rb = 0.f;
  for (int row = tid; row < R; row += BQ_THREADS) {
    const int ql = row / G, g = row - ql * G;
    if (t0 + ql < dm.L) {
      const long rowi = (b * dm.L + t0 + ql) * (long)dm.HQ + hk * G + g;
      const float a = hils_abs_row_sum_bf16(weights, rowi * dm.NW, K, (long)dm.B * dm.L * dm.HQ * dm.NW);
      float l1 = 0.f;
#pragma unroll
      for (int p8 = 0; p8 < DV / 8; ++p8) {
        float f[8];
        unpack8(*(const uint4*)(d_o + rowi * DV + p8 * 8), f);
#pragma unroll
        for (int e = 0; e < 8; ++e) l1 += fabsf(f[e]);
      }
      rb = fmaxf(rb, a * l1);
    }
  }
  for (int i = tid; i < (R + 1) * D; i += BQ_THREADS) q_acc[i] = 0;
  for (int i = tid; i < dm.nchunk; i += BQ_THREADS) cur[i] = 0;
  if (tid == 0) next_s = 0;
  if (STAGE) {
    // rows beyond the sequence end are never addressed by a pair: they re-read the last row.  Four
    // loads in flight per thread and none inside a branch (a load inside a branch is waited for there).
    auto stage_rows = [&](const bf16_t* src, char* dst, int rowb, int npc) __attribute__((always_inline)) {
      const int n = R * npc;
      for (int i0 = 0; i0 < n; i0 += 4 * BQ_THREADS) {
        bw_u4 t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * BQ_THREADS + tid;
          const int ic = i < n ? i : n - 1;
          const int row = ic / npc, pc = ic - row * npc;
          int tq = t0 + row / G;
          tq = tq < dm.L ? tq : dm.L - 1;
          t[u] = *(const bw_u4*)(src + ((b * dm.L + tq) * (long)dm.HQ + hk * G + row % G) * (npc * 8) + pc * 8);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * BQ_THREADS + tid;
          if (i < n) {
            const int row = i / npc, pc = i - row * npc;
            *(bw_u4*)(dst + row * rowb + pc * 16) = t[u];
          }
        }
      }
    };
    stage_rows(q, rows_q, QROWB, D / 8);
    stage_rows(d_o, rows_o, OROWB, DV / 8);
  }
  __syncthreads();
#pragma unroll
  for (int e = 0; e < MAXP; ++e)
    if (creg[e] >= 0) atomicAdd(&cur[creg[e]], 1);
  rb = block_max(rb, red);  // barrier: histogram complete
  float vm = 0.f, km = 0.f;
  const int per_thr = (dm.nchunk + BQ_THREADS - 1) / BQ_THREADS;
  const int c_lo = tid * per_thr;
  int local = 0;
  for (int c = c_lo; c < c_lo + per_thr && c < dm.nchunk; ++c) {
    const int h = cur[c];
    if (h > 0) {
      vm = fmaxf(vm, vmax[(b * dm.H + hk) * (long)dm.nchunk + c]);
      km = fmaxf(km, kmax[(b * dm.H + hk) * (long)dm.nchunk + c]);
    }
    local += h;
  }
  int incl = local;
#pragma unroll
  for (int o2 = 1; o2 < 64; o2 <<= 1) {
    const int x = __shfl_up(incl, o2, 64);
    if (lane >= o2) incl += x;
  }
  if (lane == 63) scan_s[wave] = incl;
  vm = block_max(vm, red);  // barrier: scan_s visible, all histogram reads done
  km = block_max(km, red);
  int base = incl - local;
  for (int w2 = 0; w2 < wave; ++w2) base += scan_s[w2];
  for (int c = c_lo; c < c_lo + per_thr && c < dm.nchunk; ++c) {
    const int h = cur[c];
    cur[c] = base;
    base += h;
  }
  __syncthreads();
#pragma unroll
  for (int e = 0; e < MAXP; ++e)
    if (creg[e] >= 0) pairs[atomicAdd(&cur[creg[e]], 1)] = (unsigned short)preg[e];
  __syncthreads();  // now chunk c owns pairs[cur[c-1] .. cur[c])

  const float bound = 2.f * dm.sm_scale * rb * vm * km;
  float fx_scale = 1.f;
  if (bound > 0.f && bound < 3.0e38f) {
    int e2 = 28 - ilogbf(bound);
    e2 = e2 > 90 ? 90 : (e2 < -90 ? -90 : e2);
    fx_scale = ldexpf(1.f, e2);
  }
  const float fx_inv = 1.f / fx_scale;
  const float c2 = dm.sm_scale * HILS_LOG2E;
  const float out_scale = dm.sm_scale * fx_scale;
  const int qs = r / G, g = r - qs * G;  // this lane's row of a tile: query slot, head
  const int hq = hk * G + g;
  const float sl = dm.slope ? dm.slope[hq] : 0.f;
  const int npair_valid = cur[dm.nchunk - 1];

  for (;;) {
    int c = 0;
    if (lane == 0) c = atomicAdd(&next_s, 1);
    c = __builtin_amdgcn_readfirstlane(c);
    if (c >= dm.nchunk) break;
    const int vs = c ? cur[c - 1] : 0;
    if (vs >= npair_valid) break;
    const int ve = cur[c];
    if (vs == ve) continue;
    const long chunk = (b * dm.H + hk) * (long)dm.nchunk + c;
    const bf16_t* ka_c = ka + chunk * (long)BW_S * D + lane * 8;
    const bf16_t* va_c = va + chunk * (long)BW_S * DV + lane * 8;
    const bf16_t* kt_c = kt + chunk * (long)BW_S * D + lane * 8;
    // Operands of the chunk: K and V as A operands of the two score products, K transposed as B
    // operand of dQ = dS K.  With 64-wide heads all three stay in registers for every tile of the
    // visit; wider heads reload them per tile (K transposed into the registers of the first set).
    constexpr bool KEEP = D <= 64 && DV <= 64;
    bw_u4 xa[4 * KS], ya[4 * VS], xt[KEEP ? 2 * DT : 1];
    if (KEEP) {
#pragma unroll
      for (int u = 0; u < 4 * KS; ++u) xa[u] = *(const bw_u4*)(ka_c + u * 512);
#pragma unroll
      for (int u = 0; u < 4 * VS; ++u) ya[u] = *(const bw_u4*)(va_c + u * 512);
#pragma unroll
      for (int u = 0; u < 2 * DT; ++u) xt[u] = *(const bw_u4*)(kt_c + u * 512);
    }
    // rows of a tile starting at pair p: this lane's row (pair, gathered q and dO pieces, lse, weight)
    bw_u4 bq[KS], bdo[VS], bq_n[KEEP ? KS : 1], bdo_n[KEEP ? VS : 1];
    float l2 = 0.f, l2_n = 0.f;
    bf16_t wb = 0, wb_n = 0;
    int pk = 0, pk_n = 0;
    auto load_rows = [&](int p, bw_u4* q_r, bw_u4* o_r, float& l_r, bf16_t& w_r, int& pk_r)
                         __attribute__((always_inline)) {
      const int last = ((ve - p < QT) ? ve - p : QT) - 1;  // padding rows repeat the tile's last pair
      pk_r = pairs[p + (qs < last ? qs : last)];
      const long rowi = (b * dm.L + t0 + (pk_r >> 8)) * (long)dm.HQ + hq;
      if (STAGE) {
        const int row_l = (pk_r >> 8) * G + g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) q_r[ks] = *(const bw_u4*)(rows_q + row_l * QROWB + (ks * 32 + j * 8) * 2);
#pragma unroll
        for (int ks = 0; ks < VS; ++ks) o_r[ks] = *(const bw_u4*)(rows_o + row_l * OROWB + (ks * 32 + j * 8) * 2);
      } else {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) q_r[ks] = *(const bw_u4*)(q + rowi * D + ks * 32 + j * 8);
#pragma unroll
        for (int ks = 0; ks < VS; ++ks) o_r[ks] = *(const bw_u4*)(d_o + rowi * DV + ks * 32 + j * 8);
      }
      l_r = lse[rowi * K + (pk_r & 255)];
      w_r = weights[rowi * dm.NW + (pk_r & 255)];
    };
    if (KEEP) load_rows(vs, bq, bdo, l2, wb, pk);
    for (int p = vs; p < ve; p += QT) {
      const int last = ((ve - p < QT) ? ve - p : QT) - 1;
      if (!KEEP) {
        load_rows(p, bq, bdo, l2, wb, pk);
#pragma unroll
        for (int u = 0; u < 4 * KS; ++u) xa[u] = *(const bw_u4*)(ka_c + u * 512);
#pragma unroll
        for (int u = 0; u < 4 * VS; ++u) ya[u] = *(const bw_u4*)(va_c + u * 512);
      }
      const bool more = KEEP && p + QT < ve;
      if (more) load_rows(p + QT, bq_n, bdo_n, l2_n, wb_n, pk_n);  // in flight behind this tile's arithmetic
      int pk_o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int qsl = (4 * j + i) / G;
        pk_o[i] = pairs[p + (qsl < last ? qsl : last)];
      }
      const int ql = pk >> 8, slot = pk & 255;
      const long rowi = (b * dm.L + t0 + ql) * (long)dm.HQ + hq;
      if (l2 == HILS_NEG_INF) l2 = INFINITY;
      const float w_row = bf2f(wb);
      int orow[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int rr = 4 * j + i;
        const int qsl = rr / G;
        const int row = (qsl <= last) ? (pk_o[i] >> 8) * G + (rr - qsl * G) : R;
        orow[i] = row * D + r;
      }
      // ---- S^T and dP^T: tokens x rows, four token tiles each
      f32x4_t st[4], dpt[4];
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) {
        st[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        dpt[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
          st[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, xa[mt * KS + ks]),
                                                           __builtin_bit_cast(bf16x8_t, bq[ks]), st[mt], 0, 0, 0);
#pragma unroll
      for (int ks = 0; ks < VS; ++ks)
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
          dpt[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ya[mt * VS + ks]),
                                                            __builtin_bit_cast(bf16x8_t, bdo[ks]), dpt[mt], 0, 0, 0);
      if (!KEEP) {  // K of the chunk as B operand of dQ = dS K replaces the first operand set
#pragma unroll
        for (int u = 0; u < 2 * DT; ++u) xa[u] = *(const bw_u4*)(kt_c + u * 512);
      }
      if (dm.slope) {
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int dist = BW_S - 2 - (mt * 16 + j * 4 + i);
            st[mt][i] -= sl * (float)(dist > 0 ? dist : 0);
          }
      }
      // ---- P, delta, dS (this lane: row r of the tile, tokens mt*16 + 4j + i)
      float delta = 0.f;
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float pv = __builtin_amdgcn_exp2f(st[mt][i] * c2 - l2);
          st[mt][i] = pv;
          delta += pv * dpt[mt][i];
        }
      if (dm.mask_last && j == 3) {  // token 63 = tile 3, lane group 3, register 3
        delta -= st[3][3] * dpt[3][3];
        st[3][3] = 0.f;
      }
      delta = rows_sum(delta);
      if (j == 0 && qs <= last) dw[rowi * dm.NW + slot] = delta;
      const float f = w_row * out_scale;
      bf16x8_t ap[2];
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        uint4 x;
        x.x = pack_bf2(f * st[2 * s2][0] * (dpt[2 * s2][0] - delta), f * st[2 * s2][1] * (dpt[2 * s2][1] - delta));
        x.y = pack_bf2(f * st[2 * s2][2] * (dpt[2 * s2][2] - delta), f * st[2 * s2][3] * (dpt[2 * s2][3] - delta));
        x.z = pack_bf2(f * st[2 * s2 + 1][0] * (dpt[2 * s2 + 1][0] - delta), f * st[2 * s2 + 1][1] * (dpt[2 * s2 + 1][1] - delta));
        x.w = pack_bf2(f * st[2 * s2 + 1][2] * (dpt[2 * s2 + 1][2] - delta), f * st[2 * s2 + 1][3] * (dpt[2 * s2 + 1][3] - delta));
        ap[s2] = __builtin_bit_cast(bf16x8_t, x);
      }
      // ---- dQ tile += dS K: four column tiles at a time
#pragma unroll
      for (int d0 = 0; d0 < DT; d0 += 4) {
        f32x4_t acc[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) acc[u] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const bw_u4 kb2 = KEEP ? xt[KEEP ? (d0 + u) * 2 + s2 : 0] : xa[(d0 + u) * 2 + s2];
            acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ap[s2], __builtin_bit_cast(bf16x8_t, kb2), acc[u], 0, 0, 0);
          }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) atomicAdd(&q_acc[orow[i] + (d0 + u) * 16], __float2int_rn(acc[u][i]));
      }
      if (more) {  // the next tile's rows become the current ones
#pragma unroll
        for (int ks = 0; ks < (KEEP ? KS : 1); ++ks) bq[ks] = bq_n[ks];
#pragma unroll
        for (int ks = 0; ks < (KEEP ? VS : 1); ++ks) bdo[ks] = bdo_n[ks];
        l2 = l2_n;
        wb = wb_n;
        pk = pk_n;
      }
    }
  }
  __syncthreads();
  constexpr int C8 = D / 8;
  for (int i = tid; i < R * C8; i += BQ_THREADS) {
    const int row = i / C8, c8 = i - row * C8;
    const int ql = row / G, g2 = row - ql * G;
    const int t = t0 + ql;
    if (t < dm.L) {
      const int* src = q_acc + (size_t)row * D + c8 * 8;
      uint4 x;
      x.x = pack_bf2((float)src[0] * fx_inv, (float)src[1] * fx_inv);
      x.y = pack_bf2((float)src[2] * fx_inv, (float)src[3] * fx_inv);
      x.z = pack_bf2((float)src[4] * fx_inv, (float)src[5] * fx_inv);
      x.w = pack_bf2((float)src[6] * fx_inv, (float)src[7] * fx_inv);
      *(uint4*)(dq + ((b * dm.L + t) * (long)dm.HQ + hk * G + g2) * D + c8 * 8) = x;
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static size_t bw_round(size_t n) { return (n + 255) & ~(size_t)255; }

// sm_n (an extra term in every chunk's softmax denominator) reaches the backward only through
// the saved per-chunk LSE, so any sm_n >= 0 is covered.
bool hils_bw_covers(int L, int Lkv, int HQ, int H, int D, int Dv, int K, int S, int q_block, int WH,
                    float sm_n, const float* slope) {
  if (H <= 0 || HQ % H != 0) return false;
  const int G = HQ / H;
  return S == BW_S && (D == 64 || D == 128) && (Dv == 64 || Dv == 128) &&
         (G == 1 || G == 2 || G == 4 || G == 8 || G == 16) && q_block == 1 && WH == HQ && sm_n >= 0.f &&
         Lkv >= S && K <= 256 && L < (1 << 24) && Lkv / S <= 12288;
}

void hils_ga_pack_launch(const void* a, const void* b, void* ap, void* bp, float* bmax, int B, int Lkv,
                         int H, int Da, int Db, void* stream);

// T queries per workgroup of the dQ kernel such that the fixed-point tile, the chunk histogram
// and the pair list (and, with `stage`, the block's own query and dO rows) fit in LDS; 0 when the
// shape does not fit.
static size_t bq_smem_bytes(int T, int G, int D, int Dv, int K, int nchunk, bool stage) {
  size_t n = (size_t)(T * G + 1) * D * 4 + (size_t)nchunk * 4 + (((size_t)T * K * 2 + 15) & ~(size_t)15);
  if (stage) n += (size_t)T * G * ((size_t)D * 2 + 16 + (size_t)Dv * 2 + 16);
  return n;
}
static int bq_pick_T(int L, int G, int D, int Dv, int K, int nchunk, bool stage, size_t* smem_out) {
  // the largest block that fits: the more rows share a visit, the fewer K/V bytes per row
  const size_t limit = 156 * 1024;
  const size_t per_q = (size_t)G * D * 4 + (size_t)K * 2 + (stage ? (size_t)G * ((size_t)(D + Dv) * 2 + 32) : 0);
  const size_t fixed = (size_t)D * 4 + (size_t)nchunk * 4 + 16;  // spare row, histogram, alignment
  if (fixed + per_q > limit) return 0;
  long T = (long)((limit - fixed) / per_q);
  if (T > 256) T = 256;  // a pair is (query << 8 | slot) in 16 bits
  if (T * K > BQ_MAXP * BQ_THREADS) T = (BQ_MAXP * BQ_THREADS) / K;
  if (T > L) T = L;
  if (T >= 8) T &= ~7L;
  if (T < 1) return 0;
  *smem_out = bq_smem_bytes((int)T, G, D, Dv, K, nchunk, stage);
  return (int)T;
}

struct BwLayout {
  size_t counts, offsets, cursor, pairs, ka, va, kt, vmax, kmax, total;
};
static BwLayout bw_layout(int B, int L, int Lkv, int H, int D, int Dv, int K) {
  const size_t cells = (size_t)B * H * (Lkv / BW_S);
  BwLayout lo;
  size_t o = 0;
  lo.counts = o; o += bw_round((cells + 1) * 4);
  lo.offsets = o; o += bw_round((cells + 1) * 4);
  lo.cursor = o; o += bw_round((cells + 1) * 4);
  lo.pairs = o; o += bw_round((size_t)B * L * H * K * 4);
  lo.ka = o; o += bw_round(cells * BW_S * D * 2);
  lo.va = o; o += bw_round(cells * BW_S * Dv * 2);
  lo.kt = o; o += bw_round(cells * BW_S * D * 2);
  lo.vmax = o; o += bw_round(cells * 4);
  lo.kmax = o; o += bw_round(cells * 4);
  lo.total = o;
  return lo;
}

size_t hils_bw_workspace_bytes(int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K, int S,
                               int q_block, int WH, float sm_n) {
  if (!hils_bw_covers(L, Lkv, HQ, H, D, Dv, K, S, q_block, WH, sm_n, nullptr)) return 0;
  size_t smem;
  if (bq_pick_T(L, HQ / H, D, Dv, K, Lkv / S, false, &smem) == 0) return 0;
  return bw_layout(B, L, Lkv, H, D, Dv, K).total;
}

template <int D, int DV>
static int bw_launch_dkdv(int G, dim3 grid, hipStream_t st, const bf16_t* q, const bf16_t* k,
                          const bf16_t* v, const bf16_t* w, const float* lse, const float* delta,
                          const bf16_t* d_o, const int* offsets, const uint32_t* pairs, void* dk, void* dv,
                          const BwDims& dm) {
#define BW_CALL(G_)                                                                                 \
  hipLaunchKernelGGL((bw_dkdv_kernel<D, DV, G_>), grid, dim3(256), smem, st, q, k, v, w, lse, delta, d_o, \
                     offsets, pairs, dk, dv, dm)
  constexpr int DMAX = D > DV ? D : DV;
  constexpr int NSUB = 256 / DMAX;
  const size_t smem = 2 * ((size_t)16 * NSUB * (D * 2 + 16) + (size_t)16 * NSUB * (DV * 2 + 16) +
                           (size_t)3 * 16 * NSUB * sizeof(float));  // two staging buffers
  switch (G) {
    case 1: BW_CALL(1); break;
    case 2: BW_CALL(2); break;
    case 4: BW_CALL(4); break;
    case 8: BW_CALL(8); break;
    case 16: BW_CALL(16); break;
    default: return -1;
  }
#undef BW_CALL
  return HILS_OK;
}

template <int D, int DV, int G, bool STAGE>
static int bq_launch(dim3 grid, size_t smem, hipStream_t st, const bf16_t* q, const bf16_t* d_o,
                     const bf16_t* ka, const bf16_t* va, const bf16_t* kt, const float* vmax,
                     const float* kmax, const bf16_t* w, const int32_t* idx, const float* lse, bf16_t* dq,
                     float* dw, const BqDims& dm) {
  auto kern = bw_dq_kernel<D, DV, G, STAGE>;
  static HilsLdsReserve reserved;  // per instantiation
  if (int rc = hils_reserve_lds(&reserved, (const void*)kern, smem, "hils_sparse_attn_bwd")) return rc;
  hipLaunchKernelGGL(kern, grid, dim3(BQ_THREADS), smem, st, q, d_o, ka, va, kt, vmax, kmax, w, idx, lse, dq, dw, dm);
  return HILS_OK;
}

template <int D, int DV>
static int bq_dispatch_g(int G, bool stage, dim3 grid, size_t smem, hipStream_t st, const bf16_t* q,
                         const bf16_t* d_o, const bf16_t* ka, const bf16_t* va, const bf16_t* kt,
                         const float* vmax, const float* kmax, const bf16_t* w, const int32_t* idx,
                         const float* lse, bf16_t* dq, float* dw, const BqDims& dm) {
  if (stage)  // only built without head grouping (see bq_stage_pays)
    return bq_launch<D, DV, 1, true>(grid, smem, st, q, d_o, ka, va, kt, vmax, kmax, w, idx, lse, dq, dw, dm);
  switch (G) {
    case 1: return bq_launch<D, DV, 1, false>(grid, smem, st, q, d_o, ka, va, kt, vmax, kmax, w, idx, lse, dq, dw, dm);
    case 2: return bq_launch<D, DV, 2, false>(grid, smem, st, q, d_o, ka, va, kt, vmax, kmax, w, idx, lse, dq, dw, dm);
    case 4: return bq_launch<D, DV, 4, false>(grid, smem, st, q, d_o, ka, va, kt, vmax, kmax, w, idx, lse, dq, dw, dm);
    case 8: return bq_launch<D, DV, 8, false>(grid, smem, st, q, d_o, ka, va, kt, vmax, kmax, w, idx, lse, dq, dw, dm);
    case 16: return bq_launch<D, DV, 16, false>(grid, smem, st, q, d_o, ka, va, kt, vmax, kmax, w, idx, lse, dq, dw, dm);
  }
  return -1;
}

// Staging the block's rows in LDS pays when it costs little block size: the block shrinks by the
// rows' bytes, and a smaller block pulls more K/V bytes per row.
static bool bq_stage_pays(int L, int G, int D, int Dv, int K, int nchunk) {
  if (G != 1) return false;
  size_t a, b2;
  const int t_plain = bq_pick_T(L, G, D, Dv, K, nchunk, false, &a);
  const int t_stage = bq_pick_T(L, G, D, Dv, K, nchunk, true, &b2);
  return t_stage > 0 && 4 * t_stage >= 3 * t_plain;
}

// Inverse index of an index tensor (B, L, H, K) with values in [0, nchunk) or < 0: counts,
// offsets (cells + 1 ints, cells = B*H*nchunk), cursor (scratch) and the pairs (t << 8 | slot)
// grouped by (b, h, chunk).  Also used by the top-k backward.
void hils_build_chunk_index(const int32_t* indices, int* counts, int* offsets, int* cursor, uint32_t* pairs,
                            int B, int L, int H, int K, int nchunk, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  const long cells = (long)B * H * nchunk;
  {
    const long n = cells + 1;
    hipLaunchKernelGGL(bw_fill_int_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, counts, 0, n);
  }
  // segments of queries per workgroup: short enough for a few thousand workgroups (the LDS atomics of
  // a workgroup on one chunk's counter serialise), long enough that a workgroup's one global atomic per
  // chunk stays cheap
  int seg_len = L;
  while ((long)B * H * ((L + seg_len - 1) / seg_len) < 4096 && seg_len > 128) seg_len = (seg_len + 1) / 2;
  dim3 gs((L + seg_len - 1) / seg_len, H, B);
  hipLaunchKernelGGL(bw_count_kernel, gs, dim3(1024), (size_t)nchunk * 4, st, indices, counts, L, H, K, nchunk, seg_len);
  hipLaunchKernelGGL(bw_scan_kernel, dim3(1), dim3(1024), 0, st, counts, offsets, cursor, cells);
  hipLaunchKernelGGL(bw_scatter_kernel, gs, dim3(1024), (size_t)nchunk * 4, st, indices, cursor, pairs, L, H, K, nchunk, seg_len);
}

// Whole backward on the MFMA kernels: dq (bf16, written), dw (fp32, written at the valid slots),
// dk / dv (fp32, accumulated into the caller's buffers; or, with kv16, bf16 tensors that are overwritten).
int hils_bw_run(const void* q, const void* k, const void* v, const void* weights, const int32_t* indices,
                const float* slope, const float* lse, const void* d_o, void* dq, void* dk, void* dv,
                float* dw, void* workspace, int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K, int NW,
                float sm_scale, int mask_last, int kv16, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  const int nchunk = Lkv / BW_S;
  const size_t cells = (size_t)B * H * nchunk;
  const BwLayout lo = bw_layout(B, L, Lkv, H, D, Dv, K);
  char* ws = (char*)workspace;
  int* counts = (int*)(ws + lo.counts);
  int* offsets = (int*)(ws + lo.offsets);
  int* cursor = (int*)(ws + lo.cursor);
  uint32_t* pairs = (uint32_t*)(ws + lo.pairs);
  bf16_t* ka = (bf16_t*)(ws + lo.ka);
  bf16_t* va = (bf16_t*)(ws + lo.va);
  bf16_t* kt = (bf16_t*)(ws + lo.kt);
  float* vmax = (float*)(ws + lo.vmax);
  float* kmax = (float*)(ws + lo.kmax);
  const int G = HQ / H;
  if (H > 65535 || B > 65535) return -1;
  // ---- operand packing: K as A operand (+ max|V|), V as A operand + K transposed (+ max|K|)
  hils_ga_pack_launch(k, v, ka, nullptr, vmax, B, Lkv, H, D, Dv, stream);
  hils_ga_pack_launch(v, k, va, kt, kmax, B, Lkv, H, Dv, D, stream);
  // ---- dQ, dW
  {
    size_t smem;
    const bool stage = bq_stage_pays(L, G, D, Dv, K, nchunk);
    int T = bq_pick_T(L, G, D, Dv, K, nchunk, stage, &smem);
    if (T == 0) return -1;
    // small problems: rather every compute unit busy than the largest blocks
    while (T >= 72 && (long)((L + T - 1) / T) * H * B < 256) {
      T -= 8;
      smem = bq_smem_bytes(T, G, D, Dv, K, nchunk, stage);
    }
    const int nblk = (L + T - 1) / T;
    const long total = (long)nblk * H * B;
    if (total > (1L << 30)) return -1;
    BqDims dm{L, Lkv, HQ, H, B, K, NW, T, nblk, nchunk, mask_last, sm_scale, slope, hils_udiv_magic((uint32_t)K)};
    dim3 grid((unsigned)(((total + 7) / 8) * 8));
    int rc = -1;
#define BQ_D(D_, DV_)                                                                                 \
  rc = bq_dispatch_g<D_, DV_>(G, stage, grid, smem, st, (const bf16_t*)q, (const bf16_t*)d_o, ka, va, kt, vmax, \
                              kmax, (const bf16_t*)weights, indices, lse, (bf16_t*)dq, dw, dm)
    if (D == 64 && Dv == 64) BQ_D(64, 64);
    else if (D == 128 && Dv == 128) BQ_D(128, 128);
    else if (D == 64 && Dv == 128) BQ_D(64, 128);
    else if (D == 128 && Dv == 64) BQ_D(128, 64);
#undef BQ_D
    if (rc != HILS_OK) return rc;
  }
  // ---- inverse index, then dK, dV
  hils_build_chunk_index(indices, counts, offsets, cursor, pairs, B, L, H, K, nchunk, stream);
  BwDims dm{L, Lkv, HQ, H, K, NW, nchunk, mask_last, sm_scale, kv16, B, slope};
  if (kv16 && Lkv > nchunk * BW_S) {  // tokens behind the last whole chunk are never attended
    for (int b2 = 0; b2 < B; ++b2) {
      const long nk = (long)(Lkv - nchunk * BW_S) * H * D / 2, nv = (long)(Lkv - nchunk * BW_S) * H * Dv / 2;
      int* pk = (int*)((bf16_t*)dk + ((long)b2 * Lkv + (long)nchunk * BW_S) * H * D);
      int* pv = (int*)((bf16_t*)dv + ((long)b2 * Lkv + (long)nchunk * BW_S) * H * Dv);
      hipLaunchKernelGGL(bw_fill_int_kernel, dim3((unsigned)((nk + 255) / 256)), dim3(256), 0, st, pk, 0, nk);
      hipLaunchKernelGGL(bw_fill_int_kernel, dim3((unsigned)((nv + 255) / 256)), dim3(256), 0, st, pv, 0, nv);
    }
  }
  const long unit_rounds = ((long)H * B + 7) / 8;
  if (unit_rounds * nchunk * 8 > 2147483647L) return -1;
  dim3 grid((unsigned)(unit_rounds * nchunk * 8));
  int rc = -1;
#define BW_D(D_, DV_)                                                                              \
  rc = bw_launch_dkdv<D_, DV_>(G, grid, st, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v,   \
                               (const bf16_t*)weights, lse, dw, (const bf16_t*)d_o, offsets, pairs, dk, dv, dm)
  if (D == 64 && Dv == 64) BW_D(64, 64);
  else if (D == 128 && Dv == 128) BW_D(128, 128);
  else if (D == 64 && Dv == 128) BW_D(64, 128);
  else if (D == 128 && Dv == 64) BW_D(128, 64);
#undef BW_D
  return rc;
}
