// Prefill top-k chunk selection, one pass over the chunk keys.
//
// One wavefront owns 16/GMAX consecutive queries of a (batch, KV head): the 16 rows of its MFMA
// tile are (queries x the GMAX heads of the KV head).  It streams the chunk keys once (B operands,
// 16 chunks per block, repacked into operand order by topk_pack_lmk_kernel) and keeps every scaled
// logit in registers: accumulator register i of block nt in lane (col, j) is row 4j+i, chunk
// nt*16+col, so a query's logits for up to 512 chunks lie in the 16 lanes of one lane row, 32 per
// lane.  From there, without touching memory again:
//   * the log-sum-exp of every row (in-lane maxima and sums, one 16-lane reduction per row),
//   * the selection score of every (query, chunk): max over the heads of logit - lse_total, a float
//     (in-lane: the heads of a query are registers of one lane),
//   * the top-K per query, the four lane rows working on four queries at once: the K-th largest
//     score is bracketed from the two largest scores of every lane (their minimum over the lanes is
//     a lower bound with at least 32 scores above it), the scores above the bound (about 1.5 K of
//     512) are compacted through LDS to at most 8 per lane, turned into order-preserving unsigned
//     keys, and the threshold is found on those by a bitwise search whose counts are 16-lane DPP
//     reductions (no ballots, no scalar round trip) and which stops at the first probe that counts
//     exactly K; ties at the threshold go to the lower chunk indices,
//   * the ascending order of the winners from a 512-bit map of the winning chunks in LDS
//     (rank = set bits below the chunk), and the winners' raw scores straight from the logits.
// Five to eight query heads per KV head (HALF below) take two wavefronts per four queries, one for the
// heads 0..3 and one for the rest: each forms the partial selection scores of its heads, the two
// trade them through LDS, and both then select on the same scores and write their own heads' outputs.
// Covers G = 1..8, D in {64, 128}, N <= 512, topk <= 32, an optional additive bias per
// (chunk, head) (the layer's prior bias), no Gumbel noise / drop mask; everything else runs on the
// kernels of topk.hip.  With a bias the registers hold the biased logits (what the log-sum-exp and
// the selection work on) and a winner's raw score is its logit minus the bias again.
#include <type_traits>
#include "decode_rows.h"
#include "../../include/hils_amd.h"

#define TG_NB 32     // chunk blocks of 16 a lane row can hold (N <= 512)
#define TG_CAND 128  // compacted candidates per query (8 per lane)

// Order-preserving unsigned image of a finite score (larger score <-> larger key, -0 as +0) and its
// inverse.  Every finite score has a key above 0x00800000, so 0 stands for "no key".
__device__ __forceinline__ uint32_t tg_score_key(float f) {
  f = f + 0.0f;  // -0 -> +0
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float tg_key_score(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// all-reduce over the 16 lanes of a lane row
template <class F>
__device__ __forceinline__ uint32_t tg_row_reduce_u(uint32_t x, F f) {
  x = f(x, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xF, 0xF, false));
  x = f(x, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, false));
  x = f(x, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x141, 0xF, 0xF, false));
  x = f(x, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x140, 0xF, 0xF, false));
  return x;
}
__device__ __forceinline__ uint32_t tg_row_max_u(uint32_t x) {
  return tg_row_reduce_u(x, [](uint32_t a, uint32_t b) { return a > b ? a : b; });
}
__device__ __forceinline__ uint32_t tg_row_min_u(uint32_t x) {
  return tg_row_reduce_u(x, [](uint32_t a, uint32_t b) { return a < b ? a : b; });
}
__device__ __forceinline__ int tg_row_sum_i(int x) {
  return (int)tg_row_reduce_u((uint32_t)x, [](uint32_t a, uint32_t b) { return a + b; });
}
__device__ __forceinline__ float tg_row_max_f(float x) {
  x = fmaxf(x, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xF, 0xF, false)));
  x = fmaxf(x, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xF, 0xF, false)));
  x = fmaxf(x, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xF, 0xF, false)));
  x = fmaxf(x, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xF, 0xF, false)));
  return x;
}
__device__ __forceinline__ float tg_row_min_f(float x) {
  x = fminf(x, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xF, 0xF, false)));
  x = fminf(x, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xF, 0xF, false)));
  x = fminf(x, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xF, 0xF, false)));
  x = fminf(x, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x140, 0xF, 0xF, false)));
  return x;
}
// exclusive prefix sum over the 16 lanes of a lane row (lanes shifted in from outside read 0)
__device__ __forceinline__ int tg_row_excl_scan(int x) {
  int s = x;
  s += __builtin_amdgcn_update_dpp(0, s, 0x111, 0xF, 0xF, true);  // row_shr:1
  s += __builtin_amdgcn_update_dpp(0, s, 0x112, 0xF, 0xF, true);  // row_shr:2
  s += __builtin_amdgcn_update_dpp(0, s, 0x114, 0xF, 0xF, true);  // row_shr:4
  s += __builtin_amdgcn_update_dpp(0, s, 0x118, 0xF, 0xF, true);  // row_shr:8
  return s - x;
}

// Threshold of the K largest keys a lane row holds, NE per lane (0 = no key), all non-zero keys in
// [lo, hi] and at least K of them: returns T in [lo, hi] with count(key >= T) >= K >= count(key > T)
// and count(key > T) + count(key == T) >= K.  The bitwise search of a lane row stops as soon as a
// probe at or above lo counts exactly K keys (the winners are then known, exact is set and no tie
// needs breaking: with about 1.5 K keys in the range that takes a third of the steps of a search
// down to the last bit, and unless the K-th and (K+1)-th largest keys are equal some probe does);
// rows that are not live take no part, and the loop, which is wavefront-uniform, ends when no row
// is live.
template <int NE>
__device__ __forceinline__ uint32_t tg_kth_largest(const uint32_t (&k)[NE], uint32_t lo, uint32_t hi, int K,
                                                   bool live, bool& exact) {
  const uint32_t diff = lo ^ hi;
  // bits above the highest differing one are shared by every key; the search runs over the rest
  const int top = diff ? 31 - __clz((int)diff) : -1;
  uint32_t T = (top >= 31 || top < 0) ? (top < 0 ? lo : 0u) : (lo & ~((2u << top) - 1u));
  live = live & (top >= 0);
  const int top_l = live ? top : -1;
  int top_w = __builtin_amdgcn_readlane(top_l, 0);
  top_w = max(top_w, __builtin_amdgcn_readlane(top_l, 16));
  top_w = max(top_w, __builtin_amdgcn_readlane(top_l, 32));
  top_w = max(top_w, __builtin_amdgcn_readlane(top_l, 48));
  for (int bit = top_w; bit >= 0; --bit) {
    if (!__any(live)) break;
    const uint32_t c = T | (1u << bit);
    int cl = 0;
#pragma unroll
    for (int e = 0; e < NE; ++e) cl += (k[e] >= c) ? 1 : 0;
    const int cnt = tg_row_sum_i(cl);
    const bool act = live & (bit <= top);
    if (act & (cnt >= K)) T = c;
    if (act & (cnt == K) & (c >= lo)) {
      live = false;
      exact = true;
    }
  }
  return T;
}

// NB: chunk blocks the launch covers, 8, 16, 24 or 32.  Every query of the launch sees at most 16*NB
// chunks and more than 16*NB/2 (NB = 8: any number), so only the blocks from NMASK on can hold
// invisible chunks; t_base: first query.  Everything is unrolled over the NB blocks: register-resident
// data has no other way of being indexed, and the host splits a call into launches by NB so that
// early queries do not pay for 32.  (The 24-block instantiation pays through its occupancy: held to
// 168 registers it runs three wavefronts per SIMD with ten spilled dwords, 114 us for the queries that
// see 257..384 chunks against 133 us of the 32-block kernel; at two wavefronts per SIMD it was no
// faster than 32 blocks.)
// Wavefronts per workgroup, each with queries of its own (they never synchronise).  A workgroup keeps
// its registers and LDS until its slowest wavefront is through (the threshold searches differ in
// length): 4 per workgroup ran 3.5 % slower than 2, and 8 ran 17 % slower; 1 was no faster than 2.
#define TG_WAVES 2
// PERQ: one chunk key per QUERY head (lmk_packed holds h_kv * G heads).  A workgroup is then four
// wavefronts on 16 queries: for the logits wavefront w takes head w of all 16 queries (full MFMA
// rows, that head's keys streamed once for 16 queries), and block by block the four wavefronts
// trade accumulators through LDS so that each ends up with the rows the shared-key layout gives it
// (its 4 queries x 4 heads); everything behind the logits is the same code.
// HALF (G = 5..8): the wavefronts come in pairs on the same four queries, wavefront 2p takes the heads
// 0..3 and 2p+1 the heads 4..G-1; with PERQ a workgroup is eight wavefronts (head w's keys in
// wavefront w) on 16 queries, otherwise one pair.
template <int GMAX, int KS, int NB, bool EXPORT, bool BIAS, bool PERQ, bool HALF>
__global__ void __launch_bounds__(64 * (PERQ ? (HALF ? 8 : 4) : TG_WAVES))
    // (eight-wavefront workgroups: three per SIMD leave room for one workgroup only, i.e. two per SIMD)
    __attribute__((amdgpu_waves_per_eu(NB <= 8 ? 5 : (NB <= 16 ? 4 : (NB <= 24 && !(PERQ && HALF) ? 3 : 2)))))
topk_fwd_group_kernel(const bf16_t* __restrict__ q, const uint4* __restrict__ lmk_packed,
                      const float* __restrict__ lse_swa, const float* __restrict__ bias,
                      int32_t* __restrict__ indices,
                      bf16_t* __restrict__ scores, float* __restrict__ lse_total_out,
                      float* __restrict__ sel_logits_out, int L, int N, int h_kv, int G, int topk,
                      int block_size, int window_size, int causal, int q_offset, float sm_scale,
                      int t_base, int t_end, int bs_shift, int lse_bf16) {
  constexpr int D = KS * 32;
  constexpr int QPL = 4 / GMAX;   // queries per lane (its four accumulator rows)
  constexpr int NQ = 16 / GMAX;   // queries per wavefront
  constexpr int NMASK = EXPORT ? 0 : (NB > 8 ? NB / 2 : 0);  // blocks below it are visible to every row
  constexpr int TGW = PERQ ? (HALF ? 8 : 4) : TG_WAVES;      // wavefronts per workgroup
  constexpr int QGROUPS = HALF ? TGW / 2 : TGW;              // ... and how many have queries of their own
  static_assert(!PERQ || GMAX == 4, "per-query-head keys: four heads, four wavefronts");
  static_assert(!HALF || (GMAX == 4 && TG_WAVES == 2), "halves: four heads each, a pair per workgroup");
  constexpr int PB = NB >= 32 ? 2 : 1;  // blocks per load group (two groups are live: 16 registers per block and group)
  // LDS that several wavefronts share.  PERQ: accumulators of a load group on their way between the
  // wavefronts, [buffer][block][from wavefront = head][register][lane]; two buffers take turns, so that
  // one barrier a group is enough.  HALF: the selection scores a pair trades, [pair][block][lane].  With
  // both the two uses follow each other in the same memory, and so do the eight wavefronts' selection
  // areas (candidates and output stage), which would not fit beside them.
  constexpr bool OVER = PERQ && HALF;
  constexpr int XCH_F = PERQ ? 2 * PB * TGW * 4 * 64 : 0, KX_F = HALF ? QGROUPS * NB * 64 : 0;
  constexpr int SEL_B = 4 * TG_CAND * 4 + NQ * 32 * 4 + NQ * GMAX * 32 * 2;  // bytes of a wavefront's selection areas
  constexpr int XB_F = OVER ? (XCH_F > KX_F ? (XCH_F > TGW * SEL_B / 4 ? XCH_F : TGW * SEL_B / 4)
                                            : (KX_F > TGW * SEL_B / 4 ? KX_F : TGW * SEL_B / 4))
                            : (XCH_F + KX_F > 0 ? XCH_F + KX_F : 1);
  __shared__ __align__(16) float xbuf[XB_F];
  __shared__ uint32_t cand_w[OVER ? 1 : TGW][4][TG_CAND];          // compacted candidate keys, per lane row
  __shared__ uint32_t words_w[TGW][4][16], wbase_w[TGW][4][16];  // winner map of a query and its word prefix counts
  __shared__ __align__(16) int stage_i_w[OVER ? 1 : TGW][NQ * 32];               // winners' chunk indices, [query][slot]
  __shared__ __align__(16) bf16_t stage_s_w[OVER ? 1 : TGW][NQ * GMAX * 32];  // their raw scores, [query][slot][head]
  // the bias of this (batch, KV head): [chunk][head, padded to 4] fp32, a copy per wavefront (they never
  // synchronise); read back 16 bytes per lane right where a block's logits are formed, instead of
  // global loads whose latency the compiler covers with registers this kernel does not have.
  // (One copy per workgroup, filled by its wavefronts together before they part; with HALF one per half of
  // the heads.)
  __shared__ __align__(16) float bias_w[BIAS ? (HALF ? (PERQ ? 2 : TGW) : 1) : 1][BIAS ? NB * 16 : 1][4];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int half = HALF ? (wave & 1) : 0;   // this wavefront's heads are 4 * half ..
  const int pw = HALF ? (wave >> 1) : wave; // which of the workgroup's queries it has
  const int gofs = 4 * half;
  char* const sel_area = (char*)xbuf + (OVER ? wave * SEL_B : 0);
  uint32_t (*cand)[TG_CAND] = OVER ? (uint32_t (*)[TG_CAND])sel_area : cand_w[OVER ? 0 : wave];
  uint32_t (*words)[16] = words_w[wave];
  uint32_t (*wbase)[16] = wbase_w[wave];
  int* stage_i = OVER ? (int*)(sel_area + 4 * TG_CAND * 4) : stage_i_w[OVER ? 0 : wave];
  bf16_t* stage_s = OVER ? (bf16_t*)(sel_area + 4 * TG_CAND * 4 + NQ * 32 * 4) : stage_s_w[OVER ? 0 : wave];
  const int lane = threadIdx.x & 63, col = lane & 15, j = lane >> 4;
  const int t0 = t_base + (blockIdx.x * QGROUPS + pw) * NQ;
  const int t_wg = t_base + blockIdx.x * QGROUPS * NQ;  // PERQ: the workgroup's 16 queries
  // (with a bias and shared keys the wavefronts of a workgroup first stage the bias together, below)
  const bool gone = (PERQ ? t_wg : t0) >= t_end;    // (PERQ: the wavefronts meet at barriers until the logits are in)
  if (!(BIAS && !PERQ && !HALF) && gone) return;
  const int t_safe = PERQ ? t_wg : t0;              // a query of this launch, for the addresses of rows that have none
  const int hk = blockIdx.y;
  const long b = blockIdx.z;
  float (*bias_s)[4] = bias_w[BIAS ? (OVER ? half : (HALF ? wave : 0)) : 0];
  if constexpr (BIAS) {
    const float* bias_u = bias + (b * N * (long)h_kv + hk) * G;
    if constexpr (HALF) {
      // this half's heads; PERQ: the four wavefronts of a half fill its copy together (the first
      // barrier of the logits comes before anybody reads it)
      for (int c = OVER ? pw * 64 + lane : lane; c < NB * 16; c += OVER ? 64 * QGROUPS : 64) {
        float e4[4] = {0.f, 0.f, 0.f, 0.f};
        if (c < N) {
          const float* bp = bias_u + (long)c * h_kv * G + gofs;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (gofs + e < G) e4[e] = bp[e];
        }
        *(float4*)bias_s[c] = make_float4(e4[0], e4[1], e4[2], e4[3]);
      }
    } else {
#pragma unroll
    for (int c = wave * 64 + lane; c < NB * 16; c += 64 * TGW) {  // the workgroup's wavefronts together
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);  // chunks past N (never visible) and heads past G: 0
      if (c < N) {
        const float* bp = bias_u + (long)c * h_kv * G;
        v.x = bp[0];
        if (GMAX > 1 && G > 1) v.y = bp[1];
        if (GMAX > 2 && G > 2) v.z = bp[2];
        if (GMAX > 2 && G > 3) v.w = bp[3];
      }
      *(float4*)bias_s[c] = v;
    }
    __syncthreads();  // (with a key per query head the bias is added before the first exchange)
    }
  }
  if (BIAS && !PERQ && !HALF && gone) return;

  // chunks a query sees (visible_limit of common.h; bs_shift >= 0: the chunk size is 1 << bs_shift and
  // the division is an arithmetic shift, which rounds towards minus infinity as floordiv does)
  auto limit_of = [&](int tq) -> int {
    const int a = window_size > 0 ? tq + q_offset - window_size + 1 : tq + q_offset;
    int lm = causal ? (bs_shift >= 0 ? (a >> bs_shift) : floordiv(a, block_size)) : N;
    return lm < 0 ? 0 : (lm > N ? N : lm);
  };
  // accumulator row 4j+i <-> (query t0 + (4j+i)/GMAX, head (4j+i)%GMAX): a lane has QPL queries
  int lim[4];
  bool rowok[4];
#pragma unroll
  for (int u = 0; u < QPL; ++u) {
    const int tq = t0 + j * QPL + u;
    const int lq = tq < t_end ? limit_of(tq) : 0;
#pragma unroll
    for (int e = 0; e < GMAX; ++e) {
      rowok[u * GMAX + e] = (tq < t_end) & (gofs + e < G);
      lim[u * GMAX + e] = gofs + e < G ? lq : 0;
    }
  }
  const int nb_real = (N + 15) / 16;  // blocks the packed chunk keys hold

  // query rows as A operands
  bf16x8_t afrag[KS];
  {
    const int r = lane & 15;
    const int g = PERQ ? wave : gofs + r % GMAX, tq = PERQ ? t_wg + r : t0 + r / GMAX;
    const bool ok = tq < t_end && g < G;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 v = *(const uint4*)(q + (((b * L + (ok ? tq : t_safe)) * h_kv + hk) * (long)G + (ok ? g : 0)) * D + ks * 32 + j * 8);
      if (!ok) v = make_uint4(0, 0, 0, 0);
      afrag[ks] = *(bf16x8_t*)&v;
    }
  }
  float swa[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * j + i;
    const int tq = t0 + r / GMAX, g = gofs + r % GMAX;
    const long li = ((b * L + (rowok[i] ? tq : t_safe)) * (long)h_kv + hk) * G + (rowok[i] ? g : 0);
    float x;  // the layer hands lse_swa over in its hidden dtype (hils_attention.py:547)
    if (lse_bf16) x = bf2f(((const bf16_t*)lse_swa)[li]); else x = lse_swa[li];
    swa[i] = rowok[i] ? x : HILS_NEG_INF;
  }

  // ---- the logits: x[nt][i] = sm_scale * <q_row, lmk_chunk>, -inf where the chunk is not visible ----
  const uint4* pbase = PERQ ? lmk_packed + (((b * h_kv + hk) * (long)G + (wave < G ? wave : 0)) * nb_real * KS) * 64 + lane
                            : lmk_packed + ((b * h_kv + hk) * (long)nb_real * KS) * 64 + lane;
  float x[NB][4];
  // the keys of two blocks travel together, one such group ahead of their use (the loads of a
  // block issued right before its MFMAs would each expose a full memory latency)
  typedef unsigned tg_u32x4 __attribute__((ext_vector_type(4)));
  static_assert(NB % PB == 0, "blocks come in load groups");
  auto load_group = [&](int g0, tg_u32x4 (&dst)[PB][KS]) {
#pragma unroll
    for (int p2 = 0; p2 < PB; ++p2) {
      const int nt = g0 + p2;
      const int nn = nt < nb_real ? nt : nb_real - 1;  // blocks past the tensor re-read its last one and are masked
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) dst[p2][ks] = *(const tg_u32x4*)&pbase[((long)nn * KS + ks) * 64];
    }
  };
  // bias (B, N, h_kv, G) fp32: the G values of a (chunk, KV head) are contiguous; accumulator row
  // 4j+i is head (4j+i) % GMAX
  auto bias_of = [&](int c, float (&bv)[4]) {  // c < 16 * NB
    const float4 v = *(const float4*)bias_s[c];
    const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) bv[i] = e[i % GMAX];
  };
  auto xch = [&](int buf, int p2, int w, int i, int l) -> float& {
    return xbuf[(((buf * PB + p2) * TGW + w) * 4 + i) * 64 + l];
  };
  auto use_group = [&](int g0, const tg_u32x4 (&src)[PB][KS]) {
    const int buf = (g0 / PB) & 1;
    if constexpr (PERQ) {
#pragma unroll
      for (int p2 = 0; p2 < PB; ++p2) {
        const int nt = g0 + p2;
        float bv[4];
        if constexpr (BIAS && !HALF) bias_of(nt * 16 + col, bv);
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag[ks], __builtin_bit_cast(bf16x8_t, src[p2][ks]), acc, 0, 0, 0);
        // rows 4j+i are queries here; the bias of (chunk, head = this wavefront)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = __fmul_rn(acc[i], sm_scale);
          if constexpr (BIAS && !HALF) v = __fadd_rn(v, bv[wave]);  // (HALF: added by the reader, which has its heads' bias)
          xch(buf, p2, wave, i, lane) = v;
        }
      }
      __syncthreads();
    }
#pragma unroll
    for (int p2 = 0; p2 < PB; ++p2) {
      const int nt = g0 + p2;
      float bv[4];
      if constexpr (BIAS && (!PERQ || HALF)) bias_of(nt * 16 + col, bv);
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
      if constexpr (!PERQ) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag[ks], __builtin_bit_cast(bf16x8_t, src[p2][ks]), acc, 0, 0, 0);
      }
      const int c = nt * 16 + col;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v;
        if constexpr (PERQ) {
          // row (query j of this wavefront, head i of its heads): that head's wavefront's register j of
          // the lane that holds this chunk column for the queries 4 * pw .. 4 * pw + 3
          v = xch(buf, p2, gofs + i, j, col + 16 * pw);
          if constexpr (BIAS && HALF) v = __fadd_rn(v, bv[i]);
        } else {
          v = __fmul_rn(acc[i], sm_scale);
          if constexpr (BIAS) v = __fadd_rn(v, bv[i]);
        }
        if (nt >= NMASK) v = (c < lim[i]) ? v : HILS_NEG_INF;
        x[nt][i] = v;
        // (pinned here: left alone the compiler forms some of these sums only where they are used and
        // keeps product and bias alive in their place, which this kernel has no registers for)
        if constexpr (BIAS && (!PERQ || HALF)) asm volatile("" : "+v"(x[nt][i]));
      }
      if (EXPORT) {
        if (sel_logits_out && c < N) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (rowok[i]) {
              const int r = 4 * j + i;
              sel_logits_out[(((b * L + t0 + r / GMAX) * (long)h_kv + hk) * G + gofs + r % GMAX) * N + c] = x[nt][i];
            }
        }
      }
    }
  };
  {
    tg_u32x4 ba[PB][KS], bb2[PB][KS];
    load_group(0, ba);
#pragma unroll
    for (int g0 = 0; g0 < NB; g0 += 2 * PB) {
      // scheduling barriers: left to itself the compiler, when registers are short, sinks the loads
      // of the next group to their uses and every MFMA then waits a full memory latency
      if (g0 + PB < NB) load_group(g0 + PB, bb2);
      __builtin_amdgcn_sched_barrier(0);
      use_group(g0, ba);
      __builtin_amdgcn_sched_barrier(0);
      if (g0 + PB < NB) {
        if (g0 + 2 * PB < NB) load_group(g0 + 2 * PB, ba);
        __builtin_amdgcn_sched_barrier(0);
        use_group(g0 + PB, bb2);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  if (PERQ && !HALF && t0 >= t_end) return;  // no barrier behind this point
  // ---- lse_total per row = logaddexp(lse_swa, logsumexp of the visible logits) ----
  float lse_tot[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float m = HILS_NEG_INF;
#pragma unroll
    for (int nt = 0; nt < NB; ++nt) m = fmaxf(m, x[nt][i]);
    m = tg_row_max_f(m);
    const float m2 = (m > HILS_NEG_INF) ? m * HILS_LOG2E : 0.f;
    float l = 0.f;
#pragma unroll
    for (int nt = 0; nt < NB; ++nt) l += __builtin_amdgcn_exp2f(fmaf(x[nt][i], HILS_LOG2E, -m2));
    l = row_sum<16>(l);
    const float hils2 = (l > 0.f) ? m2 + __builtin_amdgcn_logf(l) : HILS_NEG_INF;  // log2 domain
    const float swa2 = swa[i] * HILS_LOG2E;
    const float mx = fmaxf(swa2, hils2), mn = fminf(swa2, hils2);
    float tot2 = mx;
    if (mn > HILS_NEG_INF) tot2 = mx + __builtin_amdgcn_logf(1.f + __builtin_amdgcn_exp2f(mn - mx));
    // a row that does not exist (a padding head of a group of three, a query past the end) must not
    // reach the selection: its logits are not masked in the blocks every real row sees (they are 0 there)
    const float lt = tot2 * HILS_LN2;
    if (lse_total_out && col == 0 && rowok[i]) {
      const int r = 4 * j + i;
      lse_total_out[((b * L + t0 + r / GMAX) * (long)h_kv + hk) * G + gofs + r % GMAX] = lt;
    }
    // A row that sees no chunk and has lse_swa = -inf has lse_total = -inf; its logits are all -inf,
    // and -inf - -inf would be a NaN, which this file is compiled not to expect: such a row subtracts
    // 0 instead (its scores stay -inf, nothing is selected).
    lse_tot[i] = rowok[i] ? (tot2 > HILS_NEG_INF ? lt : 0.f) : __builtin_inff();
  }

  // outputs start as "no winner"
  auto clear_stage = [&]() {
    for (int e = lane; e < NQ * 8; e += 64) ((int4*)stage_i)[e] = make_int4(-1, -1, -1, -1);
    ((uint4*)stage_s)[lane] = make_uint4(0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u);  // 512 x -inf
    __builtin_amdgcn_wave_barrier();
  };
  if constexpr (!OVER) clear_stage();  // (OVER: once the memory is the stage's)

  // ---- selection, one query of every lane row at a time ----
#pragma unroll
  for (int u = 0; u < QPL; ++u) {
    const int qi = j * QPL + u;  // query of the wavefront this lane row works on
    // selection score of chunk nt*16+col: max over the heads of (logit - lse_total), one fp32
    // subtraction each; -inf where the chunk is not visible (lse_tot is never -inf, so no NaN is
    // formed).  Scores are compared as floats (+0 == -0, as in the reference's sort); only the few
    // candidates of the threshold search are turned into integer keys.
    float key[NB];
#pragma unroll
    for (int nt = 0; nt < NB; ++nt) {
      float best = HILS_NEG_INF;
#pragma unroll
      for (int e = 0; e < GMAX; ++e) best = fmaxf(best, __fsub_rn(x[nt][u * GMAX + e], lse_tot[u * GMAX + e]));
      key[nt] = best;
    }
    if constexpr (HALF) {
      // the pair's scores: the first half's go to LDS, the second half's wavefront forms the maxima and
      // leaves them there for the first (both go on with the same numbers, whatever a maximum of +0
      // and -0 is).  A pair without queries takes part in the barriers and leaves behind them.
      float* kxp = xbuf + (OVER ? 0 : XCH_F) + pw * NB * 64 + lane;
      if constexpr (OVER) __syncthreads();  // everybody is through with the accumulators in this memory
      if (half == 0) {
#pragma unroll
        for (int nt = 0; nt < NB; ++nt) kxp[nt * 64] = key[nt];
      }
      __syncthreads();
      if (half == 1) {
#pragma unroll
        for (int nt = 0; nt < NB; ++nt) {
          key[nt] = fmaxf(key[nt], kxp[nt * 64]);
          kxp[nt * 64] = key[nt];
        }
      }
      __syncthreads();
      if (half == 0) {
#pragma unroll
        for (int nt = 0; nt < NB; ++nt) key[nt] = kxp[nt * 64];
      }
      if constexpr (OVER) {
        __syncthreads();  // the selection areas lie over the scores
        if (t0 >= t_end) return;
        clear_stage();
      }
    }
    // the two largest scores of the lane, the number of valid ones
    float m1 = HILS_NEG_INF, m2 = HILS_NEG_INF;
    int nv = 0;
#pragma unroll
    for (int nt = 0; nt < NB; ++nt) {
      const float kk = key[nt];
      m2 = fmaxf(m2, fminf(kk, m1));
      m1 = fmaxf(m1, kk);
      nv += (kk > HILS_NEG_INF) ? 1 : 0;
    }
    const int nvalid = tg_row_sum_i(nv);
    float Tf = HILS_NEG_INF;  // every valid score wins ...
    int cutoff = -1;          // ... and among the scores equal to Tf those with a chunk index <= cutoff
    bool cut = false;         // cutoff excludes some of them
    if (__any(nvalid > topk)) {
      const bool want = nvalid > topk;
      const float hi = tg_row_max_f(m1);
      const float bound = tg_row_min_f(m2);  // >= 2 scores per lane reach it: >= 32 >= topk in all
      // a query that keeps everything has no candidates; -inf (a lane with fewer than two scores)
      // makes every register one, which sends the wavefront to the search over all scores below
      const float cbound = want ? bound : __builtin_inff();
      int nc = 0;
#pragma unroll
      for (int nt = 0; nt < NB; ++nt) nc += (key[nt] >= cbound) ? 1 : 0;
      const int ntot = tg_row_sum_i(nc);
      uint32_t T;
      bool exact = false;
      if (!__any(want & ((ntot > TG_CAND) | !(bound > HILS_NEG_INF)))) {
        // compact the candidates of the lane row (any order) and take at most 8 per lane
        int pos = tg_row_excl_scan(nc);
#pragma unroll
        for (int nt = 0; nt < NB; ++nt) {
          if (key[nt] >= cbound) {
            cand[j][pos] = __float_as_uint(key[nt]);
            ++pos;
          }
        }
        __builtin_amdgcn_wave_barrier();
        uint32_t ck[TG_CAND / 16];
#pragma unroll
        for (int e = 0; e < TG_CAND / 16; ++e)
          ck[e] = (e * 16 + col < ntot) ? tg_score_key(__uint_as_float(cand[j][e * 16 + col])) : 0u;
        __builtin_amdgcn_wave_barrier();
        const uint32_t lo_k = tg_score_key(want ? bound : 0.f), hi_k = tg_score_key(want ? hi : 0.f);
        T = tg_kth_largest(ck, lo_k, hi_k, topk, want & (ntot != topk), exact);
        if (ntot == topk) {  // exactly the candidates win
          T = lo_k;
          exact = true;
        }
      } else {
        // rare: too many scores at the bound (many equal ones) or a lane with fewer than two
        // scores while the query has more than topk: search over all scores of the lane row
        uint32_t uk[NB];
        uint32_t mn = 0xffffffffu;
#pragma unroll
        for (int nt = 0; nt < NB; ++nt) {
          uk[nt] = (key[nt] > HILS_NEG_INF) ? tg_score_key(key[nt]) : 0u;
          if (uk[nt] != 0u) mn = uk[nt] < mn ? uk[nt] : mn;
        }
        mn = tg_row_min_u(mn);
        const uint32_t hi_k = (hi > HILS_NEG_INF) ? tg_score_key(hi) : 1u;
        T = tg_kth_largest(uk, mn == 0xffffffffu ? 1u : mn, hi_k, topk, want, exact);
      }
      if (want) {
        Tf = tg_key_score(T);
        cutoff = 1 << 30;
      }
      // ties at the threshold (only where the search ran down to the last bit): the lowest chunk
      // indices win
      const bool loose = want & !exact;
      if (__any(loose)) {
        int ngt = 0, neq = 0;
#pragma unroll
        for (int nt = 0; nt < NB; ++nt) {
          ngt += (key[nt] > Tf) ? 1 : 0;
          neq += (key[nt] == Tf) ? 1 : 0;
        }
        ngt = tg_row_sum_i(ngt);
        neq = tg_row_sum_i(neq);
        const int need = topk - ngt;  // scores equal to Tf still to take
        if (__any(loose & (neq > need))) {
          // smallest index C with count(score == Tf and chunk <= C) >= need, bit by bit (chunks < 512)
          int C = 0;
          for (int bit = 8; bit >= 0; --bit) {
            const int c2 = C | (1 << bit);  // count the ties below c2
            int cl = 0;
#pragma unroll
            for (int nt = 0; nt < NB; ++nt) cl += ((key[nt] == Tf) & (nt * 16 + col < c2)) ? 1 : 0;
            if (tg_row_sum_i(cl) < need) C = c2;
          }
          if (loose & (neq > need)) {
            cutoff = C;
            cut = true;
          }
        }
      }
    }
    // winners of this lane as a bit mask over its blocks
    uint32_t mask = 0u;
    if (__any(cut)) {
#pragma unroll
      for (int nt = NB - 1; nt >= 0; --nt) {
        const bool win = (key[nt] > Tf) | ((key[nt] == Tf) & (nt * 16 + col <= cutoff));
        mask = (mask << 1) | (win ? 1u : 0u);
      }
    } else {
      // no tie to break in this wavefront: everything from the threshold up wins (a query that keeps
      // all its valid scores has Tf = -inf: the lowest finite float stands in for it)
      const float Tlow = fmaxf(Tf, -3.402823466e38f);
#pragma unroll
      for (int nt = NB - 1; nt >= 0; --nt) mask = (mask << 1) | ((key[nt] >= Tlow) ? 1u : 0u);
    }
    // 512-bit map of the winning chunks (chunk c = bit c): word w holds blocks 2w and 2w+1
    words[j][col] = 0u;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int w = 0; w < (NB + 1) / 2; ++w) {
      const uint32_t bits = (((mask >> (2 * w)) & 1u) << col) | (((mask >> (2 * w + 1)) & 1u) << (16 + col));
      if (bits) atomicOr(&words[j][w], bits);
    }
    __builtin_amdgcn_wave_barrier();
    {
      const int pc = __popc(words[j][col]);
      wbase[j][col] = (uint32_t)tg_row_excl_scan(pc);
    }
    __builtin_amdgcn_wave_barrier();
    // every winner: its slot = winners with a lower chunk index; index and raw scores to the stage
#pragma unroll
    for (int nt = 0; nt < NB; ++nt) {
      if ((mask >> nt) & 1u) {
        const int c = nt * 16 + col, w = c >> 5;
        const int slot = (int)wbase[j][w] + __popc(words[j][w] & ((1u << (c & 31)) - 1u));
        if (slot < topk) {
          stage_i[qi * 32 + slot] = c;
          // the heads of the winner in one store (heads past G are never read back)
          bf16_t* dst = &stage_s[(qi * 32 + slot) * GMAX];
          float raw[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) raw[i] = x[nt][i];
          if constexpr (BIAS) {  // the returned scores carry no bias
            float bv[4];
            bias_of(c, bv);
#pragma unroll
            for (int i = 0; i < 4; ++i) raw[i] = __fsub_rn(raw[i], bv[i]);
          }
          if constexpr (GMAX == 4) {
            *(uint2*)dst = make_uint2(pack_bf2(raw[0], raw[1]), pack_bf2(raw[2], raw[3]));
          } else if constexpr (GMAX == 2) {
            *(uint32_t*)dst = pack_bf2(raw[u * 2], raw[u * 2 + 1]);
          } else {
            *dst = f2bf(raw[u]);
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  // ---- write out: indices (B,L,h_kv,topk) int32, scores (B,L,h_kv,G,topk) bf16 ----
  // the stage is walked in its own padded order (32 slots per row): no division by topk, and a
  // lane row stores consecutive slots of one output row
  const long row0 = ((b * L + t0) * (long)h_kv + hk);  // (query t0, this KV head); the next query is h_kv further
  int32_t* ind0 = indices + row0 * topk;
  bf16_t* sc0 = scores + row0 * G * topk;
#pragma unroll
  for (int e0 = 0; e0 < NQ * 32; e0 += 64) {
    const int e = e0 + lane, qi = e >> 5, k = e & 31;
    if ((k < topk) & (t0 + qi < t_end) & (half == 0)) ind0[qi * h_kv * topk + k] = stage_i[e];
  }
#pragma unroll
  for (int e0 = 0; e0 < NQ * GMAX * 32; e0 += 64) {
    const int e = e0 + lane, k = e & 31, g = (e >> 5) % GMAX, qi = e / (32 * GMAX);
    if ((k < topk) & (gofs + g < G) & (t0 + qi < t_end))
      sc0[(qi * h_kv * G + gofs + g) * topk + k] = stage_s[(qi * 32 + k) * GMAX + g];
  }
}

// plain: no Gumbel noise and no drop mask (a bias is fine)
bool hils_topk_group_covers(int N, int G, int D, int topk, int per_qhead, bool plain) {
  if (per_qhead && (G < 2 || G > 8)) return false;  // (one head a group: the keys are shared anyway)
  return plain && G >= 1 && G <= 8 && (D == 64 || D == 128) && N <= 16 * TG_NB && topk <= 32;
}

template <int GMAX, int KS, bool BIAS, bool PERQ, bool HALF>
static void tg_launch_range(int NB, bool exp, dim3 grid, hipStream_t st, const bf16_t* q, const uint4* pk,
                            const float* lse_swa, const float* bias, int32_t* indices, bf16_t* scores, float* lse_total,
                            float* sel_logits, int L, int N, int h_kv, int G, int topk, int block_size,
                            int window_size, int causal, int q_offset, float sm_scale, int t_base, int t_end,
                            int lse_bf16) {
#define TG_CALL(NB_, EX_)                                                                              \
  hipLaunchKernelGGL((topk_fwd_group_kernel<GMAX, KS, NB_, EX_, BIAS, PERQ, HALF>), grid, dim3(64 * (PERQ ? (HALF ? 8 : 4) : TG_WAVES)), 0, st, q, pk, lse_swa, \
                     bias, indices, scores, lse_total, sel_logits, L, N, h_kv, G, topk, block_size, window_size, \
                     causal, q_offset, sm_scale, t_base, t_end, bs_shift, lse_bf16)
  const int bs_shift = (block_size > 0 && (block_size & (block_size - 1)) == 0) ? __builtin_ctz(block_size) : -1;
  if (exp) { TG_CALL(32, true); return; }
  switch (NB) {
    case 8: TG_CALL(8, false); break;
    case 16: TG_CALL(16, false); break;
    case 24: TG_CALL(24, false); break;
    default: TG_CALL(32, false); break;
  }
#undef TG_CALL
}

// lmk_packed: the chunk keys in topk_pack_lmk_kernel's order.  The queries are split by how many
// chunks they can see (at most 8, 16, 24 or 32 blocks of 16) into one launch each.
int hils_topk_group_launch(const void* q, const void* lmk_packed, const float* lse_swa, const float* bias,
                           int32_t* indices,
                           void* scores, float* lse_total, float* sel_logits, int B, int L, int N, int h_kv,
                           int G, int D, int topk, int block_size, int window_size, int causal, int q_offset,
                           float sm_scale, int lse_bf16, int per_qhead, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  // rows of a tile: queries x 1, 2 or 4 heads (three heads, and two with a key per query head, whose
  // wavefronts are one per head of four: padding rows)
  const int GM = (G == 1) ? 1 : ((G == 2 && !per_qhead) ? 2 : 4);
  const bool halves = G > 4;  // two wavefronts per four queries
  const int QGROUPS = halves ? (per_qhead ? 4 : 1) : (per_qhead ? 4 : TG_WAVES);  // wavefronts (pairs) of a workgroup with queries of their own
  const int NQ = 16 / GM;
  const bool exp = sel_logits != nullptr;
  auto limit_of = [&](int tq) -> int {
    int lm = causal ? visible_limit(tq + q_offset, window_size, block_size) : N;
    return lm < 0 ? 0 : (lm > N ? N : lm);
  };
  int t = 0;
  while (t < L) {
    // the bucket of query t and the last query that still falls into it (limits grow with t)
    int NB = 32, t_hi = L;
    if (!exp) {
      const int lm = limit_of(t);
      NB = lm <= 128 ? 8 : (lm <= 256 ? 16 : (lm <= 384 ? 24 : 32));
      if (NB < 32) {
        int lo = t, hi = L;  // first query whose limit exceeds 16 * NB
        while (lo < hi) {
          const int mid = lo + (hi - lo) / 2;
          if (limit_of(mid) <= 16 * NB) lo = mid + 1; else hi = mid;
        }
        t_hi = lo;
      }
    }
    dim3 grid((t_hi - t + NQ * QGROUPS - 1) / (NQ * QGROUPS), h_kv, B);
#define TG_RANGE_B(G_, KS_, B_, P_, H_)                                                               \
  tg_launch_range<G_, KS_, B_, P_, H_>(NB, exp, grid, st, (const bf16_t*)q, (const uint4*)lmk_packed, lse_swa, bias, \
                               indices, (bf16_t*)scores, lse_total, sel_logits, L, N, h_kv, G, topk,   \
                               block_size, window_size, causal, q_offset, sm_scale, t, t_hi, lse_bf16)
#define TG_RANGE(G_, KS_, P_, H_)                                                                     \
  do {                                                                                                \
    if (bias) TG_RANGE_B(G_, KS_, true, P_, H_); else TG_RANGE_B(G_, KS_, false, P_, H_);             \
  } while (0)
    if (GM == 1) { if (D == 64) TG_RANGE(1, 2, false, false); else TG_RANGE(1, 4, false, false); }
    else if (GM == 2) { if (D == 64) TG_RANGE(2, 2, false, false); else TG_RANGE(2, 4, false, false); }
    else if (halves && per_qhead) { if (D == 64) TG_RANGE(4, 2, true, true); else TG_RANGE(4, 4, true, true); }
    else if (halves) { if (D == 64) TG_RANGE(4, 2, false, true); else TG_RANGE(4, 4, false, true); }
    else if (per_qhead) { if (D == 64) TG_RANGE(4, 2, true, false); else TG_RANGE(4, 4, true, false); }
    else { if (D == 64) TG_RANGE(4, 2, false, false); else TG_RANGE(4, 4, false, false); }
#undef TG_RANGE
#undef TG_RANGE_B
    t = t_hi;
  }
  return HILS_OK;
}
