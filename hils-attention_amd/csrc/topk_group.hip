// Prefill top-k chunk selection, one pass over the chunk keys.
//
// One wavefront owns 16/GMAX consecutive queries of a (batch, KV head): the 16 rows of its MFMA
// tile are (queries x the GMAX heads of the KV head).  It streams the chunk keys once (B operands,
// 16 chunks per block, repacked into operand order by topk_pack_lmk_kernel) and keeps every scaled
// logit in registers: accumulator register i of block nt in lane (col, j) is row 4j+i, chunk
// nt*16+col, so a query's logits for up to 512 chunks lie in the 16 lanes of one lane row, 32 per
// lane.  From there, without touching memory again:
//   * the log-sum-exp of every row (in-lane maxima and sums, one 16-lane reduction per row),
//   * the selection key of every (query, chunk): max over the heads of logit - lse_total, as an
//     order-preserving unsigned key (in-lane: the heads of a query are registers of one lane),
//   * the top-K per query, the four lane rows working on four queries at once: the K-th largest
//     key is bracketed from the two largest keys of every lane (their minimum over the lanes is a
//     lower bound with at least 32 keys above it), the keys above the bound (about 1.5 K of 512)
//     are compacted through LDS to at most 8 per lane and the exact threshold is found on those by
//     a bitwise search whose counts are 16-lane DPP reductions (no ballots, no scalar round trip);
//     ties at the threshold go to the lower chunk indices,
//   * the ascending order of the winners from a 512-bit map of the winning chunks in LDS
//     (rank = set bits below the chunk), and the winners' raw scores straight from the logits.
// Covers shared chunk keys, G <= 4, D in {64, 128}, N <= 512, topk <= 32, no bias / Gumbel noise /
// drop mask; everything else runs on the kernels of topk.hip.
#include <type_traits>
#include "decode_rows.h"
#include "../../include/hils_amd.h"

#define TG_NB 32     // chunk blocks of 16 a lane row can hold (N <= 512)
#define TG_CAND 128  // compacted candidates per query (8 per lane)

__device__ __forceinline__ uint32_t tg_score_key(float f) {  // larger float <-> larger key; 0 = not a candidate
  if (!(f > HILS_NEG_INF)) return 0u;  // -inf and NaN
  f = f + 0.0f;                        // -0 -> +0
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
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
// exclusive prefix sum over the 16 lanes of a lane row (lanes shifted in from outside read 0)
__device__ __forceinline__ int tg_row_excl_scan(int x) {
  int s = x;
  s += __builtin_amdgcn_update_dpp(0, s, 0x111, 0xF, 0xF, true);  // row_shr:1
  s += __builtin_amdgcn_update_dpp(0, s, 0x112, 0xF, 0xF, true);  // row_shr:2
  s += __builtin_amdgcn_update_dpp(0, s, 0x114, 0xF, 0xF, true);  // row_shr:4
  s += __builtin_amdgcn_update_dpp(0, s, 0x118, 0xF, 0xF, true);  // row_shr:8
  return s - x;
}

// K-th largest of the keys a lane row holds, NE per lane (0 = no key), all non-zero keys in
// [lo, hi] and at least K of them: returns T with count(key >= T) >= K > count(key > T).
template <int NE>
__device__ __forceinline__ uint32_t tg_kth_largest(const uint32_t (&k)[NE], uint32_t lo, uint32_t hi, int K) {
  const uint32_t diff = lo ^ hi;
  // bits above the highest differing one are shared by every key; the search runs over the rest,
  // as many steps as the lane row with the widest range needs (the loop is wavefront-uniform)
  const int top = diff ? 31 - __clz((int)diff) : -1;
  uint32_t T = (top >= 31 || top < 0) ? (top < 0 ? lo : 0u) : (lo & ~((2u << top) - 1u));
  int top_w = top;
  top_w = max(top_w, __builtin_amdgcn_readlane(top, 16));
  top_w = max(top_w, __builtin_amdgcn_readlane(top, 32));
  top_w = max(top_w, __builtin_amdgcn_readlane(top, 48));
  top_w = max(top_w, __builtin_amdgcn_readlane(top, 0));
  for (int bit = top_w; bit >= 0; --bit) {
    const uint32_t c = T | (1u << bit);
    int cl = 0;
#pragma unroll
    for (int e = 0; e < NE; ++e) cl += (k[e] >= c) ? 1 : 0;
    const int cnt = tg_row_sum_i(cl);
    if (bit <= top && cnt >= K) T = c;
  }
  return T;
}

// NB: chunk blocks the launch covers (every query of the launch sees at most 16*NB chunks and at
// least 16*(NB-9)+1, so only the last nine blocks can hold invisible chunks); t_base: first query.
// Everything is unrolled over the NB blocks: register-resident data has no other way of being
// indexed, and the host splits a call into launches by NB so that early queries do not pay for 32.
#define TG_WAVES 4  // wavefronts per workgroup, each with queries of its own (they never synchronise)
template <int GMAX, int KS, int NB, bool EXPORT>
__global__ void __launch_bounds__(64 * TG_WAVES)
    __attribute__((amdgpu_waves_per_eu(NB <= 8 ? 5 : (NB <= 16 ? 4 : (NB <= 24 ? 3 : 2)))))
topk_fwd_group_kernel(const bf16_t* __restrict__ q, const uint4* __restrict__ lmk_packed,
                      const float* __restrict__ lse_swa, int32_t* __restrict__ indices,
                      bf16_t* __restrict__ scores, float* __restrict__ lse_total_out,
                      float* __restrict__ sel_logits_out, int L, int N, int h_kv, int G, int topk,
                      int block_size, int window_size, int causal, int q_offset, float sm_scale,
                      int t_base, int t_end) {
  constexpr int D = KS * 32;
  constexpr int QPL = 4 / GMAX;   // queries per lane (its four accumulator rows)
  constexpr int NQ = 16 / GMAX;   // queries per wavefront
  constexpr int NMASK = EXPORT ? 0 : (NB > 9 ? NB - 9 : 0);  // blocks below it are visible to every row
  __shared__ uint32_t cand_w[TG_WAVES][4][TG_CAND];          // compacted candidate keys, per lane row
  __shared__ uint32_t words_w[TG_WAVES][4][16], wbase_w[TG_WAVES][4][16];  // winner map of a query and its word prefix counts
  __shared__ int stage_i_w[TG_WAVES][NQ * 32];               // winners' chunk indices, [query][slot]
  __shared__ __align__(16) bf16_t stage_s_w[TG_WAVES][NQ * GMAX * 32];  // their raw scores, [query][head][slot]

  const int wave = threadIdx.x >> 6;
  uint32_t (*cand)[TG_CAND] = cand_w[wave];
  uint32_t (*words)[16] = words_w[wave];
  uint32_t (*wbase)[16] = wbase_w[wave];
  int* stage_i = stage_i_w[wave];
  bf16_t* stage_s = stage_s_w[wave];
  const int lane = threadIdx.x & 63, col = lane & 15, j = lane >> 4;
  const int t0 = t_base + (blockIdx.x * TG_WAVES + wave) * NQ;
  if (t0 >= t_end) return;
  const int hk = blockIdx.y;
  const long b = blockIdx.z;

  auto limit_of = [&](int tq) -> int {
    int lm = causal ? visible_limit(tq + q_offset, window_size, block_size) : N;
    return lm < 0 ? 0 : (lm > N ? N : lm);
  };
  // accumulator row 4j+i <-> (query t0 + (4j+i)/GMAX, head (4j+i)%GMAX)
  int lim[4];
  bool rowok[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * j + i;
    const int tq = t0 + r / GMAX;
    rowok[i] = tq < t_end && (r % GMAX) < G;
    lim[i] = rowok[i] ? limit_of(tq) : 0;
  }
  const int nb_real = (N + 15) / 16;  // blocks the packed chunk keys hold

  // query rows as A operands
  bf16x8_t afrag[KS];
  {
    const int r = lane & 15;
    const int g = r % GMAX, tq = t0 + r / GMAX;
    const bool ok = tq < t_end && g < G;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 v = *(const uint4*)(q + (((b * L + (ok ? tq : t0)) * h_kv + hk) * (long)G + (ok ? g : 0)) * D + ks * 32 + j * 8);
      if (!ok) v = make_uint4(0, 0, 0, 0);
      afrag[ks] = *(bf16x8_t*)&v;
    }
  }
  float swa[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * j + i;
    const int tq = t0 + r / GMAX, g = r % GMAX;
    const float x = lse_swa[((b * L + (rowok[i] ? tq : t0)) * (long)h_kv + hk) * G + (rowok[i] ? g : 0)];
    swa[i] = rowok[i] ? x : HILS_NEG_INF;
  }

  // ---- the logits: x[nt][i] = sm_scale * <q_row, lmk_chunk>, -inf where the chunk is not visible ----
  const uint4* pbase = lmk_packed + ((b * h_kv + hk) * (long)nb_real * KS) * 64 + lane;
  float x[NB][4];
  // the keys of two blocks travel together, one such group ahead of their use (the loads of a
  // block issued right before its MFMAs would each expose a full memory latency)
  typedef unsigned tg_u32x4 __attribute__((ext_vector_type(4)));
  constexpr int PB = 2;  // blocks per load group
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
  auto use_group = [&](int g0, const tg_u32x4 (&src)[PB][KS]) {
#pragma unroll
    for (int p2 = 0; p2 < PB; ++p2) {
      const int nt = g0 + p2;
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag[ks], __builtin_bit_cast(bf16x8_t, src[p2][ks]), acc, 0, 0, 0);
      const int c = nt * 16 + col;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = __fmul_rn(acc[i], sm_scale);
        if (nt >= NMASK) v = (c < lim[i]) ? v : HILS_NEG_INF;
        x[nt][i] = v;
      }
      if (EXPORT) {
        if (sel_logits_out && c < N) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (rowok[i]) {
              const int r = 4 * j + i;
              sel_logits_out[(((b * L + t0 + r / GMAX) * (long)h_kv + hk) * G + r % GMAX) * N + c] = x[nt][i];
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
      if (g0 + PB < NB) load_group(g0 + PB, bb2);
      use_group(g0, ba);
      if (g0 + PB < NB) {
        if (g0 + 2 * PB < NB) load_group(g0 + 2 * PB, ba);
        use_group(g0 + PB, bb2);
      }
    }
  }

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
    lse_tot[i] = tot2 * HILS_LN2;
    if (lse_total_out && col == 0 && rowok[i]) {
      const int r = 4 * j + i;
      lse_total_out[((b * L + t0 + r / GMAX) * (long)h_kv + hk) * G + r % GMAX] = lse_tot[i];
    }
  }

  // outputs start as "no winner"
  for (int e = lane; e < NQ * 32; e += 64) stage_i[e] = -1;
  for (int e = lane; e < NQ * GMAX * 32; e += 64) stage_s[e] = 0xff80;  // -inf
  __builtin_amdgcn_wave_barrier();

  // ---- selection, one query of every lane row at a time ----
#pragma unroll
  for (int u = 0; u < QPL; ++u) {
    const int qi = j * QPL + u;  // query of the wavefront this lane row works on
    // selection key of chunk nt*16+col: max over the heads of (logit - lse_total), one fp32
    // subtraction each; -inf and NaN give key 0 (-inf - lse is -inf or NaN, and fmaxf skips NaN)
    uint32_t key[NB];
#pragma unroll
    for (int nt = 0; nt < NB; ++nt) {
      float best = HILS_NEG_INF;
#pragma unroll
      for (int e = 0; e < GMAX; ++e) best = fmaxf(best, __fsub_rn(x[nt][u * GMAX + e], lse_tot[u * GMAX + e]));
      key[nt] = tg_score_key(best);
    }
    // the two largest keys of the lane, the number of valid ones
    uint32_t m1 = 0u, m2 = 0u;
    int nv = 0;
#pragma unroll
    for (int nt = 0; nt < NB; ++nt) {
      const uint32_t kk = key[nt];
      const uint32_t lo2 = kk < m1 ? kk : m1;
      m2 = lo2 > m2 ? lo2 : m2;
      m1 = kk > m1 ? kk : m1;
      nv += kk != 0u;
    }
    const int nvalid = tg_row_sum_i(nv);
    uint32_t T = 1u;        // every valid key wins ...
    int cutoff = 1 << 30;   // ... and among the keys equal to T those with a chunk index <= cutoff
    if (__any(nvalid > topk)) {
      const uint32_t hi = tg_row_max_u(m1);
      const uint32_t bound = tg_row_min_u(m2);  // >= 2 keys per lane reach it: >= 32 >= topk in all
      int nc = 0;
#pragma unroll
      for (int nt = 0; nt < NB; ++nt) nc += (key[nt] >= bound && key[nt] != 0u) ? 1 : 0;
      const int ntot = tg_row_sum_i(nc);
      const bool want = nvalid > topk;
      if (!__any(want && (ntot > TG_CAND || bound == 0u))) {
        // compact the candidates of the lane row (any order) and take at most 8 per lane
        int pos = tg_row_excl_scan(nc);
#pragma unroll
        for (int nt = 0; nt < NB; ++nt) {
          if (key[nt] >= bound && key[nt] != 0u) {
            cand[j][pos] = key[nt];
            ++pos;
          }
        }
        __builtin_amdgcn_wave_barrier();
        uint32_t ck[TG_CAND / 16];
#pragma unroll
        for (int e = 0; e < TG_CAND / 16; ++e) ck[e] = (e * 16 + col < ntot) ? cand[j][e * 16 + col] : 0u;
        __builtin_amdgcn_wave_barrier();
        const uint32_t Tc = tg_kth_largest(ck, bound, hi, topk);
        if (want) T = Tc;
      } else {
        // rare: too many keys at the bound (many equal scores) or a lane with fewer than two
        // keys while the query has more than topk: search over all keys of the lane row
        uint32_t mn = 0xffffffffu;
#pragma unroll
        for (int nt = 0; nt < NB; ++nt)
          if (key[nt] != 0u) mn = key[nt] < mn ? key[nt] : mn;
        mn = tg_row_min_u(mn);
        const uint32_t Tc = tg_kth_largest(key, mn == 0xffffffffu ? 1u : mn, hi ? hi : 1u, topk);
        if (want) T = Tc;
      }
      // ties at the threshold: the lowest chunk indices win
      int ngt = 0, neq = 0;
#pragma unroll
      for (int nt = 0; nt < NB; ++nt) {
        ngt += (key[nt] > T) ? 1 : 0;
        neq += (key[nt] == T) ? 1 : 0;
      }
      ngt = tg_row_sum_i(ngt);
      neq = tg_row_sum_i(neq);
      const int need = topk - ngt;  // keys equal to T still to take (>= 1 when want)
      if (__any(want && neq > need)) {
        // smallest index C with count(key == T and chunk <= C) >= need, bit by bit (chunks < 512)
        int C = 0;
        for (int bit = 8; bit >= 0; --bit) {
          const int c2 = C | (1 << bit);  // count the ties below c2
          int cl = 0;
#pragma unroll
          for (int nt = 0; nt < NB; ++nt) cl += (key[nt] == T && nt * 16 + col < c2) ? 1 : 0;
          if (tg_row_sum_i(cl) < need) C = c2;
        }
        if (want && neq > need) cutoff = C;
      }
    }
    // winners of this lane as a bit mask over its blocks
    uint32_t mask = 0u;
#pragma unroll
    for (int nt = NB - 1; nt >= 0; --nt) {
      const bool win = key[nt] != 0u && (key[nt] > T || (key[nt] == T && nt * 16 + col <= cutoff));
      mask = (mask << 1) | (win ? 1u : 0u);
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
#pragma unroll
          for (int e = 0; e < GMAX; ++e)
            if (e < G) stage_s[(qi * GMAX + e) * 32 + slot] = f2bf(x[nt][u * GMAX + e]);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  // ---- write out: indices (B,L,h_kv,topk) int32, scores (B,L,h_kv,G,topk) bf16 ----
  for (int e = lane; e < NQ * topk; e += 64) {
    const int qi = e / topk, k = e - qi * topk;
    if (t0 + qi < t_end) indices[((b * L + t0 + qi) * (long)h_kv + hk) * topk + k] = stage_i[qi * 32 + k];
  }
  for (int e = lane; e < NQ * G * topk; e += 64) {
    const int qi = e / (G * topk), rem = e - qi * (G * topk);
    const int g = rem / topk, k = rem - g * topk;
    if (t0 + qi < t_end)
      scores[(((b * L + t0 + qi) * (long)h_kv + hk) * G + g) * topk + k] = stage_s[(qi * GMAX + g) * 32 + k];
  }
}

bool hils_topk_group_covers(int N, int G, int D, int topk, int per_qhead, bool plain) {
  return plain && !per_qhead && (G == 1 || G == 3 || G == 4) && (D == 64 || D == 128) && N <= 16 * TG_NB &&
         topk <= 32;
}

template <int GMAX, int KS>
static void tg_launch_range(int NB, bool exp, dim3 grid, hipStream_t st, const bf16_t* q, const uint4* pk,
                            const float* lse_swa, int32_t* indices, bf16_t* scores, float* lse_total,
                            float* sel_logits, int L, int N, int h_kv, int G, int topk, int block_size,
                            int window_size, int causal, int q_offset, float sm_scale, int t_base, int t_end) {
#define TG_CALL(NB_, EX_)                                                                              \
  hipLaunchKernelGGL((topk_fwd_group_kernel<GMAX, KS, NB_, EX_>), grid, dim3(64 * TG_WAVES), 0, st, q, pk, lse_swa, \
                     indices, scores, lse_total, sel_logits, L, N, h_kv, G, topk, block_size, window_size, \
                     causal, q_offset, sm_scale, t_base, t_end)
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
// chunks they can see (8, 16, 24 or 32 blocks of 16) into one launch each.
int hils_topk_group_launch(const void* q, const void* lmk_packed, const float* lse_swa, int32_t* indices,
                           void* scores, float* lse_total, float* sel_logits, int B, int L, int N, int h_kv,
                           int G, int D, int topk, int block_size, int window_size, int causal, int q_offset,
                           float sm_scale, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  const int GM = (G == 1) ? 1 : 4;
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
    dim3 grid((t_hi - t + NQ * TG_WAVES - 1) / (NQ * TG_WAVES), h_kv, B);
#define TG_RANGE(G_, KS_)                                                                             \
  tg_launch_range<G_, KS_>(NB, exp, grid, st, (const bf16_t*)q, (const uint4*)lmk_packed, lse_swa, indices, \
                           (bf16_t*)scores, lse_total, sel_logits, L, N, h_kv, G, topk, block_size,   \
                           window_size, causal, q_offset, sm_scale, t, t_hi)
    if (GM == 1) { if (D == 64) TG_RANGE(1, 2); else TG_RANGE(1, 4); }
    else { if (D == 64) TG_RANGE(4, 2); else TG_RANGE(4, 4); }
#undef TG_RANGE
    t = t_hi;
  }
  return HILS_OK;
}
