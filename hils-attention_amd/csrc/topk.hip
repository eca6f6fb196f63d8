// Query -> chunk-key scoring with per-(query, KV head) top-k selection.
//
// One workgroup (4 wavefronts) owns 16 consecutive queries of one (batch, KV head).
// The logits of a 16-query x 16-chunk tile come from one chain of 16x16x32 bf16 MFMAs
// per query head g (A = the 16 query rows of head g, B = 16 chunk keys).  Two passes
// over the visible chunks: pass 1 keeps an online log-sum-exp per (query, g); pass 2
// recomputes the logits, forms max_g(logit - lse_total), parks the pooled scores of a
// segment of chunks in LDS and lets one wavefront per query pick the top-k with a
// bitwise threshold search on order-preserving integer keys.  Ties: lower index wins.
#include <type_traits>
#include "decode_rows.h"
#include "decode_rows_body.h"
#include "../../include/hils_amd.h"

#define TOPK_THREADS 256
#define TOPK_QT 16        // queries per workgroup
#define TOPK_NSEG 512     // chunks per selection segment
#define TOPK_SLOTS (TOPK_NSEG / 64)
#define TOPK_MAXK 64

__device__ __forceinline__ float logaddexp_f(float a, float b) {
  if (a == HILS_NEG_INF) return b;
  if (b == HILS_NEG_INF) return a;
  const float m = fmaxf(a, b), n = fminf(a, b);
  return m + log1pf(expf(n - m));
}

// order-preserving key: larger float <-> larger key; 0 = "not a candidate"
__device__ __forceinline__ uint32_t score_key(float f) {
  if (!(f > HILS_NEG_INF)) return 0u;  // -inf and NaN
  f = f + 0.0f;                        // -0 -> +0
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_score(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// K-th largest of one value per lane by a bitwise threshold search.  Every non-zero x lies in
// [lo, hi] and at least K lanes hold a non-zero x; the leading bits lo and hi share are
// skipped.  Counting is one ballot + scalar popcount per bit.  Returns T with
// count(x >= T) >= K and count(x > T) < K (T need not be one of the values when exactly K
// values are >= T).
__device__ __forceinline__ uint32_t lane_kth_largest(uint32_t x, uint32_t lo, uint32_t hi, int K) {
  const uint32_t diff = lo ^ hi;
  if (diff == 0u) return lo;
  const int top = 31 - __clz((int)diff);
  uint32_t T = (top == 31) ? 0u : (lo & ~((2u << top) - 1u));
  // two bits per step: the three counts are independent, so one step costs about one count's latency
  int bit = top;
  for (; bit >= 1; bit -= 2) {
    const uint32_t c2 = T | (2u << (bit - 1)), c1 = T | (1u << (bit - 1)), c3 = c2 | c1;
    const int n3 = __popcll(__ballot(x >= c3)), n2 = __popcll(__ballot(x >= c2)),
              n1 = __popcll(__ballot(x >= c1));
    int cnt = 0;
    if (n3 >= K) { T = c3; cnt = n3; }
    else if (n2 >= K) { T = c2; cnt = n2; }
    else if (n1 >= K) { T = c1; cnt = n1; }
    if (cnt == K) return T;
  }
  if (bit == 0) {
    const uint32_t c = T | 1u;
    if (__popcll(__ballot(x >= c)) >= K) T = c;
  }
  return T;
}

// One wavefront selects the top-K of (previous candidates) U (segment scores).
// cand_* hold the previous winners in ascending index order (ncand of them, all with
// an index below seg_base); seg holds ns pooled scores of chunks seg_base..seg_base+ns-1.
// With KEYS the segment already holds order-preserving keys instead of floats.
// With seg_idx the chunk index of seg[i] is seg_idx[i] (ascending in i) instead of seg_base + i.
// The winners are written back to cand_* in ascending index order; returns the count.
//
// Fast path: the K-th largest of the 64 per-lane maxima is a lower bound of the K-th largest
// key with at least K keys above it; the keys that reach it (about 1.3 K for K = 32 of 512)
// are compacted to one per lane through a 64-entry scratch (scr_*, by default cand_*, which
// must then hold 64 entries) and the exact threshold is searched on those with ballots.
// If more than 64 keys reach the bound, the K-th largest key is found bit by bit over all
// slots (per-lane tallies plus one DPP reduction per bit).
template <bool KEYS = false, int SLOTS = TOPK_SLOTS>
__device__ __forceinline__ int wave_select(const float* seg, int ns, int seg_base, float* cand_s,
                                           int* cand_i, int ncand, int K, const int* seg_idx = nullptr,
                                           float* scr_s = nullptr, int* scr_i = nullptr) {
  const int lane = threadIdx.x & 63;
  if (!scr_s) { scr_s = cand_s; scr_i = cand_i; }
  uint32_t key[SLOTS + 1];
  int cidx = -1;
  key[0] = 0u;
  if (lane < ncand) {
    key[0] = score_key(cand_s[lane]);
    cidx = cand_i[lane];
  }
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) {
    const int i = s * 64 + lane;
    key[s + 1] = (i < ns) ? (KEYS ? ((const uint32_t*)seg)[i] : score_key(seg[i])) : 0u;
  }
  const int nslot = (ns + 63) / 64 + 1;
  auto index_of = [&](int s) -> int {
    return (s == 0) ? cidx : (seg_idx ? seg_idx[(s - 1) * 64 + lane] : seg_base + (s - 1) * 64 + lane);
  };
  const unsigned long long lt = (1ull << lane) - 1ull;
  uint32_t lm = 0u;  // largest key of this lane
#pragma unroll
  for (int s = 0; s <= SLOTS; ++s) lm = key[s] > lm ? key[s] : lm;
  const bool many = __popcll(__ballot(lm != 0u)) >= K;  // at least K lanes hold a valid key
  uint32_t thr = 1u, hi = 0u;  // every valid key is >= 1
  if (many) {
    hi = wave_max_u(lm);
    const uint32_t lo = ~wave_max_u(lm ? ~lm : 0u);  // smallest non-zero lane maximum
    thr = lane_kth_largest(lm, lo, hi, K);
  }
  // compact the keys >= thr, in index order, to one per lane
  uint32_t* cs_u = (uint32_t*)scr_s;
  int pos = 0;
#pragma unroll
  for (int s = 0; s <= SLOTS; ++s) {
    if (s < nslot) {
      const bool pred = key[s] >= thr;
      const unsigned long long m = __ballot(pred);
      if (pred) {
        const int o = pos + __popcll(m & lt);
        if (o < 64) {
          cs_u[o] = key[s];
          scr_i[o] = index_of(s);
        }
      }
      pos += __popcll(m);
    }
  }
  if (pos <= 64) {
    __builtin_amdgcn_wave_barrier();
    uint32_t ck = 0u;
    int ci = -1;
    if (lane < pos) {
      ck = cs_u[lane];
      ci = scr_i[lane];
    }
    bool sel = lane < pos;  // pos <= K: every valid key wins
    if (pos > K) {
      if (!many) hi = wave_max_u(ck);
      const uint32_t T = lane_kth_largest(ck, thr, hi, K);
      const int need = K - __popcll(__ballot(ck > T));  // ties with the threshold to take, lowest index first
      const unsigned long long eq = __ballot(ck == T);
      sel = (ck > T) || (ck == T && __popcll(eq & lt) < need);
    }
    const unsigned long long sm = __ballot(sel);
    __builtin_amdgcn_wave_barrier();
    if (sel) {
      const int o = __popcll(sm & lt);
      cand_s[o] = key_score(ck);
      cand_i[o] = ci;
    }
    return __popcll(sm);
  }
  // general search over all slots (more than 64 > K keys reach the bound); the bits all
  // valid keys share are skipped
  uint32_t T;
  {
    uint32_t ka = 0xffffffffu, ko = 0u;
#pragma unroll
    for (int s = 0; s <= SLOTS; ++s)
      if (key[s] != 0u) { ka &= key[s]; ko |= key[s]; }
    ka = wave_and_u(ka);
    ko = wave_or_u(ko);
    const uint32_t diff = ka ^ ko;  // bits in which the valid keys differ
    T = ka;
    if (diff != 0u) {
      const int top = 31 - __clz((int)diff);
      T = (top == 31) ? 0u : (ka & ~((2u << top) - 1u));  // the shared leading bits
      for (int bit = top; bit >= 0; --bit) {
        const uint32_t c = T | (1u << bit);
        int cl = 0;  // keys of unused slots are 0 and never count
#pragma unroll
        for (int s = 0; s <= SLOTS; ++s) cl += (key[s] >= c) ? 1 : 0;
        const int cnt = wave_sum_i(cl);
        if (cnt >= K) {
          T = c;
          if (cnt == K) break;
        }
      }
    }
  }
  int gl = 0;
#pragma unroll
  for (int s = 0; s <= SLOTS; ++s) gl += (key[s] > T) ? 1 : 0;
  const int gt = wave_sum_i(gl);
  int need = K - gt;  // ties with the threshold still to take, lowest index first
  pos = 0;
#pragma unroll
  for (int s = 0; s <= SLOTS; ++s) {
    if (s < nslot) {
      const unsigned long long eq = __ballot(key[s] == T && key[s] != 0u);
      const bool take_eq = (key[s] == T && key[s] != 0u) && (__popcll(eq & lt) < need);
      const bool sel = (key[s] > T) || take_eq;
      const unsigned long long sm = __ballot(sel);
      if (sel) {
        const int o = pos + __popcll(sm & lt);
        cand_s[o] = key_score(key[s]);
        cand_i[o] = index_of(s);
      }
      pos += __popcll(sm);
      const int took = __popcll(eq);
      need -= took < need ? took : need;
    }
  }
  return pos;
}

template <int GMAX, int KS>
__global__ void __launch_bounds__(TOPK_THREADS)
topk_fwd_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ lmks,
                const float* __restrict__ lse_swa, const float* __restrict__ bias,
                const float* __restrict__ gumbel, const int32_t* __restrict__ drop_mask,
                int32_t* __restrict__ indices, bf16_t* __restrict__ scores,
                float* __restrict__ lse_total_out, float* __restrict__ sel_logits_out,
                int L, int N, int h_kv, int G, int topk, int block_size, int window_size,
                int causal, int q_offset, int per_qhead, float sm_scale) {
  constexpr int D = KS * 32;
  __shared__ float pooled[TOPK_QT][TOPK_NSEG];
  __shared__ float cand_s[TOPK_QT][TOPK_MAXK];
  __shared__ int cand_i[TOPK_QT][TOPK_MAXK];
  __shared__ float part_m[4][GMAX][TOPK_QT];
  __shared__ float part_l[4][GMAX][TOPK_QT];
  __shared__ float lse_tot[GMAX][TOPK_QT];
  __shared__ int ncand_s[TOPK_QT];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int t0 = blockIdx.x * TOPK_QT;
  const int hk = blockIdx.y;
  const long b = blockIdx.z;
  const int lmk_h = per_qhead ? h_kv * G : h_kv;

  // visible-chunk limit of the 4 queries this lane's accumulator rows belong to
  int lim[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tq = t0 + grp * 4 + i;
    int lm = causal ? visible_limit(tq + q_offset, window_size, block_size) : N;
    lm = lm < 0 ? 0 : (lm > N ? N : lm);
    lim[i] = (tq < L) ? lm : 0;
  }
  int tile_lim;
  {
    const int tl = (t0 + TOPK_QT - 1 < L) ? t0 + TOPK_QT - 1 : L - 1;
    int lm = causal ? visible_limit(tl + q_offset, window_size, block_size) : N;
    tile_lim = lm < 0 ? 0 : (lm > N ? N : lm);
  }
  const int nblk = (tile_lim + 15) / 16;

  // A operands: row (lane & 15) = query t0 + row of head g, 8 consecutive d per k-step
  bf16x8_t afrag[GMAX][KS];
  {
    const int tq = t0 + col;
#pragma unroll
    for (int g = 0; g < GMAX; ++g)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (g < G && tq < L)
          v = *(const uint4*)(q + (((b * L + tq) * h_kv + hk) * (long)G + g) * D + ks * 32 + grp * 8);
        afrag[g][ks] = *(bf16x8_t*)&v;
      }
  }

  // ---------------- pass 1: online log-sum-exp per (query, g) ----------------
  float rm[GMAX][4], rl[GMAX][4];
#pragma unroll
  for (int g = 0; g < GMAX; ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i) { rm[g][i] = HILS_NEG_INF; rl[g][i] = 0.f; }

  for (int blk = wave; blk < nblk; blk += 4) {
    const int c = blk * 16 + col;
    const bool cvalid = c < N;
    bf16x8_t bfrag[KS];
    if (!per_qhead) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (cvalid) v = *(const uint4*)(lmks + ((b * N + c) * (long)lmk_h + hk) * D + ks * 32 + grp * 8);
        bfrag[ks] = *(bf16x8_t*)&v;
      }
    }
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
      if (g < G) {
        if (per_qhead) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (cvalid)
              v = *(const uint4*)(lmks + ((b * N + c) * (long)lmk_h + hk * G + g) * D + ks * 32 + grp * 8);
            bfrag[ks] = *(bf16x8_t*)&v;
          }
        }
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag[g][ks], bfrag[ks], acc, 0, 0, 0);
        float add = 0.f;
        if (cvalid) {
          if (bias) add = bias[((b * N + c) * (long)h_kv + hk) * G + g];
        }
        const float gum = (cvalid && gumbel) ? gumbel[(long)(hk * G + g) * N + c] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float x = __fmul_rn(acc[i], sm_scale);
          if (bias) x = __fadd_rn(x, add);
          if (gumbel) x = __fadd_rn(x, gum);
          if (!(cvalid && c < lim[i])) x = HILS_NEG_INF;
          const float mn = fmaxf(rm[g][i], x);
          if (mn > HILS_NEG_INF) {
            rl[g][i] = rl[g][i] * __expf(rm[g][i] - mn) + __expf(x - mn);
            rm[g][i] = mn;
          }
        }
      }
    }
  }
  // combine over the 16 columns of a lane group, then over the 4 wavefronts
#pragma unroll
  for (int g = 0; g < GMAX; ++g) {
    if (g < G) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float m = rm[g][i], l = rl[g][i];
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) {
          const float m2 = __shfl_xor(m, o, 64), l2 = __shfl_xor(l, o, 64);
          const float mn = fmaxf(m, m2);
          if (mn > HILS_NEG_INF) {
            l = l * __expf(m - mn) + l2 * __expf(m2 - mn);
            m = mn;
          }
        }
        if (col == 0) {
          part_m[wave][g][grp * 4 + i] = m;
          part_l[wave][g][grp * 4 + i] = l;
        }
      }
    }
  }
  __syncthreads();
  for (int p = tid; p < G * TOPK_QT; p += TOPK_THREADS) {
    const int g = p / TOPK_QT, qi = p - g * TOPK_QT;
    float m = HILS_NEG_INF, l = 0.f;
    for (int w = 0; w < 4; ++w) {
      const float m2 = part_m[w][g][qi], l2 = part_l[w][g][qi];
      const float mn = fmaxf(m, m2);
      if (mn > HILS_NEG_INF) {
        l = l * __expf(m - mn) + l2 * __expf(m2 - mn);
        m = mn;
      }
    }
    const float lse_hils = (l > 0.f) ? m + logf(l) : HILS_NEG_INF;
    const int tq = t0 + qi;
    float tot = HILS_NEG_INF;
    if (tq < L) {
      const long o = ((b * L + tq) * (long)h_kv + hk) * G + g;
      tot = logaddexp_f(lse_swa[o], lse_hils);
      if (lse_total_out) lse_total_out[o] = tot;
    }
    lse_tot[g][qi] = tot;
  }
  if (tid < TOPK_QT) ncand_s[tid] = 0;
  __syncthreads();

  // ---------------- pass 2: pooled scores per segment + selection ----------------
  float lt_reg[GMAX][4];
#pragma unroll
  for (int g = 0; g < GMAX; ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i) lt_reg[g][i] = (g < G) ? lse_tot[g][grp * 4 + i] : 0.f;

  const int nseg = (nblk * 16 + TOPK_NSEG - 1) / TOPK_NSEG;
  for (int seg = 0; seg < nseg; ++seg) {
    const int seg_base = seg * TOPK_NSEG;
    const int blk_end = ((seg + 1) * (TOPK_NSEG / 16) < nblk) ? (seg + 1) * (TOPK_NSEG / 16) : nblk;
    for (int blk = seg * (TOPK_NSEG / 16) + wave; blk < blk_end; blk += 4) {
      const int c = blk * 16 + col;
      const bool cvalid = c < N;
      bf16x8_t bfrag[KS];
      if (!per_qhead) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          uint4 v = make_uint4(0, 0, 0, 0);
          if (cvalid) v = *(const uint4*)(lmks + ((b * N + c) * (long)lmk_h + hk) * D + ks * 32 + grp * 8);
          bfrag[ks] = *(bf16x8_t*)&v;
        }
      }
      float best[4] = {HILS_NEG_INF, HILS_NEG_INF, HILS_NEG_INF, HILS_NEG_INF};
#pragma unroll
      for (int g = 0; g < GMAX; ++g) {
        if (g < G) {
          if (per_qhead) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
              uint4 v = make_uint4(0, 0, 0, 0);
              if (cvalid)
                v = *(const uint4*)(lmks + ((b * N + c) * (long)lmk_h + hk * G + g) * D + ks * 32 + grp * 8);
              bfrag[ks] = *(bf16x8_t*)&v;
            }
          }
          f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag[g][ks], bfrag[ks], acc, 0, 0, 0);
          float add = 0.f;
          if (cvalid && bias) add = bias[((b * N + c) * (long)h_kv + hk) * G + g];
          const float gum = (cvalid && gumbel) ? gumbel[(long)(hk * G + g) * N + c] : 0.f;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float x = __fmul_rn(acc[i], sm_scale);
            if (bias) x = __fadd_rn(x, add);
            if (gumbel) x = __fadd_rn(x, gum);
            const bool vis = cvalid && c < lim[i];
            if (!vis) x = HILS_NEG_INF;
            if (sel_logits_out && cvalid) {
              const int tq = t0 + grp * 4 + i;
              if (tq < L)
                sel_logits_out[(((b * L + tq) * (long)h_kv + hk) * G + g) * N + c] = x;
            }
            const float nrm = (x == HILS_NEG_INF) ? HILS_NEG_INF : __fsub_rn(x, lt_reg[g][i]);
            best[i] = fmaxf(best[i], nrm);  // fmaxf ignores a NaN operand
          }
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float s = best[i];
        if (drop_mask && s > HILS_NEG_INF) {
          const int tq = t0 + grp * 4 + i;
          if (tq < L && cvalid && drop_mask[(b * L + tq) * (long)N + c] != 0) s = HILS_NEG_INF;
        }
        pooled[grp * 4 + i][c - seg_base] = s;
      }
    }
    __syncthreads();
    const int ns = blk_end * 16 - seg_base;
    for (int qi = wave; qi < TOPK_QT; qi += 4) {
      if (t0 + qi < L) {
        const int nc = wave_select(pooled[qi], ns, seg_base, cand_s[qi], cand_i[qi], ncand_s[qi], topk);
        if (lane == 0) ncand_s[qi] = nc;
      }
    }
    __syncthreads();
  }

  // ---------------- epilogue: indices and raw scaled scores ----------------
  for (int qi = wave; qi < TOPK_QT; qi += 4) {
    const int tq = t0 + qi;
    if (tq >= L) continue;
    const int nc = ncand_s[qi];
    int32_t* irow = indices + ((b * L + tq) * (long)h_kv + hk) * topk;
    for (int k = lane; k < topk; k += 64) irow[k] = (k < nc) ? cand_i[qi][k] : -1;
    // raw scaled scores at the selected chunks: one MFMA chain per 16 slots with the
    // selected chunk keys as rows and the G query heads as columns
    bf16x8_t bq[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (col < G) v = *(const uint4*)(q + (((b * L + tq) * h_kv + hk) * (long)G + col) * D + ks * 32 + grp * 8);
      bq[ks] = *(bf16x8_t*)&v;
    }
    const int ntile = (topk + 15) / 16;
    const int g_loops = per_qhead ? G : 1;
    const long srow = ((b * L + tq) * (long)h_kv + hk) * G;
    for (int gq = 0; gq < g_loops; ++gq) {
      for (int tile = 0; tile < ntile; ++tile) {
        const int slot_r = tile * 16 + col;
        const int c = (slot_r < nc) ? cand_i[qi][slot_r] : -1;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          uint4 v = make_uint4(0, 0, 0, 0);
          if (c >= 0)
            v = *(const uint4*)(lmks + ((b * N + c) * (long)lmk_h + (per_qhead ? hk * G + gq : hk)) * D + ks * 32 + grp * 8);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(bf16x8_t*)&v, bq[ks], acc, 0, 0, 0);
        }
        const bool mine = per_qhead ? (col == gq) : (col < G);
        if (mine) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int slot = tile * 16 + grp * 4 + i;
            if (slot < topk)
              scores[(srow + col) * topk + slot] = f2bf(slot < nc ? __fmul_rn(acc[i], sm_scale) : HILS_NEG_INF);
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Row-packed variant for G <= 4 with one chunk key per KV head: the 16 rows of an MFMA
// tile are (16/GMAX queries) x (GMAX query heads), so the max over the heads of a query is
// a max over accumulator registers of one lane, and a wavefront needs nobody else: one
// wavefront per workgroup owns 8 consecutive queries of a (batch, KV head), keeps their
// query rows in registers as A operands and streams the chunk keys as B operands.
// Pass 1 accumulates sum exp2(y - ref) per lane against a reference that is only moved when
// a logit exceeds it by 2^40 (one exp2 per logit); pass 2 recomputes the logits, writes the
// pooled scores of a segment of chunks to LDS and selects per query.
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_max(float x) {
  const int v = __builtin_amdgcn_update_dpp(__float_as_int(x), __float_as_int(x), CTRL, 0xF, 0xF, false);
  return fmaxf(x, __int_as_float(v));
}
__device__ __forceinline__ float row_max16(float x) {
  x = dpp_max<0xB1>(x);
  x = dpp_max<0x4E>(x);
  x = dpp_max<0x141>(x);
  x = dpp_max<0x140>(x);
  return x;
}

// Chunk keys of a (batch, KV head) in the register order of the MFMA B operand: block of 16
// chunks x k-step x lane (chunk = lane & 15, 8 features from 8 * (lane >> 4)) x 8 bf16, so that a
// wavefront's operand load is one contiguous 1 KiB burst (from the token-major tensor the 16
// chunk rows of a block lie 2*h_kv*D bytes apart and every lane touches its own 64-byte segment).
// Chunks past N are zero.  One thread per 16-byte piece.
__global__ void __launch_bounds__(256)
topk_pack_lmk_kernel(const bf16_t* __restrict__ lmks, uint4* __restrict__ packed, int N, int h_kv,
                     int D, int nblk16, long total) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int KS = D / 32;
  const int lane = (int)(i & 63);
  long r = i >> 6;
  const int ks = (int)(r % KS);
  r /= KS;
  const int blk = (int)(r % nblk16);
  r /= nblk16;
  const int hk = (int)(r % h_kv);
  const long b = r / h_kv;
  const int c = blk * 16 + (lane & 15);
  uint4 v = make_uint4(0, 0, 0, 0);
  if (c < N) v = *(const uint4*)(lmks + ((b * N + c) * (long)h_kv + hk) * D + ks * 32 + (lane >> 4) * 8);
  packed[i] = v;
}

// (the variants with a bias / noise / drop mask / export hold a block's bias beside its keys: three
// wavefronts per SIMD instead of four, which their LDS allows anyway, rather than 100 bytes of scratch)
// The additive bias (B, N, heads) fp32 head-major in blocks of 16 chunks, (B, heads, nblk16, 16), zero
// past N: the 16 lanes of a chunk block then read one head's bias as 64 contiguous bytes (from the
// caller's tensor every lane touches a cache line of its own, once per head).  One thread per element.
__global__ void __launch_bounds__(256)
topk_pack_bias_kernel(const float* __restrict__ bias, float* __restrict__ packed, int N, int heads, int nblk16,
                      long total) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int col = (int)(i & 15);
  long r = i >> 4;
  const int blk = (int)(r % nblk16);
  r /= nblk16;
  const int h = (int)(r % heads);
  const long b = r / heads;
  const int c = blk * 16 + col;
  packed[i] = c < N ? bias[(b * N + c) * (long)heads + h] : 0.f;
}

template <int GMAX, int KS, bool PLAIN, bool PACKED, bool PERQ = false, bool BIASONLY = false>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(PLAIN ? 4 : 3, 4)))
topk_fwd_rows_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ lmks,
                     const float* __restrict__ lse_swa, const float* __restrict__ bias,
                     const float* __restrict__ gumbel, const int32_t* __restrict__ drop_mask,
                     int32_t* __restrict__ indices, bf16_t* __restrict__ scores,
                     float* __restrict__ lse_total_out, float* __restrict__ sel_logits_out,
                     int L, int N, int h_kv, int G, int topk, int block_size, int window_size,
                     int causal, int q_offset, float sm_scale, int segw, int pool_floats,
                     const uint4* __restrict__ lmk_packed, const float* __restrict__ bias_packed,
                     int lmk_group_heads) {
  // lmk_group_heads (PERQ only): chunk-key heads per KV head, G (a key per query head) or 1 (shared keys
  // walked head by head all the same: how more than four query heads per KV head run here)
  // bias_packed: the bias in topk_pack_bias_kernel's order (or null: read from bias)
  // PLAIN: no bias, Gumbel noise, drop mask or logit export (the inference path)
  // PACKED: the chunk keys of the two passes come from lmk_packed (topk_pack_lmk_kernel's order)
  // BIASONLY (not PLAIN, bias_packed given): a bias and nothing else (the layer's prior bias at inference).
  // The general variant tests its optional inputs per element, and behind every such branch the compiler
  // waits for all loads in flight, the next block's keys included; this one has no branch in its loops.
  static_assert(!BIASONLY || (!PLAIN && PACKED), "the bias-only variant reads the packed bias");
  // PERQ: one chunk key per QUERY head, lmks (B,N,h_kv*G,D) and lmk_packed with h_kv*G heads.  The tile
  // rows are then 16 queries of one head (GMAX = 1) and the wavefront walks the G heads of its KV head
  // one after the other, in both passes: a head's log-sum-exp waits in LDS, and the pooled score of a
  // (query, chunk) is the running maximum over the heads of what the same lane wrote there before.
  static_assert(!PERQ || (GMAX == 1 && PACKED), "a key per query head: 16 queries of one head per tile, packed keys");
  constexpr int D = KS * 32;
  constexpr int QPT = 16 / GMAX;            // queries per 16-row tile
  constexpr int NT = (GMAX == 4) ? 2 : 1;   // tiles per wavefront
  constexpr int NQ = NT * QPT;              // queries per wavefront (8)
  constexpr int GPL = 4 / GMAX;             // queries per lane and tile
  extern __shared__ float tr_smem[];
  const int stride = segw + 16;             // row stride: lane groups on disjoint banks
  float* pooled = tr_smem;                  // NQ x stride (pool_floats >= that, and >= the score staging)
  float* scr_s = pooled + pool_floats;      // 64-entry compaction scratch of the selection
  int* scr_i = (int*)(scr_s + 64);
  float* car_s = (float*)(scr_i + 64);      // NQ x topk winners carried across segments
  int* car_i = (int*)(car_s + NQ * topk);
  float* lt_s = (float*)(car_i + NQ * topk);  // PERQ: lse_total, [head][query]
  const int LPG = PERQ ? lmk_group_heads : 1;
  const int h_lmk = h_kv * LPG;               // heads of the chunk-key tensor
  const int GH = PERQ ? G : 1;                // heads the wavefront walks
  int cur_gh = 0;                             // ... and the one it is at

  const int lane = threadIdx.x, col = lane & 15, j = lane >> 4;
  const int t0 = blockIdx.x * NQ;
  const int hk = blockIdx.y;
  const long b = blockIdx.z;

  auto limit_of = [&](int tq) -> int {
    int lm = causal ? visible_limit(tq + q_offset, window_size, block_size) : N;
    return lm < 0 ? 0 : (lm > N ? N : lm);
  };
  // accumulator row 4j+i of tile nt <-> (query t0 + nt*QPT + (4j+i)/GMAX, head (4j+i)%GMAX)
  int lim[NT][4];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 4 * j + i;
      const int tq = t0 + nt * QPT + r / GMAX;
      lim[nt][i] = (tq < L && (PERQ || (r % GMAX) < G)) ? limit_of(tq) : 0;
    }
  const int t_last = (t0 + NQ - 1 < L) ? t0 + NQ - 1 : L - 1;
  const int nblk = (limit_of(t_last) + 15) / 16;
  // blocks below nfull are visible to every row: no masking there
  const int nfull = ((PERQ || G == GMAX) && t0 + NQ <= L) ? limit_of(t0) / 16 : 0;

  bf16x8_t afrag[NT][KS];
  auto load_a = [&](int gh) {  // the query rows as A operands (PERQ: of head gh)
    const int r = lane & 15;
    const int g = PERQ ? gh : r % GMAX;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int tq = t0 + nt * QPT + r / GMAX;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bool ok = tq < L && g < G;
        uint4 v = *(const uint4*)(q + (((b * L + (ok ? tq : t0)) * h_kv + hk) * (long)G + (ok ? g : 0)) * D + ks * 32 + j * 8);
        if (!ok) v = make_uint4(0, 0, 0, 0);
        afrag[nt][ks] = *(bf16x8_t*)&v;
      }
    }
  };
  load_a(0);
  // chunk keys as B operands; rows beyond N are read from row N-1 and masked by the caller
  const long bstride = (long)h_lmk * D;  // elements between consecutive chunk keys
  const bf16_t* bbase;
  const uint4* pbase;
  const char* ubase;  // blocks that lie wholly inside [0, N): uniform block address + a 32-bit lane offset
  auto set_head = [&](int gh) {  // the key head the loads below read (PERQ: head gh of the KV head's group)
    const int hl = hk * LPG + (LPG > 1 ? gh : 0);
    cur_gh = gh;
    bbase = lmks + (b * N * (long)h_lmk + hl) * D + j * 8;
    pbase = PACKED ? lmk_packed + ((b * h_lmk + hl) * (long)((N + 15) / 16) * KS) * 64 + lane : nullptr;
    ubase = (const char*)lmks + ((b * N * (long)h_lmk + hl) * D) * 2;
  };
  set_head(0);
  auto load_b = [&](int blk, uint4* dst) {
    if (PACKED) {
      const int bc = blk < (N + 15) / 16 ? blk : (N + 15) / 16 - 1;  // a prefetch may run past the end
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) dst[ks] = pbase[((long)bc * KS + ks) * 64];
      return;
    }
    int c = blk * 16 + col;
    c = c < N ? c : N - 1;
    const bf16_t* p = bbase + c * bstride;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) dst[ks] = *(const uint4*)(p + ks * 32);
  };
  auto scores_of = [&](const uint4* bb, f32x4_t* acc) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      acc[nt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag[nt][ks], *(const bf16x8_t*)&bb[ks], acc[nt], 0, 0, 0);
    }
  };
  // the additive bias of a block's chunk column for this lane's heads (accumulator row 4j+i is head
  // (4j+i) % GMAX): loaded together with the block's keys, unconditionally from a clamped address, so
  // that the loads of a block are all in flight at once (a load behind a branch is waited for inside
  // it, one memory latency per element)
  struct BiasRow { float v[GMAX]; };
  const bool bias_vec4 = !PLAIN && bias && G == 4 && (((size_t)bias) & 15) == 0;
  auto load_bias = [&](int blk, BiasRow& dst) {
    if (PLAIN || (!BIASONLY && !bias)) return;
    if (BIASONLY || bias_packed) {
      const int nb16 = (N + 15) / 16;
      const float* p = bias_packed + ((b * h_kv + hk) * (long)G * nb16 + (blk < nb16 ? blk : nb16 - 1)) * 16 + col;
      if (PERQ) {
        dst.v[0] = p[(long)cur_gh * nb16 * 16];
        return;
      }
#pragma unroll
      for (int g = 0; g < GMAX; ++g) dst.v[g] = p[(long)(g < G ? g : 0) * nb16 * 16];
      return;
    }
    int c = blk * 16 + col;
    c = c < N ? c : N - 1;
    const float* p = bias + ((b * N + c) * (long)h_kv + hk) * G;
    if (PERQ) {
      dst.v[0] = p[cur_gh];
      return;
    }
    if (GMAX == 4 && bias_vec4) {  // four heads, 16-byte aligned rows: one load
      const float4 t = *(const float4*)p;
      dst.v[0] = t.x; dst.v[1 % GMAX] = t.y; dst.v[2 % GMAX] = t.z; dst.v[3 % GMAX] = t.w;
      return;
    }
#pragma unroll
    for (int g = 0; g < GMAX; ++g) dst.v[g] = p[g < G ? g : 0];
  };
  // exact fp32 logit of accumulator element i of chunk c (before masking)
  auto logit = [&](float acc, int c, int i, const BiasRow& bz) -> float {
    float x = __fmul_rn(acc, sm_scale);
    if (!PLAIN) {
      const int g = PERQ ? cur_gh : (4 * j + i) % GMAX;
      if (BIASONLY) {
        // (chunks past N and heads past G get a finite value added and are masked by their limits)
        x = __fadd_rn(x, bz.v[PERQ ? 0 : g]);
      } else if (c < N && g < G) {
        if (bias) x = __fadd_rn(x, bz.v[PERQ ? 0 : g]);
        if (gumbel) x = __fadd_rn(x, gumbel[(long)(hk * G + g) * N + c]);
      }
    }
    return x;
  };
  const uint32_t lane_off = (uint32_t)((col * bstride + j * 8) * 2);
  auto load_b_full = [&](int blk, uint4* dst) {
    if (PACKED) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) dst[ks] = pbase[((long)blk * KS + ks) * 64];
      return;
    }
    const char* p = ubase + (long)blk * (32 * bstride);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) dst[ks] = *(const uint4*)(p + lane_off + ks * 64);
  };
  // run body(bb, blk, masked) over blocks [lo, hi): two operand buffers in turn, the next
  // block's keys always in flight (a load past hi re-reads an earlier row and is never used)
  auto for_range = [&](int lo, int hi, auto masked_t, auto& body) {
    constexpr bool MASKED = decltype(masked_t)::value;
    if (lo >= hi) return;
    auto ld = [&](int blk, uint4* dst) {
      if (MASKED) load_b(blk, dst);
      else load_b_full(blk < hi ? blk : hi - 1, dst);
    };
    uint4 b0[KS], b1[KS];
    BiasRow z0, z1;
#pragma unroll
    for (int g = 0; g < GMAX; ++g) z0.v[g] = z1.v[g] = 0.f;
    ld(lo, b0);
    load_bias(lo, z0);
    int blk = lo;
    for (; blk + 1 < hi; blk += 2) {
      ld(blk + 1, b1);
      load_bias(blk + 1, z1);
      body(b0, blk, masked_t, z0);
      ld(blk + 2, b0);
      load_bias(blk + 2, z0);
      body(b1, blk + 1, masked_t, z1);
    }
    if (blk < hi) body(b0, blk, masked_t, z0);
  };
  auto for_blocks = [&](int lo, int hi, auto body) {
    const int mid = nfull < hi ? (nfull > lo ? nfull : lo) : hi;  // masking starts here
    for_range(lo, mid, std::false_type{}, body);
    for_range(mid, hi, std::true_type{}, body);
  };

  // ---------------- pass 1: sum of exp2(y - ref) per lane and row ----------------
  const float c2 = sm_scale * HILS_LOG2E;
  float lse_tot[NT][4];
  for (int gh = 0; gh < GH; ++gh) {
  if (PERQ && gh > 0) {
    set_head(gh);
    load_a(gh);
  }
  float swa[NT][4];  // lse_swa of this lane's rows (-inf for padding rows)
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 4 * j + i;
      const int tq = t0 + nt * QPT + r / GMAX, g = PERQ ? gh : r % GMAX;
      // unconditional loads from a clamped address: all eight are in flight together (a load
      // inside a branch is waited for inside it, one memory latency after the other)
      const bool ok = tq < L && g < G;
      const float x = lse_swa[((b * L + (ok ? tq : t0)) * (long)h_kv + hk) * G + (ok ? g : 0)];
      swa[nt][i] = ok ? x : HILS_NEG_INF;
    }
  float ref[NT][4], l[NT][4];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) { ref[nt][i] = -1e30f; l[nt][i] = 0.f; }
  for_blocks(0, nblk, [&](const uint4* bb, int blk, auto masked_t, const BiasRow& bz) {
    constexpr bool MASKED = decltype(masked_t)::value;
    const int c = blk * 16 + col;
    f32x4_t acc[NT];
    scores_of(bb, acc);
    float y[NT][4], d[NT][4];
    float dmax = HILS_NEG_INF;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // one rounding (acc * c2) whenever nothing is added to the logit, in both variants, so that
        // the export variant and the plain one select from bit-identical lse_total
        float yy = (PLAIN || (!BIASONLY && !bias && !gumbel)) ? acc[nt][i] * c2 : logit(acc[nt][i], c, i, bz) * HILS_LOG2E;
        if (MASKED && !(c < lim[nt][i])) yy = HILS_NEG_INF;
        y[nt][i] = yy;
        d[nt][i] = yy - ref[nt][i];
        dmax = fmaxf(dmax, d[nt][i]);
      }
    if (__any(dmax > 40.f)) {  // move the reference of the rows that outgrew it
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (d[nt][i] > 40.f) {
            l[nt][i] *= __builtin_amdgcn_exp2f(ref[nt][i] - y[nt][i]);
            ref[nt][i] = y[nt][i];
            d[nt][i] = 0.f;
          }
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i) l[nt][i] += __builtin_amdgcn_exp2f(d[nt][i]);
  });
  // combine the 16 lanes (chunk columns) of each row; lse_total per row, in the log2 domain
  // with the hardware exp2/log2 (absolute error ~1e-6, far inside the 1e-4 the LSE needs)
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float M = row_max16(ref[nt][i]);
      const float ls = row_sum<16>(l[nt][i] * __builtin_amdgcn_exp2f(ref[nt][i] - M));
      const float hils2 = (ls > 0.f) ? M + __builtin_amdgcn_logf(ls) : HILS_NEG_INF;
      const float swa2 = swa[nt][i] * HILS_LOG2E;
      const float mx = fmaxf(swa2, hils2), mn = fminf(swa2, hils2);
      float tot2 = mx;
      if (mn > HILS_NEG_INF) tot2 = mx + __builtin_amdgcn_logf(1.f + __builtin_amdgcn_exp2f(mn - mx));
      const float tot = tot2 * HILS_LN2;
      const int r = 4 * j + i;
      const int tq = t0 + nt * QPT + r / GMAX, g = PERQ ? gh : r % GMAX;
      if (lse_total_out && col == 0 && tq < L && g < G)
        lse_total_out[((b * L + tq) * (long)h_kv + hk) * G + g] = tot;
      lse_tot[nt][i] = tot;
      if (PERQ && col == 0) lt_s[gh * NQ + nt * QPT + r] = tot;  // waits for pass 2
    }
  }  // heads
  if (PERQ) __builtin_amdgcn_wave_barrier();

  // ---------------- pass 2: pooled scores per segment + selection ----------------
  int ncand_v = 0;  // lane qi holds the number of winners of query qi so far
  const int bps = segw / 16;
  const int nseg = (nblk + bps - 1) / bps;
  for (int seg = 0; seg < nseg; ++seg) {
    const int seg_base = seg * segw;
    const int blk_end = ((seg + 1) * bps < nblk) ? (seg + 1) * bps : nblk;
    for (int gh = 0; gh < GH; ++gh) {
    if (PERQ) {
      set_head(gh);
      if (GH > 1) load_a(gh);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) lse_tot[nt][i] = lt_s[gh * NQ + nt * QPT + 4 * j + i];
    }
    for_blocks(seg * bps, blk_end, [&](const uint4* bb, int blk, auto masked_t, const BiasRow& bz) {
      constexpr bool MASKED = decltype(masked_t)::value;
      const int c = blk * 16 + col;
      f32x4_t acc[NT];
      scores_of(bb, acc);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        float nrm[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float x = logit(acc[nt][i], c, i, bz);
          if (MASKED && !(c < lim[nt][i])) x = HILS_NEG_INF;
          if (!PLAIN && !BIASONLY) {
            if (sel_logits_out && c < N) {
              const int r = 4 * j + i;
              const int tq = t0 + nt * QPT + r / GMAX, g = PERQ ? gh : r % GMAX;
              if (tq < L && g < G) sel_logits_out[(((b * L + tq) * (long)h_kv + hk) * G + g) * N + c] = x;
            }
          }
          nrm[i] = __fsub_rn(x, lse_tot[nt][i]);
          if (MASKED || !PLAIN) nrm[i] = (x == HILS_NEG_INF) ? HILS_NEG_INF : nrm[i];
        }
#pragma unroll
        for (int u = 0; u < GPL; ++u) {
          float best = nrm[u * GMAX];
#pragma unroll
          for (int e = 1; e < GMAX; ++e) best = fmaxf(best, nrm[u * GMAX + e]);  // fmaxf ignores a NaN operand
          const int ql = nt * QPT + (4 * j) / GMAX + u;
          if (!PLAIN && !BIASONLY) {
            if (drop_mask && best > HILS_NEG_INF && t0 + ql < L && c < N &&
                drop_mask[(b * L + t0 + ql) * (long)N + c] != 0)
              best = HILS_NEG_INF;
          }
          float* pp = &pooled[ql * stride + (c - seg_base)];
          *pp = (PERQ && gh > 0) ? fmaxf(*pp, best) : best;  // (the same lane wrote the heads before)
        }
      }
    });
    }  // heads
    __builtin_amdgcn_wave_barrier();
    const int ns = blk_end * 16 - seg_base;
#pragma unroll 1
    for (int qi = 0; qi < NQ; ++qi) {
      if (t0 + qi < L) {
        const int prev = __builtin_amdgcn_readlane(ncand_v, qi);
        const int nc = wave_select(pooled + qi * stride, ns, seg_base, car_s + qi * topk, car_i + qi * topk,
                                   prev, topk, nullptr, scr_s, scr_i);
        if (lane == qi) ncand_v = nc;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  // ---------------- epilogue: indices and raw scaled scores ----------------
  // Indices: the winners sit in LDS as [query][topk]; 16-byte lane stores when rows allow it.
  if ((topk & 3) == 0) {
    const int per_q = topk / 4;
    for (int e = lane; e < NQ * per_q; e += 64) {
      const int qi = e / per_q, k0 = (e - qi * per_q) * 4;
      const int nc = __shfl(ncand_v, qi, 64);
      int4 v = *(const int4*)(car_i + qi * topk + k0);
      v.x = (k0 + 0 < nc) ? v.x : -1;
      v.y = (k0 + 1 < nc) ? v.y : -1;
      v.z = (k0 + 2 < nc) ? v.z : -1;
      v.w = (k0 + 3 < nc) ? v.w : -1;
      if (t0 + qi < L) *(int4*)(indices + ((b * L + t0 + qi) * (long)h_kv + hk) * topk + k0) = v;
    }
  } else {
    for (int e = lane; e < NQ * topk; e += 64) {
      const int qi = e / topk, k = e - qi * topk;
      const int nc = __shfl(ncand_v, qi, 64);
      if (t0 + qi < L) indices[((b * L + t0 + qi) * (long)h_kv + hk) * topk + k] = (k < nc) ? car_i[e] : -1;
    }
  }
  // Raw scaled scores at the winners: the query rows are still the A operands; the B operand
  // gathers 16 winning chunk keys of one query, and the rows of that query are kept.  Four
  // queries (gathers) are in flight at a time.  The scores are staged in LDS (over the dead
  // pooled rows) as [query][head][slot], the layout of the output, and stored in 16-byte pieces.
  bf16_t* stage = (bf16_t*)pooled;
  const int ntile = (topk + 15) / 16;
  for (int gh = 0; gh < GH; ++gh) {
  if (PERQ) {
    set_head(gh);
    if (GH > 1) load_a(gh);
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
    for (int qq = 0; qq < QPT; qq += 4) {
#pragma unroll 1
      for (int tile = 0; tile < ntile; ++tile) {
        uint4 bg[4][KS];
        int ncs[4];
        const int slot = tile * 16 + col;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int qi = nt * QPT + qq + u;
          ncs[u] = __builtin_amdgcn_readlane(ncand_v, qi);
          const int c = (slot < ncs[u]) ? car_i[qi * topk + slot] : 0;  // chunk 0 stands in; masked below
          const bf16_t* p = bbase + c * bstride;
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) bg[u][ks] = *(const uint4*)(p + ks * 32);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int qi = nt * QPT + qq + u;
          f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag[nt][ks], *(const bf16x8_t*)&bg[u][ks], acc, 0, 0, 0);
          if (slot < topk) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int r = 4 * j + i;
              const int g = PERQ ? gh : r % GMAX;
              if (r / GMAX == qq + u && g < G)
                stage[(qi * G + g) * topk + slot] = f2bf(slot < ncs[u] ? __fmul_rn(acc[i], sm_scale) : HILS_NEG_INF);
            }
          }
        }
      }
    }
  }
  }  // heads
  __builtin_amdgcn_wave_barrier();
  const int row_e = G * topk;  // bf16 elements per query
  if ((row_e & 7) == 0) {
    const int per_q = row_e / 8;
    for (int e = lane; e < NQ * per_q; e += 64) {
      const int qi = e / per_q, part = e - qi * per_q;
      if (t0 + qi < L)
        *(uint4*)(scores + ((b * L + t0 + qi) * (long)h_kv + hk) * row_e + part * 8) =
            *(const uint4*)(stage + qi * row_e + part * 8);
    }
  } else {
    for (int e = lane; e < NQ * row_e; e += 64) {
      const int qi = e / row_e;
      if (t0 + qi < L) scores[((b * L + t0 + qi) * (long)h_kv + hk) * row_e + (e - qi * row_e)] = stage[e];
    }
  }
}

static int topk_rows_segw(int N) {
  const int n16 = (N + 15) / 16 * 16;
  return n16 < 256 ? n16 : 256;
}

template <int GMAX>
static int launch_topk(int D, dim3 grid, hipStream_t st, const bf16_t* q, const bf16_t* lmks,
                       const float* lse_swa, const float* bias, const float* gumbel,
                       const int32_t* drop_mask, int32_t* indices, bf16_t* scores, float* lse_total,
                       float* sel_logits, int L, int N, int h_kv, int G, int topk, int block_size,
                       int window_size, int causal, int q_offset, int per_qhead, float sm_scale) {
#define HILS_TOPK_LAUNCH(KS_)                                                                    \
  hipLaunchKernelGGL((topk_fwd_kernel<GMAX, KS_>), grid, dim3(TOPK_THREADS), 0, st, q, lmks,     \
                     lse_swa, bias, gumbel, drop_mask, indices, scores, lse_total, sel_logits, L, \
                     N, h_kv, G, topk, block_size, window_size, causal, q_offset, per_qhead,     \
                     sm_scale)
  switch (D) {
    case 64: HILS_TOPK_LAUNCH(2); break;
    case 128: HILS_TOPK_LAUNCH(4); break;
    default:
      hils_set_error("hils_topk_fwd: head dim %d not supported (64 or 128)", D);
      return HILS_ERR_ARG;
  }
#undef HILS_TOPK_LAUNCH
  return HILS_OK;
}

// ---------------------------------------------------------------------------
// Split path for few queries (decode, short chunked prefill): the fused kernel above has
// one workgroup per 16 queries, too few to pull the chunk keys at HBM rate.  Here kernel A
// spreads the logits over (256-chunk segment) x (KV head) x (query) workgroups and parks
// the raw scaled logits in a scratch; kernel B, one workgroup per (query, KV head), does
// LSE, pooling and selection from the scratch.
// ---------------------------------------------------------------------------
#define TOPK_A_THREADS 256
#define TOPK_A_CHUNKS 256   // chunk keys per workgroup (64 per wavefront)

// Kernel A: raw scaled logits.  Chunk-key rows are streamed with fully coalesced 16-byte
// lane loads (LR = D/8 lanes per row); q.k uses packed bf16 dot2 and a DPP row reduction.
template <int D, int GMAX>
__global__ void __launch_bounds__(TOPK_A_THREADS)
topk_logits_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ lmks,
                   float* __restrict__ raw, int L, int N, int h_kv, int G, int per_qhead,
                   float sm_scale) {
  constexpr int LR = D / 8, TPI = 64 / LR, NI = 64 / TPI;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int piece = lane % LR, tsub = lane / LR;
  const int hk = blockIdx.y;
  const long bt = blockIdx.z;  // b * L + t
  const long b = bt / L;
  const int lmk_h = per_qhead ? h_kv * G : h_kv;
  const int c0 = blockIdx.x * TOPK_A_CHUNKS + wave * 64;
  if (c0 >= N) return;
  uint4 qp[GMAX];
#pragma unroll
  for (int g = 0; g < GMAX; ++g) {
    qp[g] = make_uint4(0, 0, 0, 0);
    if (g < G) qp[g] = *(const uint4*)(q + ((bt * h_kv + hk) * (long)G + g) * D + piece * 8);
  }
  float* out = raw + (bt * h_kv + hk) * (long)G * N;
  __shared__ float s_out[TOPK_A_THREADS / 64][GMAX][64];  // logits of this wavefront's 64 chunks
  if (!per_qhead) {
    uint4 kr[NI];
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int c = c0 + it * TPI + tsub;
      kr[it] = make_uint4(0, 0, 0, 0);
      if (c < N) kr[it] = *(const uint4*)(lmks + ((b * N + c) * (long)lmk_h + hk) * D + piece * 8);
    }
#pragma unroll
    for (int it = 0; it < NI; ++it) {
#pragma unroll
      for (int g = 0; g < GMAX; ++g)
        if (g < G) {
          const float s = row_sum<LR>(dot8_bf16(qp[g], kr[it], 0.f));
          if (piece == 0) s_out[wave][g][it * TPI + tsub] = __fmul_rn(s, sm_scale);
        }
    }
  } else {
#pragma unroll
    for (int g = 0; g < GMAX; ++g)
      if (g < G) {
        uint4 kr[NI];
#pragma unroll
        for (int it = 0; it < NI; ++it) {
          const int c = c0 + it * TPI + tsub;
          kr[it] = make_uint4(0, 0, 0, 0);
          if (c < N) kr[it] = *(const uint4*)(lmks + ((b * N + c) * (long)lmk_h + hk * G + g) * D + piece * 8);
        }
#pragma unroll
        for (int it = 0; it < NI; ++it) {
          const float s = row_sum<LR>(dot8_bf16(qp[g], kr[it], 0.f));
          if (piece == 0) s_out[wave][g][it * TPI + tsub] = __fmul_rn(s, sm_scale);
        }
      }
  }
  // wavefront-private LDS slice: written and read by the same wavefront, in program order
  if (c0 + lane < N)
    for (int g = 0; g < G; ++g) out[(long)g * N + c0 + lane] = s_out[wave][g][lane];
}

#define TOPK_B_THREADS 256
// Selection tail shared by the kernel-B variants: pooled[0..lim) holds the pooled scores.
// Each wavefront selects from its contiguous quarter, wavefront 0 merges, then indices and
// the raw scaled scores at the selected chunks are written.
struct TopkTailShared {
  float cand_s[4][TOPK_MAXK];
  int cand_i[4][TOPK_MAXK];
  float merge_s[4 * TOPK_MAXK];
  int merge_i[4 * TOPK_MAXK];
  int ncand_s[4];
};

__device__ __forceinline__ void topk_tail(TopkTailShared& sh, const float* pooled, int lim,
                                          const float* rrow, long row, int N, int G, int topk,
                                          int32_t* indices, bf16_t* scores) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  {
    const int nseg_all = (lim + TOPK_NSEG - 1) / TOPK_NSEG;
    const int per = (nseg_all + 3) / 4;
    int nc = 0;
    for (int sg = wave * per; sg < (wave + 1) * per && sg < nseg_all; ++sg) {
      const int base = sg * TOPK_NSEG;
      const int ns = (lim - base < TOPK_NSEG) ? lim - base : TOPK_NSEG;
      nc = wave_select(pooled + base, ns, base, sh.cand_s[wave], sh.cand_i[wave], nc, topk);
    }
    if (lane == 0) sh.ncand_s[wave] = nc;
  }
  __syncthreads();
  if (wave == 0) {
    int tot = 0;
    for (int w = 0; w < 4; ++w) {
      const int n = sh.ncand_s[w];
      if (lane < n) {
        sh.merge_s[tot + lane] = sh.cand_s[w][lane];
        sh.merge_i[tot + lane] = sh.cand_i[w][lane];
      }
      tot += n;
    }
    const int nc = wave_select(sh.merge_s, tot, 0, sh.cand_s[0], sh.cand_i[0], 0, topk, sh.merge_i);
    if (lane == 0) sh.ncand_s[0] = nc;
  }
  __syncthreads();
  const int nc = sh.ncand_s[0];
  for (int kk = tid; kk < topk; kk += TOPK_B_THREADS) indices[row * topk + kk] = (kk < nc) ? sh.cand_i[0][kk] : -1;
  for (int p = tid; p < topk * G; p += TOPK_B_THREADS) {
    const int g = p / topk, kk = p - g * topk;
    const float val = (kk < nc) ? rrow[(long)g * N + sh.cand_i[0][kk]] : HILS_NEG_INF;
    scores[(row * G + g) * (long)topk + kk] = f2bf(val);
  }
}

// Kernel B, register variant (N <= 256 * EPT): each thread owns EPT consecutive chunks and
// keeps their G logits in registers from one vector load to the pooled score.
template <int GMAX, int EPT>
__global__ void __launch_bounds__(TOPK_B_THREADS)
topk_select_reg_kernel(const float* __restrict__ raw, const float* __restrict__ lse_swa,
                       const float* __restrict__ bias, const float* __restrict__ gumbel,
                       const int32_t* __restrict__ drop_mask, int32_t* __restrict__ indices,
                       bf16_t* __restrict__ scores, float* __restrict__ lse_total_out,
                       float* __restrict__ sel_logits_out, int L, int N, int h_kv, int G, int topk,
                       int block_size, int window_size, int causal, int q_offset) {
  extern __shared__ float pooled[];  // N floats
  __shared__ float redv[4][16];
  __shared__ float gmax[16];
  __shared__ float lse_tot[16];
  __shared__ TopkTailShared tail_sh;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long row = blockIdx.x;
  const int hk = (int)(row % h_kv);
  const long bt = row / h_kv;
  const int t = (int)(bt % L);
  const long b = bt / L;
  int lim = causal ? visible_limit(t + q_offset, window_size, block_size) : N;
  lim = lim < 0 ? 0 : (lim > N ? N : lim);
  const float* rrow = raw + row * (long)G * N;
  const int cb = tid * EPT;
  float x[GMAX][EPT];
  const bool vec = ((N & 3) == 0);
#pragma unroll
  for (int g = 0; g < GMAX; ++g) {
    if (g < G) {
      if (vec) {
#pragma unroll
        for (int e4 = 0; e4 < EPT / 4; ++e4) {
          float4 v4 = make_float4(0.f, 0.f, 0.f, 0.f);
          if (cb + e4 * 4 < N) v4 = *(const float4*)(rrow + (long)g * N + cb + e4 * 4);
          x[g][e4 * 4] = v4.x; x[g][e4 * 4 + 1] = v4.y; x[g][e4 * 4 + 2] = v4.z; x[g][e4 * 4 + 3] = v4.w;
        }
      } else {
#pragma unroll
        for (int e = 0; e < EPT; ++e) x[g][e] = (cb + e < N) ? rrow[(long)g * N + cb + e] : 0.f;
      }
#pragma unroll
      for (int e = 0; e < EPT; ++e) {
        const int c = cb + e;
        float xv = x[g][e];
        if (c < lim) {
          if (bias) xv = __fadd_rn(xv, bias[((b * N + c) * (long)h_kv + hk) * G + g]);
          if (gumbel) xv = __fadd_rn(xv, gumbel[(long)(hk * G + g) * N + c]);
        } else {
          xv = HILS_NEG_INF;
        }
        x[g][e] = xv;
      }
      float m = HILS_NEG_INF;
#pragma unroll
      for (int e = 0; e < EPT; ++e) m = fmaxf(m, x[g][e]);
      m = wave_max(m);
      if (lane == 0) redv[wave][g] = m;
    }
  }
  __syncthreads();
  if (tid < G) gmax[tid] = fmaxf(fmaxf(redv[0][tid], redv[1][tid]), fmaxf(redv[2][tid], redv[3][tid]));
  __syncthreads();
#pragma unroll
  for (int g = 0; g < GMAX; ++g) {
    if (g < G) {
      const float m = gmax[g];
      float l = 0.f;
      if (m > HILS_NEG_INF) {
#pragma unroll
        for (int e = 0; e < EPT; ++e) l += __expf(x[g][e] - m);
      }
      l = wave_sum(l);
      if (lane == 0) redv[wave][g] = l;
    }
  }
  __syncthreads();
  if (tid < G) {
    const float l = redv[0][tid] + redv[1][tid] + redv[2][tid] + redv[3][tid];
    const float lse_hils = (l > 0.f) ? gmax[tid] + logf(l) : HILS_NEG_INF;
    const float tot = logaddexp_f(lse_swa[row * G + tid], lse_hils);
    lse_tot[tid] = tot;
    if (lse_total_out) lse_total_out[row * G + tid] = tot;
  }
  __syncthreads();
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int c = cb + e;
    float best = HILS_NEG_INF;
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
      if (g < G) {
        const float xv = x[g][e];
        const float nrm = (xv == HILS_NEG_INF) ? HILS_NEG_INF : __fsub_rn(xv, lse_tot[g]);
        best = fmaxf(best, nrm);
        if (sel_logits_out && c < N) sel_logits_out[(row * G + g) * (long)N + c] = xv;
      }
    }
    if (c < lim) {
      if (drop_mask && drop_mask[bt * (long)N + c] != 0) best = HILS_NEG_INF;
      pooled[c] = best;
    }
  }
  __syncthreads();
  topk_tail(tail_sh, pooled, lim, rrow, row, N, G, topk, indices, scores);
}

// Kernel B, generic variant (any N up to 16384): logits are re-read from the scratch.
__global__ void __launch_bounds__(TOPK_B_THREADS)
topk_select_kernel(const float* __restrict__ raw, const float* __restrict__ lse_swa,
                   const float* __restrict__ bias, const float* __restrict__ gumbel,
                   const int32_t* __restrict__ drop_mask, int32_t* __restrict__ indices,
                   bf16_t* __restrict__ scores, float* __restrict__ lse_total_out,
                   float* __restrict__ sel_logits_out, int L, int N, int h_kv, int G, int topk,
                   int block_size, int window_size, int causal, int q_offset) {
  extern __shared__ float pooled[];  // N floats
  __shared__ float redv[4][16];
  __shared__ float gmax[16];
  __shared__ float lse_tot[16];
  __shared__ TopkTailShared tail_sh;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long row = blockIdx.x;  // (b*L + t)*h_kv + hk
  const int hk = (int)(row % h_kv);
  const long bt = row / h_kv;
  const int t = (int)(bt % L);
  const long b = bt / L;
  int lim = causal ? visible_limit(t + q_offset, window_size, block_size) : N;
  lim = lim < 0 ? 0 : (lim > N ? N : lim);
  const float* rrow = raw + row * (long)G * N;
  auto xval = [&](int g, int c) -> float {
    float x = rrow[(long)g * N + c];
    if (bias) x = __fadd_rn(x, bias[((b * N + c) * (long)h_kv + hk) * G + g]);
    if (gumbel) x = __fadd_rn(x, gumbel[(long)(hk * G + g) * N + c]);
    return x;
  };
  for (int g = 0; g < G; ++g) {
    float m = HILS_NEG_INF;
    for (int c = tid; c < lim; c += TOPK_B_THREADS) m = fmaxf(m, xval(g, c));
    m = wave_max(m);
    if (lane == 0) redv[wave][g] = m;
  }
  __syncthreads();
  if (tid < G) gmax[tid] = fmaxf(fmaxf(redv[0][tid], redv[1][tid]), fmaxf(redv[2][tid], redv[3][tid]));
  __syncthreads();
  for (int g = 0; g < G; ++g) {
    const float m = gmax[g];
    float l = 0.f;
    if (m > HILS_NEG_INF)
      for (int c = tid; c < lim; c += TOPK_B_THREADS) l += __expf(xval(g, c) - m);
    l = wave_sum(l);
    if (lane == 0) redv[wave][g] = l;
  }
  __syncthreads();
  if (tid < G) {
    const float l = redv[0][tid] + redv[1][tid] + redv[2][tid] + redv[3][tid];
    const float lse_hils = (l > 0.f) ? gmax[tid] + logf(l) : HILS_NEG_INF;
    const float tot = logaddexp_f(lse_swa[row * G + tid], lse_hils);
    lse_tot[tid] = tot;
    if (lse_total_out) lse_total_out[row * G + tid] = tot;
  }
  __syncthreads();
  for (int c = tid; c < N; c += TOPK_B_THREADS) {
    float best = HILS_NEG_INF;
    for (int g = 0; g < G; ++g) {
      float x = HILS_NEG_INF;
      if (c < lim) {
        x = xval(g, c);
        const float nrm = (x == HILS_NEG_INF) ? HILS_NEG_INF : __fsub_rn(x, lse_tot[g]);
        best = fmaxf(best, nrm);
      }
      if (sel_logits_out) sel_logits_out[(row * G + g) * (long)N + c] = x;
    }
    if (c < lim) {
      if (drop_mask && drop_mask[bt * (long)N + c] != 0) best = HILS_NEG_INF;
      pooled[c] = best;
    }
  }
  __syncthreads();
  topk_tail(tail_sh, pooled, lim, rrow, row, N, G, topk, indices, scores);
}

// ---------------------------------------------------------------------------
// Few queries, about one (query, KV head) row per compute unit: one workgroup of 16 wavefronts
// per row does everything.  The row's chunk keys are streamed once with coalesced 16-byte lane
// loads (two register buffers in flight per wavefront), the raw scaled logits stay in LDS, and
// LSE, pooling, the 16 per-wavefront selections and their merge follow without leaving the
// workgroup: no scratch in HBM and no second launch.
// ---------------------------------------------------------------------------
#define TOPK_R_WAVES 16  // most wavefronts of a row workgroup (sizes the shared arrays)
#define TOPK_R_MAXN 4096

__device__ __forceinline__ float wave_max_f(float x) {
  x = fmaxf(x, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(x), __float_as_int(x), 0xB1, 0xF, 0xF, false)));
  x = fmaxf(x, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(x), __float_as_int(x), 0x4E, 0xF, 0xF, false)));
  x = fmaxf(x, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(x), __float_as_int(x), 0x141, 0xF, 0xF, false)));
  x = fmaxf(x, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(x), __float_as_int(x), 0x140, 0xF, 0xF, false)));
  const int xi = __float_as_int(x);
  return fmaxf(fmaxf(__int_as_float(__builtin_amdgcn_readlane(xi, 0)), __int_as_float(__builtin_amdgcn_readlane(xi, 16))),
               fmaxf(__int_as_float(__builtin_amdgcn_readlane(xi, 32)), __int_as_float(__builtin_amdgcn_readlane(xi, 48))));
}
__device__ __forceinline__ float wave_sum_f(float x) {
  x = row_sum<16>(x);
  const int xi = __float_as_int(x);
  return (__int_as_float(__builtin_amdgcn_readlane(xi, 0)) + __int_as_float(__builtin_amdgcn_readlane(xi, 16))) +
         (__int_as_float(__builtin_amdgcn_readlane(xi, 32)) + __int_as_float(__builtin_amdgcn_readlane(xi, 48)));
}

// GM: the query heads of a row the kernel is built for (4 or 8)
template <int GM>
struct TopkRowSharedT {
  float cand_s[TOPK_R_WAVES][64];
  int cand_i[TOPK_R_WAVES][64];
  float merge_s[TOPK_R_WAVES * TOPK_MAXK];
  int merge_i[TOPK_R_WAVES * TOPK_MAXK];
  int ncand[TOPK_R_WAVES];
  // (max, sum of exponentials) of every streamed key group, one component per head: combined in a
  // fixed order, so the log-sum-exp does not depend on which wavefront drew which group
  float grp_m[TOPK_R_MAXN / 32][GM];
  float grp_l[TOPK_R_MAXN / 32][GM];
  uint32_t gmax[64];           // largest selection key of every 16-lane group of the workgroup
  int wcnt[TOPK_R_WAVES];      // keys of a wavefront that reach the candidate bound
  float tot[GM];               // lse_total per head
  int rank[64];                            // one-launch decode step: candidates ahead of each candidate
  int win_i[TOPK_MAXK];                    // ... the winners' chunks, ascending, -1 padded
  bf16_t win_w[GM * (TOPK_MAXK + 1) + 2];   // ... and the heads' inter-chunk weights, [head][topk + 1]
  uint32_t thr;                // the candidate bound
  int next_group;
};
#define TOPK_R_CAND 256  // candidates the single-wavefront final selection takes

// One (query, KV head) row (row = (b*L + t)*h_kv + hk) by a workgroup of NW wavefronts; dyn = the
// workgroup's dynamic LDS (topk_row_smem bytes).
// FUSED (the one-launch decode step): the row's attention follows in the same workgroup.  Every
// wavefront then works out the winners itself and leaves the row's indices and inter-chunk weights in
// LDS (sh.win_i, sh.win_w: the same values from every wavefront), where the attention reads them
// without waiting for anybody; wavefront 0 writes the selection's global outputs on the way.
template <int D, int GMAX, int NW, bool PAGED, bool FUSED = false, int GI = 8>  // GI: load instructions per register buffer
__device__ __forceinline__ void
topk_row_body(const bf16_t* __restrict__ q, const bf16_t* __restrict__ lmks,
              const float* __restrict__ lse_swa, const float* __restrict__ bias, int32_t* __restrict__ indices,
              bf16_t* __restrict__ scores, float* __restrict__ lse_total_out,
              float* __restrict__ sel_logits_out, bf16_t* __restrict__ weights_out, int L, int N,
              int NP, int h_kv, int G, int topk, int block_size, int window_size, int causal, int q_offset,
              float sm_scale, const int32_t* __restrict__ page_table, int max_pages, int num_pages,
              int lmk_hm, int lmk_cap, int perq, int bias_inplace, float* dyn, const long row,
              TopkRowSharedT<GMAX>* sh_p = nullptr) {
  // bias_inplace (with a bias only): the staged bias and the logits share one array, a slot holding the
  // bias until the chunk's logit is added to it; a winner's bias is then read again from global memory
  // and its raw score is the biased logit minus that bias (one rounding of the sum away from the raw
  // product, far inside the bf16 the score is returned in).  For rows whose two arrays do not fit the LDS.
  // perq: one chunk key per QUERY head, lmks = (B,N,h_kv*G,D) / (B,h_kv*G,lmk_cap,D) / (num_pages,h_kv*G,D):
  // the row streams G key tensors, a key group of head g gives the logits of MFMA column g only
  constexpr int LR = D / 8, TPI = 64 / LR;
  constexpr int THREADS = NW * 64;       // NW = 8 or 16 wavefronts
  constexpr int EPT = TOPK_R_MAXN / THREADS;  // 64-chunk slots of a wavefront's share
  static_assert(GI == 8 || GI == 16, "a key group is 8 or 16 load instructions");
  constexpr int KG = GI * TPI;   // chunk keys per buffer
  float* logit_s = dyn;                       // [GMAX][NP] raw scaled logits
  float* pooled = dyn + (size_t)GMAX * NP;    // [NP]
  // paged chunk keys, lmks = (num_pages, h_kv, D): the row's page ids are staged behind the pooled scores
  int* page_s = (int*)(pooled + NP);          // [NP], only with a page table (else 0 entries)
  const int NPG = PAGED ? NP : 0;
  // the row's additive bias (the layer's prior bias: added to the logits for the log-sum-exp and the
  // selection, and, rounded the layer's way, to the winners' scores before the inter-chunk softmax),
  // staged head-major like the logits; 0 for the chunks past the causal limit
  const bool inplace = bias && bias_inplace;
  float* bias_s = inplace ? logit_s : (float*)(page_s + NPG);  // [GMAX][NP], only with a bias
  const int NBS = (bias && !inplace) ? GMAX * NP : 0;          // the wavefronts' staging areas follow
  __shared__ TopkRowSharedT<GMAX> sh_own;
  TopkRowSharedT<GMAX>& sh = FUSED ? *sh_p : sh_own;  // FUSED: the caller's, which the attention reads after the return
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int piece = lane % LR, tsub = lane / LR;
  const int hk = (int)(row % h_kv);
  const long bt = row / h_kv;
  const int t = (int)(bt % L);
  const long b = bt / L;
  int lim = causal ? visible_limit(t + q_offset, window_size, block_size) : N;
  lim = lim < 0 ? 0 : (lim > N ? N : lim);
  float swa[GMAX];
#pragma unroll
  for (int g = 0; g < GMAX; ++g) swa[g] = (g < G) ? lse_swa[row * G + g] : 0.f;
  if (tid == 0) sh.next_group = 2 * NW;
  if (bias) {
    // chunk c of this row: the G biases are contiguous in all three layouts
    for (int c = tid; c < NP; c += THREADS) {
      float bv[GMAX];
#pragma unroll
      for (int g = 0; g < GMAX; ++g) bv[g] = 0.f;
      if (c < lim) {
        long e0;
        if (PAGED) {
          const int pg = c < max_pages ? page_table[b * max_pages + c] : -1;
          e0 = ((long)((pg >= 0 && pg < num_pages) ? pg : 0) * h_kv + hk) * G;
        } else if (lmk_hm) {
          e0 = ((b * h_kv + hk) * (long)lmk_cap + c) * G;
        } else {
          e0 = ((b * N + c) * (long)h_kv + hk) * G;
        }
#pragma unroll
        for (int g = 0; g < GMAX; ++g)
          if (g < G) bv[g] = bias[e0 + g];
      }
#pragma unroll
      for (int g = 0; g < GMAX; ++g) bias_s[g * NP + c] = bv[g];
    }
  }
  // the query heads as B operand of the logit products, lane (head = lane & 15, j = lane >> 4) holds
  // features ks*32 + 8j ..; loaded here so that the barrier below has waited for them
  typedef unsigned tr_u4 __attribute__((ext_vector_type(4)));
  bf16x8_t qb[D / 32];
#pragma unroll
  for (int ks = 0; ks < D / 32; ++ks) {
    tr_u4 t = {0u, 0u, 0u, 0u};
    if ((lane & 15) < G) t = *(const tr_u4*)(q + (row * (long)G + (lane & 15)) * D + ks * 32 + (lane >> 4) * 8);
    qb[ks] = __builtin_bit_cast(bf16x8_t, t);
  }
  // have them arrive here: a load still pending at the streaming loop's first use would make the
  // compiler wait for every load in flight there, in every iteration
#pragma unroll
  for (int ks = 0; ks < D / 32; ++ks) asm volatile("" : "+v"(qb[ks]));
  if (PAGED) {  // every entry a load or a mask may look at gets a value
    for (int c = tid; c < NP; c += THREADS) {
      int pg = (c < lim && c < max_pages) ? page_table[b * max_pages + c] : -1;
      page_s[c] = (pg >= 0 && pg < num_pages) ? pg : -1;
    }
  }
  __syncthreads();

  // ---- phase 1: logits of the visible chunks.  The chunk-key rows arrive by coalesced 16-byte lane
  // loads (LR lanes per row), are written row-major (rows padded by 16 bytes: no bank conflicts
  // either way) into the wavefront's staging area 16 keys at a time and read back as the A operand
  // of S^T = LMK q^T, the query heads in the MFMA columns: a few instructions per key row, so the
  // phase runs at the speed of the memory stream ----
  {
    constexpr int KS = D / 32;
    constexpr int ROWB = 2 * D + 16;
    constexpr int LPT = 16 / TPI;  // load instructions per 16-key tile
    char* stage_w = (char*)((float*)(page_s + NPG) + NBS) + (size_t)wave * 16 * ROWB;
    const int col = lane & 15, j = lane >> 4;
    char* const w_addr = stage_w + tsub * ROWB + piece * 16;
    const char* const k_addr = stage_w + col * ROWB + j * 16;
    // key groups of the row: KG chunks each, times the G heads when every query head has its own keys
    // (group number = chunk group * G + head: the heads of a chunk are neighbours in memory)
    const int GK = perq ? G : 1;                  // key tensors of the row
    const int h_lmk = h_kv * GK;                  // heads of the key tensor
    const int ngroups = ((lim + KG - 1) / KG) * GK;
    // dense chunk keys: (B, N, h_lmk, D), or head-major (B, h_lmk, lmk_cap, D) (a row's keys contiguous)
    const bf16_t* base = lmks + (lmk_hm ? (b * h_lmk + hk * GK) * (long)lmk_cap * D : (b * N * (long)h_lmk + hk * GK) * D) + piece * 8;
    const long cstride = (PAGED || !lmk_hm) ? (long)h_lmk * D : (long)D;
    const long gstride = (!PAGED && lmk_hm) ? (long)lmk_cap * D : (long)D;  // from a head to the next of the group
    const bf16_t* pbase = lmks + (long)hk * GK * D + piece * 8;  // paged: + page * h_lmk * D
    auto fetch = [&](tr_u4 (&kr)[GI], int vg) __attribute__((always_inline)) {
      const int grp = perq ? vg / G : vg;
      const long goff = perq ? (vg - grp * G) * gstride : 0;
#pragma unroll
      for (int it = 0; it < GI; ++it) {
        int c = grp * KG + it * TPI + tsub;
        c = c < N ? c : N - 1;
        if (PAGED) {
          const int pg = page_s[c];  // an unmapped or invisible chunk reads page 0 and is masked below
          kr[it] = *(const tr_u4*)(pbase + goff + (long)(pg < 0 ? 0 : pg) * cstride);
        } else {
          kr[it] = *(const tr_u4*)(base + goff + c * cstride);
        }
      }
    };
    auto consume = [&](const tr_u4 (&kr)[GI], int vg) __attribute__((always_inline)) {
      const int grp = perq ? vg / G : vg;
      const int gh = perq ? vg - grp * G : -1;  // the head these keys belong to (-1: to all heads)
      // the MFMA columns this group fills: its head's (with the last head's keys also the columns past G,
      // whose logit rows and sums hold -inf / 0 as with shared keys)
      const bool mine = gh < 0 ? col < GMAX : (col == gh || (gh == G - 1 && col >= G && col < GMAX));
      float m_run = HILS_NEG_INF, l_run = 0.f;  // this lane's head over the group's keys it sees
#pragma unroll
      for (int tt = 0; tt < GI / LPT; ++tt) {
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int ii = 0; ii < LPT; ++ii) *(tr_u4*)(w_addr + ii * TPI * ROWB) = kr[tt * LPT + ii];
        __builtin_amdgcn_wave_barrier();
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const tr_u4 a = *(const tr_u4*)(k_addr + ks * 64);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), qb[ks], acc, 0, 0, 0);
        }
        // accumulator register i of lane (head = col, j) is key c0 + 4j + i
        const int c0 = grp * KG + tt * 16 + 4 * j;
        if (mine) {  // (the rows of the heads past G hold -inf)
          f32x4_t out;
#pragma unroll
          for (int i = 0; i < 4; ++i) out[i] = (c0 + i < lim && col < G) ? __fmul_rn(acc[i], sm_scale) : HILS_NEG_INF;
          if (PAGED) {  // c0 + 3 < NP: groups end at a multiple of 64 at most
            typedef int tr_i4 __attribute__((ext_vector_type(4)));
            const tr_i4 pg4 = *(const tr_i4*)&page_s[c0];
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (pg4[i] < 0) out[i] = HILS_NEG_INF;
          }
          if (!inplace) *(f32x4_t*)&logit_s[col * NP + c0] = out;
          if (bias) {  // -inf stays -inf: the staged bias is finite (0 past the causal limit)
            const f32x4_t bb = *(const f32x4_t*)&bias_s[col * NP + c0];
#pragma unroll
            for (int i = 0; i < 4; ++i) out[i] = __fadd_rn(out[i], bb[i]);
            if (inplace) *(f32x4_t*)&logit_s[col * NP + c0] = out;
          }
          // running log-sum-exp of this lane's head over the keys it has seen
          const float mn = fmaxf(fmaxf(m_run, fmaxf(out[0], out[1])), fmaxf(out[2], out[3]));
          const float ms = (mn == HILS_NEG_INF) ? 0.f : mn * HILS_LOG2E;
          float add = 0.f;
#pragma unroll
          for (int i = 0; i < 4; ++i) add += __builtin_amdgcn_exp2f(fmaf(out[i], HILS_LOG2E, -ms));
          l_run = fmaf(l_run, __builtin_amdgcn_exp2f(fmaf(m_run, HILS_LOG2E, -ms)), add);
          m_run = mn;
        }
      }
      // the group's (max, sum) per head: the four lane rows of a column hold the same head
      const float M = rows_max(m_run);
      const float Ms = (M == HILS_NEG_INF) ? 0.f : M * HILS_LOG2E;
      const float Lg = rows_sum(l_run * __builtin_amdgcn_exp2f(fmaf(m_run, HILS_LOG2E, -Ms)));
      if (j == 0 && mine) {  // lanes of heads past G never left (-inf, 0)
        sh.grp_m[grp][col] = M;
        sh.grp_l[grp][col] = Lg;
      }
    };
    // Groups of KG keys are handed out through a counter in LDS: the wavefronts of a workgroup
    // are served unevenly by the memory system, a fixed share would wait for the slowest.
    // The first two groups of every wavefront are fixed (wave, wave + NW), the rest drawn.
    auto draw = [&]() -> int {
      int v = 0;
      if (lane == 0) v = atomicAdd(&sh.next_group, 1);
      return __builtin_amdgcn_readfirstlane(v);
    };
    // drawn group numbers only grow, so the first one past the end ends the wavefront's walk
    const int last = ngroups - 1;
    tr_u4 ka[GI], kb[GI];
    int ga = wave, gb = wave + NW;
    if (ngroups > 0) {
      fetch(ka, ga < last ? ga : last);
      fetch(kb, gb < last ? gb : last);
    }
    while (ga < ngroups) {
      consume(ka, ga);
      ga = draw();
      fetch(ka, ga < last ? ga : last);
      if (gb >= ngroups) break;
      consume(kb, gb);
      gb = draw();
      fetch(kb, gb < last ? gb : last);
    }
  }
  __syncthreads();

  // ---- phase 2: LSE per head from the key groups' partial sums.  Work every wavefront would do
  // alike costs its instruction count once per wavefront of a SIMD, so one wavefront per head does
  // it and the result goes through LDS ----
  static_assert((GMAX == 4 || GMAX == 8) && NW >= GMAX, "one wavefront per head, four or eight heads per group entry");
  if (wave < GMAX) {
    const int g = wave;
    const int ngroups = (lim + KG - 1) / KG;
    float mw = HILS_NEG_INF;
    for (int i = lane; i < ngroups; i += 64) mw = fmaxf(mw, sh.grp_m[i][g]);
    const float mx = wave_max_f(mw);
    float part = 0.f;
    for (int i = lane; i < ngroups; i += 64) {
      const float mi = sh.grp_m[i][g];
      part += (mi > HILS_NEG_INF) ? sh.grp_l[i][g] * __expf(mi - mx) : 0.f;
    }
    const float lsum = wave_sum_f(part);
    const float lse_hils = (lsum > 0.f) ? mx + __logf(lsum) : HILS_NEG_INF;
    float sw = swa[0];
#pragma unroll
    for (int g2 = 1; g2 < GMAX; ++g2) sw = (g == g2) ? swa[g2] : sw;
    // logaddexp on the hardware exp2/log2
    const float hi = fmaxf(sw, lse_hils), lo = fminf(sw, lse_hils);
    const float t = (lo == HILS_NEG_INF) ? hi : hi + __logf(1.f + __expf(lo - hi));
    if (lane == 0) {
      sh.tot[g] = t;
      if (lse_total_out && g < G) lse_total_out[row * G + g] = t;
    }
  }
  __syncthreads();
  float tot[GMAX];
#pragma unroll
  for (int g = 0; g < GMAX; ++g) tot[g] = sh.tot[g];
  // ---- phase 3: selection.  Wavefront w owns the chunks [w*per, (w+1)*per); the selection key of a
  // chunk is max over the heads of (logit - lse_total) as an order-preserving integer ----
  const int per = ((N + NW - 1) / NW + 63) & ~63;  // <= 64 * EPT
  const int cbase = wave * per;
  uint32_t key[EPT];
  uint32_t lmax = 0u;
  // (the options are decided outside the unrolled loops: a run-time flag tested per element is a branch
  // per element; the logit rows of the heads past G hold -inf, so every head is read alike)
  auto form_keys = [&](auto with_bias) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      key[e] = 0u;
      if (e * 64 < per) {  // uniform: the slots past the wavefront's share cost nothing
        const int c = cbase + e * 64 + lane;
        const bool mine = c < lim;
        float best = HILS_NEG_INF;
#pragma unroll
        for (int g = 0; g < GMAX; ++g) {
          float xv = mine ? logit_s[g * NP + c] : HILS_NEG_INF;
          if (decltype(with_bias)::value) xv = mine ? __fadd_rn(xv, bias_s[g * NP + c]) : xv;  // the sum the log-sum-exp saw
          const float nrm = (xv == HILS_NEG_INF) ? HILS_NEG_INF : __fsub_rn(xv, tot[g]);
          best = fmaxf(best, nrm);
        }
        if (mine) pooled[c] = best;
        key[e] = score_key(best);
        lmax = key[e] > lmax ? key[e] : lmax;
      }
    }
  };
  if (bias && !inplace) form_keys(std::true_type{}); else form_keys(std::false_type{});
  if (sel_logits_out) {  // the exported selection logits (a debugging output)
    for (int i = tid; i < G * N; i += THREADS) {
      const int g = i / N, c = i - g * N;
      float xv = c < lim ? logit_s[g * NP + c] : HILS_NEG_INF;
      if (bias && !inplace && c < lim) xv = __fadd_rn(xv, bias_s[g * NP + c]);
      sel_logits_out[(row * G + g) * (long)N + c] = xv;
    }
  }
  // A lower bound of the topk-th largest key with few keys above it: the topk-th largest of the
  // maxima of the workgroup's 16-lane groups (4 * NW of them), found by one wavefront.  The keys
  // that reach it are compacted in chunk order into one list and a single wavefront selects
  // among them.
  {
    uint32_t gm = lmax, y;
    y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)gm, 0xB1, 0xF, 0xF, true);  gm = gm > y ? gm : y;
    y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)gm, 0x4E, 0xF, 0xF, true);  gm = gm > y ? gm : y;
    y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)gm, 0x141, 0xF, 0xF, true); gm = gm > y ? gm : y;
    // 64 groups in all: 16-lane groups with 16 wavefronts, 8-lane groups with 8 (the bound is the
    // topk-th largest of the 64 group maxima: with fewer, coarser groups it lets too many keys through)
    if constexpr (NW >= 16) {
      y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)gm, 0x140, 0xF, 0xF, true); gm = gm > y ? gm : y;
      if ((lane & 15) == 0) sh.gmax[wave * 4 + (lane >> 4)] = gm;
      if (NW * 4 < 64 && tid >= NW * 4 && tid < 64) sh.gmax[tid] = 0u;
    } else {
      static_assert(NW == 8 || NW >= 16, "group maxima: 8 or 16 wavefronts");
      if ((lane & 7) == 0) sh.gmax[wave * 8 + (lane >> 3)] = gm;
    }
  }
  __syncthreads();
  if (wave == 0) {
    uint32_t t = 1u;  // every valid key is >= 1
    const uint32_t gv = sh.gmax[lane];
    if (__popcll(__ballot(gv != 0u)) >= topk) {
      const uint32_t hi = wave_max_u(gv);
      const uint32_t lo = ~wave_max_u(gv ? ~gv : 0u);  // smallest non-zero group maximum
      t = lane_kth_largest(gv, lo, hi, topk);
    }
    if (lane == 0) sh.thr = t;
  }
  __syncthreads();
  const unsigned long long lt = (1ull << lane) - 1ull;
  const uint32_t thr = sh.thr;
  {
    int cnt = 0;
#pragma unroll
    for (int e = 0; e < EPT; ++e)
      if (e * 64 < per) cnt += __popcll(__ballot(key[e] >= thr));
    if (lane == 0) sh.wcnt[wave] = cnt;
    if (FUSED && wave == 0) sh.rank[lane] = 0;
  }
  __syncthreads();
  int cand_base = 0, cand_total = 0;
#pragma unroll
  for (int w2 = 0; w2 < NW; ++w2) {
    const int v = sh.wcnt[w2];
    cand_total += v;
    cand_base += (w2 < wave) ? v : 0;
  }
  // the bias of (chunk c, head g) and the raw scaled score of that pair
  auto bias_at = [&](int c, int g) -> float {
    if (!inplace) return bias_s[g * NP + c];
    long e0;
    if (PAGED) {
      const int pg = page_s[c];
      e0 = ((long)(pg < 0 ? 0 : pg) * h_kv + hk) * G;
    } else if (lmk_hm) {
      e0 = ((b * h_kv + hk) * (long)lmk_cap + c) * G;
    } else {
      e0 = ((b * N + c) * (long)h_kv + hk) * G;
    }
    return bias[e0 + g];
  };
  // ---- FUSED: what every wavefront does once lane kk (kk < nc) holds winner kk's chunk (ascending) ----
  auto fused_tail = [&](int widx, int nc) __attribute__((always_inline)) {
    const bool has = lane < nc;
    float xs[GMAX], wgt[GMAX], wloc[GMAX], bws[GMAX];
    // (the winner's biases first, all heads' loads in flight together: read from global memory when the
    // bias shares the logits' array)
#pragma unroll
    for (int g = 0; g < GMAX; ++g) bws[g] = (bias && has && g < G) ? bias_at(widx, g) : 0.f;
#pragma unroll
    for (int g = 0; g < GMAX; ++g) {
      xs[g] = (has && g < G) ? logit_s[g * NP + widx] : HILS_NEG_INF;  // raw scaled score
      const float bw = bws[g];
      if (inplace && has && g < G) xs[g] = __fsub_rn(xs[g], bw);
      // the layer's inter-chunk softmax over [scores as bf16 (+ bias as bf16, summed in bf16), lse_swa]
      float x = HILS_NEG_INF;
      if (has && g < G) {
        x = bf2f(f2bf(xs[g]));
        if (bias) x = bf2f(f2bf(x + bf2f(f2bf(bw))));
      }
      const float m = fmaxf(wave_max_f(x), swa[g]);
      if (m == HILS_NEG_INF) {  // every logit -inf: NaN row, as a softmax gives
        wgt[g] = wloc[g] = __uint_as_float(0x7fc00000u);
      } else {
        const float e = (x == HILS_NEG_INF) ? 0.f : __expf(x - m);
        const float el = __expf(swa[g] - m);
        const float inv = 1.f / (wave_sum_f(e) + el);
        wgt[g] = e * inv;
        wloc[g] = el * inv;
      }
    }
    if (wave == 0) {  // the selection's outputs
      if (lane < topk) indices[row * topk + lane] = has ? widx : -1;
#pragma unroll
      for (int g = 0; g < GMAX; ++g)
        if (g < G) {
          if (lane < topk) scores[(row * G + g) * (long)topk + lane] = f2bf(xs[g]);
          if (weights_out) {
            bf16_t* wrow = weights_out + (row * G + g) * (long)(topk + 1);
            if (lane < topk) wrow[lane] = f2bf(wgt[g]);
            if (lane == 0) wrow[topk] = f2bf(wloc[g]);
          }
        }
    }
    // the row's indices and weights for the attention, in the layout of the global tensors
    if (lane < topk) sh.win_i[lane] = has ? widx : -1;
#pragma unroll
    for (int g = 0; g < GMAX; ++g)
      if (g < G) {
        if (lane < topk) sh.win_w[g * (topk + 1) + lane] = f2bf(wgt[g]);
        if (lane == 0) sh.win_w[g * (topk + 1) + topk] = f2bf(wloc[g]);
      }
    __builtin_amdgcn_wave_barrier();
  };
  if (cand_total <= TOPK_R_CAND) {
    uint32_t* ck = (uint32_t*)sh.merge_s;  // NW * TOPK_MAXK >= 512 entries
    int pos = cand_base;
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      if (e * 64 < per) {
        const bool pred = key[e] >= thr;
        const unsigned long long m = __ballot(pred);
        if (pred) {
          const int o = pos + __popcll(m & lt);
          ck[o] = key[e];
          sh.merge_i[o] = cbase + e * 64 + lane;
        }
        pos += __popcll(m);
      }
    }
    __syncthreads();
    if constexpr (FUSED) {
      if (cand_total <= 64) {
        // One candidate per lane, in chunk order: its rank among the candidates (keys descending, ties
        // to the lower chunk) says whether it wins, the winners before it give its slot.  Every
        // wavefront does this for itself: no hand-over, no barrier before the attention's first loads.
        // The 64 x 64 comparisons are shared out: wavefront w compares every candidate with candidates
        // w * 64 / NW ..., the partial ranks meet in LDS.
        const uint32_t kc = lane < cand_total ? ck[lane] : 0u;  // (valid keys are >= 1)
        const int ci = lane < cand_total ? sh.merge_i[lane] : -1;
        {
          constexpr int JW = 64 / NW;
          int part = 0;
#pragma unroll
          for (int u = 0; u < JW; ++u) {
            const int jj = wave * JW + u;
            const uint32_t kj = (uint32_t)__builtin_amdgcn_readlane((int)kc, jj);
            part += ((kj > kc) | ((kj == kc) & (jj < lane))) ? 1 : 0;
          }
          if (part) atomicAdd(&sh.rank[lane], part);
        }
        lds_barrier();
        const int rank = sh.rank[lane];
        const bool win = lane < cand_total && rank < topk;
        const unsigned long long wm = __ballot(win);
        if (win) sh.cand_i[wave][__popcll(wm & lt)] = ci;
        __builtin_amdgcn_wave_barrier();
        const int nc = __popcll(wm);
        fused_tail(lane < nc ? sh.cand_i[wave][lane] : -1, nc);
        return;
      }
    }
    if (wave == 0) {
      // (the usual case, about 1.4 topk candidates, is one key per lane)
      const int nc = cand_total <= 64
                         ? wave_select<true, 1>((const float*)ck, cand_total, 0, sh.cand_s[0], sh.cand_i[0], 0, topk,
                                                sh.merge_i)
                         : wave_select<true, TOPK_R_CAND / 64>((const float*)ck, cand_total, 0, sh.cand_s[0],
                                                               sh.cand_i[0], 0, topk, sh.merge_i);
      if (lane == 0) sh.ncand[0] = nc;
    }
  } else {
    // many keys at the bound (equal scores, or fewer than topk groups with a visible chunk while
    // more than TOPK_R_CAND chunks are visible): every wavefront selects among its own chunks,
    // winners (padded to topk entries with -inf) into its slice of the merge list, one wavefront merges
    int nc = 0;
    if (cbase < lim) {
      const int ns = (lim - cbase < per) ? lim - cbase : per;
      nc = wave_select<false, EPT>(pooled + cbase, ns, cbase, sh.merge_s + wave * topk,
                                   sh.merge_i + wave * topk, 0, topk, nullptr, sh.cand_s[wave],
                                   sh.cand_i[wave]);
    }
    if (lane >= nc && lane < topk) {
      sh.merge_s[wave * topk + lane] = HILS_NEG_INF;
      sh.merge_i[wave * topk + lane] = 0;
    }
    __syncthreads();
    if (wave == 0) {
      const int total = NW * topk;
      int nc2 = 0;
      for (int p0 = 0; p0 < total; p0 += TOPK_NSEG) {
        const int ns = (total - p0 < TOPK_NSEG) ? total - p0 : TOPK_NSEG;
        nc2 = wave_select(sh.merge_s + p0, ns, 0, sh.cand_s[0], sh.cand_i[0], nc2, topk, sh.merge_i + p0);
      }
      if (lane == 0) sh.ncand[0] = nc2;
    }
  }
  __syncthreads();
  if constexpr (FUSED) {  // the selections that did not fit one lane per candidate: winners from LDS
    const int nc = sh.ncand[0];
    fused_tail(lane < nc ? sh.cand_i[0][lane] : -1, nc);
    return;
  }
  // ---- phase 4: indices (ascending) and the raw scaled scores of the winners ----
  const int nc = sh.ncand[0];
  for (int kk = tid; kk < topk; kk += THREADS) indices[row * topk + kk] = (kk < nc) ? sh.cand_i[0][kk] : -1;
  for (int p = tid; p < topk * G; p += THREADS) {
    const int g = p / topk, kk = p - g * topk;
    float val = (kk < nc) ? logit_s[g * NP + sh.cand_i[0][kk]] : HILS_NEG_INF;
    if (inplace && kk < nc) val = __fsub_rn(val, bias_at(sh.cand_i[0][kk], g));
    scores[(row * G + g) * (long)topk + kk] = f2bf(val);
  }
  // optional: the layer's inter-chunk softmax over [scores (as bf16), lse_swa], one wavefront per head
  if (weights_out && wave < G) {
    const int g = wave;
    float lse_g = swa[0];
#pragma unroll
    for (int g2 = 1; g2 < GMAX; ++g2) lse_g = (g == g2) ? swa[g2] : lse_g;
    float x = HILS_NEG_INF;
    if (lane < topk && lane < nc) {
      const int cw = sh.cand_i[0][lane];
      const float bw = bias ? bias_at(cw, g) : 0.f;
      x = bf2f(f2bf(inplace ? __fsub_rn(logit_s[g * NP + cw], bw) : logit_s[g * NP + cw]));
      // the layer adds the gathered bias, cast to the scores' dtype, to the bf16 scores
      if (bias) x = bf2f(f2bf(x + bf2f(f2bf(bw))));
    }
    const float m = fmaxf(wave_max_f(x), lse_g);
    bf16_t* wrow = weights_out + (row * G + g) * (long)(topk + 1);
    if (m == HILS_NEG_INF) {  // every logit -inf: NaN row, as a softmax gives
      if (lane <= topk) wrow[lane] = 0x7fc0;
    } else {
      const float e = (x == HILS_NEG_INF) ? 0.f : __expf(x - m);
      const float el = __expf(lse_g - m);
      const float inv = 1.f / (wave_sum_f(e) + el);
      if (lane < topk) wrow[lane] = f2bf(e * inv);
      if (lane == 0) wrow[topk] = f2bf(el * inv);
    }
  }
}

template <int D, int GMAX, int NW, bool PAGED>
__global__ void __launch_bounds__(NW * 64)
topk_row_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ lmks,
                const float* __restrict__ lse_swa, const float* __restrict__ bias, int32_t* __restrict__ indices,
                bf16_t* __restrict__ scores, float* __restrict__ lse_total_out,
                float* __restrict__ sel_logits_out, bf16_t* __restrict__ weights_out, int L, int N,
                int NP, int h_kv, int G, int topk, int block_size, int window_size, int causal, int q_offset,
                float sm_scale, const int32_t* __restrict__ page_table, int max_pages, int num_pages,
                int lmk_hm, int lmk_cap, int perq, int bias_inplace) {
  extern __shared__ __align__(16) float topk_row_dyn[];
  topk_row_body<D, GMAX, NW, PAGED>(q, lmks, lse_swa, bias, indices, scores, lse_total_out, sel_logits_out,
                                    weights_out, L, N, NP, h_kv, G, topk, block_size, window_size, causal,
                                    q_offset, sm_scale, page_table, max_pages, num_pages, lmk_hm, lmk_cap, perq,
                                    bias_inplace, topk_row_dyn, (long)blockIdx.x);
}

// The remote branch of a decode step in one launch: the workgroup of a (query, KV head) row selects
// the row's chunks and writes indices, scores and the inter-chunk softmax weights (topk_row_body),
// then attends over the selected chunks (decode_rows_body) reading back what it has just written
// (the barrier between the two makes a workgroup's own global writes visible to it).  The rows
// drift apart, so while some compute units run the selection's tail the others keep the memory
// system busy, and the step pays one launch.
#define DS_WAVES 8
struct DsArgs {
  const bf16_t *q, *lmks, *k, *v;
  const float *lse_swa, *bias;
  int32_t* indices;
  bf16_t *scores, *weights, *o;
  float *lse_total, *sel_logits;
  int L, N, NP, h_kv, G, topk, block_size, window_size, q_offset;
  float sm_scale_sel;
  const int32_t* page_table;
  int max_pages, num_pages, lmk_hm, lmk_cap, perq, bias_inplace;
  int stagger_ticks;  // 100 MHz ticks by which every other row of an XCD starts late (0: none)
  DrDims dr;
};
// PAGED: the chunk keys (and the bias) are addressed through the page table; the attention reads
// K and V through it whenever a.dr.page_table is set.
template <int D, bool PAGED, int GMAX>
__global__ void __launch_bounds__(DS_WAVES * 64) decode_step_kernel(DsArgs a) {
  extern __shared__ __align__(16) float ds_dyn[];
  const long row = blockIdx.x;
  __shared__ TopkRowSharedT<GMAX> ds_sh;
  // With at most one row per compute unit all rows run in step: every compute unit streams keys, then
  // every one sits in the selection's tail with the memory system idle, then every one streams K and V.
  // Half of the rows (every other one of an XCD's) start a little late, so that one half's tail falls
  // into the other half's streaming (75.5 -> 72.2 us at 256 rows of 2048 keys with 8 us; 5 us: 75.0,
  // 12 us: 74.2; thirds or a continuous spread of the start times did less).
  if (a.stagger_ticks > 0 && ((blockIdx.x >> 3) & 1)) {
    const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
    while (__builtin_amdgcn_s_memrealtime() - t0 < (unsigned long long)a.stagger_ticks) __builtin_amdgcn_s_sleep(8);
  }
  topk_row_body<D, GMAX, DS_WAVES, PAGED, true>(a.q, a.lmks, a.lse_swa, a.bias, a.indices, a.scores, a.lse_total,
                                             a.sel_logits, a.weights, a.L, a.N, a.NP, a.h_kv, a.G, a.topk,
                                             a.block_size, a.window_size, 1, a.q_offset, a.sm_scale_sel,
                                             a.page_table, a.max_pages, a.num_pages, a.lmk_hm, a.lmk_cap, a.perq,
                                             a.bias_inplace, ds_dyn, row, &ds_sh);
  // The attention reads the row's indices and weights where the selection left them in LDS: the
  // pointers are offset so that the row's entries of the (B, L, heads, ...) tensors fall there.  Its
  // staging areas lie over the selection's logits: the barrier that separates the two uses runs in
  // every wavefront once its first chunk's loads are in flight.
  const int hk = (int)(row % a.h_kv);
  const long bt = row / a.h_kv;
  const bf16_t* w_row = ds_sh.win_w - (bt * a.dr.HQ + hk * a.G) * (long)a.dr.NW;
  const int32_t* i_row = ds_sh.win_i - (bt * a.dr.H + hk) * (long)a.dr.K;
  decode_rows_body<D, DS_WAVES>(a.q, a.k, a.v, w_row, i_row, a.o, nullptr, a.dr, (char*)ds_dyn, 0, hk, bt,
                                [] __device__() { lds_barrier(); });  // (no wait for the loads in flight)
}

static int topk_cus() { return hils_device_cus(); }

// the one-pass prefill kernel (topk_group.hip)
bool hils_topk_group_covers(int N, int G, int D, int topk, int per_qhead, bool plain);
int hils_topk_group_launch(const void* q, const void* lmk_packed, const float* lse_swa, const float* bias,
                           int32_t* indices, void* scores, float* lse_total, float* sel_logits, int B, int L, int N, int h_kv,
                           int G, int D, int topk, int block_size, int window_size, int causal, int q_offset,
                           float sm_scale, int lse_bf16, int per_qhead, void* stream);

// rows = (query, KV head) pairs; the row kernel wants about one row per compute unit
// LDS of a row workgroup before the wavefronts' staging areas: raw logits [gm][NP] (gm = 4 head slots, 8
// with more than four query heads per KV head), pooled scores, page ids (paged chunk keys), the staged
// bias [gm][NP]
// (inplace: the bias shares the logits' array)
static size_t topk_row_smem_base(int N, int G, bool paged, bool with_bias, bool inplace) {
  const int NP = (N + 63) & ~63;
  const int gm = G <= 4 ? 4 : 8;
  return (size_t)(gm + 1 + (paged ? 1 : 0) + (with_bias && !inplace ? gm : 0)) * NP * sizeof(float);
}
static size_t topk_row_shared_bytes(int G) { return G <= 4 ? sizeof(TopkRowSharedT<4>) : sizeof(TopkRowSharedT<8>); }
// Does a row workgroup of `waves` wavefronts fit the LDS?  *inplace: the bias has to share the logits' array.
static bool topk_row_fits(int N, int G, int D, bool paged, bool with_bias, int waves, int* inplace) {
  const size_t rest = (size_t)waves * 16 * (2 * D + 16) + topk_row_shared_bytes(G);
  *inplace = 0;
  if (topk_row_smem_base(N, G, paged, with_bias, false) + rest <= 158 * 1024) return true;
  *inplace = 1;
  return with_bias && topk_row_smem_base(N, G, paged, true, true) + rest <= 158 * 1024;
}

// plain: no Gumbel noise and no drop mask; a bias is staged in LDS beside the logits and must fit there
static bool topk_use_row(long rows, int N, int G, int D, int per_qhead, bool plain, bool with_bias = false,
                         bool paged = false) {
  int inplace;
  if ((D == 64 || D == 128) && !topk_row_fits(N, G, D, paged, with_bias, 8, &inplace)) return false;
  (void)per_qhead;  // shared chunk keys or one per query head: the same kernel
  return plain && G <= 8 && (D == 64 || D == 128) && N >= 256 && N <= TOPK_R_MAXN &&
         rows >= 96 && rows <= 2147483647L;
}

static int topk_fwd_row(const void* q, const void* lmks, const float* lse_swa, const float* bias, int32_t* indices,
                        void* scores, float* lse_total, float* sel_logits, void* weights, int B, int L, int N, int h_kv, int G, int D,
                        int topk, int block_size, int window_size, int causal, int q_offset,
                        float sm_scale, hipStream_t st, const int32_t* page_table = nullptr, int max_pages = 0,
                        int num_pages = 0, int lmk_hm = 0, int lmk_cap = 0, int perq = 0) {
  const long rows = (long)B * L * h_kv;
  const int NP = (N + 63) & ~63;
  // then 16 padded key rows of staging per wavefront
  const size_t stage_b = (size_t)16 * (2 * D + 16);
  // one round of rows or less: 16 wavefronts per row (the whole compute unit streams one row) if
  // their staging areas fit the LDS beside the logits; more rows than compute units: 8, so that
  // two workgroups share a unit and one row's selection overlaps the other row's streaming
  // (with a bias: 16 only if that does not push the bias into the logits' array where 8 would not)
  int ip16 = 0, ip8 = 0;
  const bool fit16 = rows <= topk_cus() && topk_row_fits(N, G, D, page_table != nullptr, bias != nullptr, 16, &ip16);
  const bool fit8 = topk_row_fits(N, G, D, page_table != nullptr, bias != nullptr, 8, &ip8);
  HILS_REQUIRE(fit16 || fit8, "hils_topk_fwd: too many chunks (%d) for the logits of the row's heads in LDS", N);
  const bool wide = fit16 && (!ip16 || !fit8 || ip8);
  const int bias_inplace = wide ? ip16 : ip8;
  const size_t smem = topk_row_smem_base(N, G, page_table != nullptr, bias != nullptr, bias_inplace != 0) +
                      (wide ? 16 : 8) * stage_b;
#define TOPK_ROW_CALL_G(D_, G_, W_, P_)                                                           \
  do {                                                                                           \
    auto kern = topk_row_kernel<D_, G_, W_, P_>;                                                 \
    static HilsLdsReserve reserved;                                                              \
    if (int rc = hils_reserve_lds(&reserved, (const void*)kern, smem, "hils_topk_fwd")) return rc; \
    hipLaunchKernelGGL(kern, dim3((unsigned)rows), dim3(W_ * 64), smem, st,                      \
                       (const bf16_t*)q, (const bf16_t*)lmks, lse_swa, bias, indices, (bf16_t*)scores, \
                       lse_total, sel_logits, (bf16_t*)weights, L, N, NP, h_kv, G, topk,         \
                       block_size, window_size, causal, q_offset, sm_scale, page_table, max_pages, \
                       num_pages, lmk_hm, lmk_cap, perq, bias_inplace);                          \
  } while (0)
#define TOPK_ROW_CALL_W(D_, W_, P_)                                                               \
  do {                                                                                           \
    if (G <= 4) TOPK_ROW_CALL_G(D_, 4, W_, P_); else TOPK_ROW_CALL_G(D_, 8, W_, P_);             \
  } while (0)
#define TOPK_ROW_CALL(D_, P_)                                                                    \
  do {                                                                                           \
    if (wide) TOPK_ROW_CALL_W(D_, 16, P_); else TOPK_ROW_CALL_W(D_, 8, P_);                      \
  } while (0)
  if (page_table) {
    if (D == 64) TOPK_ROW_CALL(64, true); else TOPK_ROW_CALL(128, true);
  } else {
    if (D == 64) TOPK_ROW_CALL(64, false); else TOPK_ROW_CALL(128, false);
  }
#undef TOPK_ROW_CALL
#undef TOPK_ROW_CALL_W
#undef TOPK_ROW_CALL_G
  return HILS_OK;
}

// ---- the remote branch of a decode step in one launch (decode_step_kernel) ----
bool hils_decode_rows_covers(int D, int Dv, int G, int K);

extern "C" int hils_decode_step_covers(int B, int L, int N, int HQ, int H, int D, int topk, int block_size,
                                       int with_bias) {
  if (B <= 0 || L <= 0 || H <= 0 || HQ <= 0 || HQ % H != 0 || topk < 1 || topk > TOPK_MAXK || block_size != DR_S)
    return 0;
  const int G = HQ / H;
  // (paged chunk keys stage their page ids too: the stricter of the two LDS budgets)
  return topk_use_row((long)B * L * H, N, G, D, 0, true, with_bias != 0, true) && hils_decode_rows_covers(D, D, G, topk) ? 1 : 0;
}

static int decode_step_launch(const void* q, const void* lmks, const void* k, const void* v, const float* lse_swa,
                              const float* bias, int lmk_paged, int lmk_hm, int lmk_cap, int perq, int32_t* indices, void* scores, void* weights, void* o, float* lse_total,
                              float* sel_logits, int B, int L, int Lkv, int N, int HQ, int H, int D, int topk,
                              int block_size, int window_size, int q_offset, float sm_scale_sel,
                              float sm_scale_attn, int mask_last, const int32_t* page_table, int max_pages,
                              int num_pages, hipStream_t st) {
  const int G = HQ / H;
  const long rows = (long)B * L * H;
  const int NP = (N + 63) & ~63;
  int bias_inplace = 0;
  const bool sel_fits = topk_row_fits(N, G, D, lmk_paged != 0, bias != nullptr, DS_WAVES, &bias_inplace);
  const size_t sel_b = topk_row_smem_base(N, G, lmk_paged != 0, bias != nullptr, bias_inplace != 0) +
                       (size_t)DS_WAVES * 16 * (2 * D + 16);
  HILS_REQUIRE(sel_fits,
               "hils_decode_step: too many chunks (%d) for the logits (and the bias) of the row's heads in LDS", N);
  const size_t att_b = dr_smem_bytes(D, G, DS_WAVES);
  const size_t smem = sel_b > att_b ? sel_b : att_b;
  DsArgs a;
  a.q = (const bf16_t*)q; a.lmks = (const bf16_t*)lmks; a.k = (const bf16_t*)k; a.v = (const bf16_t*)v;
  a.lse_swa = lse_swa; a.bias = bias; a.indices = indices;
  a.lmk_hm = lmk_hm; a.lmk_cap = lmk_cap; a.perq = perq; a.bias_inplace = bias_inplace;
  a.stagger_ticks = rows <= topk_cus() ? 800 : 0;  // one round of rows: they would run in step
  a.scores = (bf16_t*)scores; a.weights = (bf16_t*)weights; a.o = (bf16_t*)o;
  a.lse_total = lse_total; a.sel_logits = sel_logits;
  a.L = L; a.N = N; a.NP = NP; a.h_kv = H; a.G = G; a.topk = topk; a.block_size = block_size;
  a.window_size = window_size; a.q_offset = q_offset; a.sm_scale_sel = sm_scale_sel;
  a.page_table = page_table; a.max_pages = max_pages; a.num_pages = num_pages;
  a.dr = DrDims{L, Lkv, HQ, H, G, topk, topk + 1, page_table ? max_pages : Lkv / DR_S, 1, mask_last,
                sm_scale_attn, page_table, max_pages, num_pages};
#define DS_CALL_G(D_, P_, G_)                                                                      \
  do {                                                                                             \
    auto kern = decode_step_kernel<D_, P_, G_>;                                                    \
    static HilsLdsReserve reserved;                                                                \
    if (int rc = hils_reserve_lds(&reserved, (const void*)kern, smem, "hils_decode_step")) return rc; \
    hipLaunchKernelGGL(kern, dim3((unsigned)rows), dim3(DS_WAVES * 64), smem, st, a);              \
  } while (0)
#define DS_CALL(D_, P_)                                                                            \
  do {                                                                                             \
    if (G <= 4) DS_CALL_G(D_, P_, 4); else DS_CALL_G(D_, P_, 8);                                   \
  } while (0)
  if (lmk_paged) {
    if (D == 64) DS_CALL(64, true); else DS_CALL(128, true);
  } else {
    if (D == 64) DS_CALL(64, false); else DS_CALL(128, false);
  }
#undef DS_CALL
#undef DS_CALL_G
  return HILS_OK;
}

extern "C" int hils_decode_step(const void* q, const void* lmks, const void* k, const void* v,
                                const float* lse_swa, const float* bias, int32_t* indices, void* scores,
                                void* weights, void* o, float* lse_total, float* sel_logits, int B, int L, int Lkv,
                                int N, int HQ, int H, int D, int topk, int block_size, int window_size,
                                int q_offset, float sm_scale_sel, float sm_scale_attn, int mask_last,
                                int lmk_head_major, int lmk_cap, int lmk_per_qhead, void* stream) {
  HILS_REQUIRE(q && lmks && k && v && lse_swa && indices && scores && weights && o, "hils_decode_step: null pointer");
  HILS_REQUIRE(B > 0 && L > 0 && N > 0 && H > 0 && HQ > 0 && HQ % H == 0, "hils_decode_step: bad sizes");
  HILS_REQUIRE(!lmk_head_major || lmk_cap >= N, "hils_decode_step: lmk_cap (%d) must be at least N (%d)", lmk_cap, N);
  HILS_REQUIRE(Lkv >= (long)N * block_size, "hils_decode_step: the cache (%d tokens) is shorter than %d chunks", Lkv, N);
  HILS_REQUIRE(hils_decode_step_covers(B, L, N, HQ, H, D, topk, block_size, bias != nullptr),
               "hils_decode_step: shape not covered (hils_decode_step_covers): use hils_topk_fwd_weights + hils_sparse_attn_fwd");
  HILS_REQUIRE((long)B * L * H <= 2147483647L, "hils_decode_step: grid too large");
  if (int rc = decode_step_launch(q, lmks, k, v, lse_swa, bias, 0, lmk_head_major, lmk_cap, lmk_per_qhead, indices, scores, weights, o,
                                  lse_total, sel_logits, B, L, Lkv, N, HQ, H, D, topk, block_size, window_size,
                                  q_offset, sm_scale_sel, sm_scale_attn, mask_last, nullptr, 0, 0,
                                  (hipStream_t)stream))
    return rc;
  HILS_CHECK_LAUNCH("hils_decode_step");
  return HILS_OK;
}

extern "C" int hils_decode_step_paged(const void* q, const void* lmk_pages, const void* k_pages,
                                      const void* v_pages, const int32_t* page_table, const float* lse_swa,
                                      const float* bias, int32_t* indices, void* scores, void* weights, void* o,
                                      float* lse_total, float* sel_logits, int B, int L, int N, int HQ, int H,
                                      int D, int topk, int block_size, int window_size, int q_offset,
                                      int max_pages, int num_pages, float sm_scale_sel, float sm_scale_attn,
                                      int mask_last, int lmk_dense, int lmk_head_major, int lmk_cap,
                                      int lmk_per_qhead, void* stream) {
  HILS_REQUIRE(!lmk_dense || !lmk_head_major || lmk_cap >= N,
               "hils_decode_step_paged: lmk_cap (%d) must be at least N (%d)", lmk_cap, N);
  HILS_REQUIRE(q && lmk_pages && k_pages && v_pages && page_table && lse_swa && indices && scores && weights && o,
               "hils_decode_step_paged: null pointer");
  HILS_REQUIRE(B > 0 && L > 0 && N > 0 && H > 0 && HQ > 0 && HQ % H == 0 && max_pages >= N && num_pages > 0,
               "hils_decode_step_paged: sizes must be positive and the page table must cover N chunks");
  HILS_REQUIRE(hils_decode_step_covers(B, L, N, HQ, H, D, topk, block_size, bias != nullptr),
               "hils_decode_step_paged: shape not covered (hils_decode_step_covers): use hils_topk_fwd_weights_paged + hils_sparse_attn_decode_paged");
  HILS_REQUIRE((long)B * L * H <= 2147483647L, "hils_decode_step_paged: grid too large");
  if (int rc = decode_step_launch(q, lmk_pages, k_pages, v_pages, lse_swa, bias, lmk_dense ? 0 : 1,
                                  lmk_dense ? lmk_head_major : 0, lmk_cap, lmk_per_qhead, indices, scores, weights, o, lse_total,
                                  sel_logits, B, L, 0, N, HQ, H, D, topk, block_size, window_size, q_offset,
                                  sm_scale_sel, sm_scale_attn, mask_last, page_table, max_pages, num_pages,
                                  (hipStream_t)stream))
    return rc;
  HILS_CHECK_LAUNCH("hils_decode_step_paged");
  return HILS_OK;
}

static bool topk_use_split(int B, int L, int N, int h_kv) {
  const long fused_wgs = (long)B * ((L + TOPK_QT - 1) / TOPK_QT) * h_kv;
  return fused_wgs < 2L * topk_cus() && N >= 256 && N <= 16384;
}

// Shapes that hils_topk_fwd_weights hands to the one-pass prefill kernel, the only one that reads
// lse_swa in bf16 (mirrors the dispatch of topk_fwd_impl; the workspace must be given).
extern "C" int hils_topk_lse16_covers(int B, int L, int N, int h_kv, int G, int D, int topk) {
  if (B <= 0 || L <= 0 || N <= 0 || h_kv <= 0 || G <= 0) return 0;
  if (topk_use_split(B, L, N, h_kv)) return 0;
  if (L <= 4 && topk_use_row((long)B * L * h_kv, N, G, D, 0, true)) return 0;
  return hils_topk_group_covers(N, G, D, topk, 0, true) ? 1 : 0;
}

static size_t topk_ws_key_bytes(int B, int N, int h_kv, int G) {
  return (size_t)B * h_kv * G * ((N + 15) / 16) * 16 * 128 * sizeof(bf16_t);
}
// the bias of a call repacked behind the chunk keys of the workspace (topk_pack_bias_kernel)
static const float* topk_pack_bias(const float* bias, void* workspace, int B, int N, int h_kv, int G, hipStream_t st) {
  if (!bias || !workspace || G > 8) return nullptr;
  float* out = (float*)((char*)workspace + topk_ws_key_bytes(B, N, h_kv, G));
  const int nblk16 = (N + 15) / 16;
  const long total = (long)B * h_kv * G * nblk16 * 16;
  hipLaunchKernelGGL(topk_pack_bias_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, bias, out, N,
                     h_kv * G, nblk16, total);
  return out;
}

extern "C" size_t hils_topk_fwd_workspace(int B, int L, int N, int h_kv, int G) {
  // many queries: room for the chunk keys repacked into MFMA operand order (head dim up to 128; a key
  // per query head when the caller's keys are per query head)
  // and behind them for an additive bias in blocks of 16 chunks per head
  if (!topk_use_split(B, L, N, h_kv))
    return G <= 8 ? topk_ws_key_bytes(B, N, h_kv, G) + (size_t)B * h_kv * G * ((N + 15) / 16) * 16 * sizeof(float) : 0;
  return (size_t)B * L * h_kv * G * N * sizeof(float);
}

static int topk_fwd_split(const void* q, const void* lmks, const float* lse_swa, const float* bias,
                          const float* gumbel, const int32_t* drop_mask, int32_t* indices,
                          void* scores, float* lse_total, float* sel_logits, float* raw, int B, int L,
                          int N, int h_kv, int G, int D, int topk, int block_size, int window_size,
                          int causal, int q_offset, int per_qhead, float sm_scale, hipStream_t st) {
  dim3 ga((N + TOPK_A_CHUNKS - 1) / TOPK_A_CHUNKS, h_kv, (unsigned)((long)B * L));
#define TOPK_A_CALL(D_, G_)                                                                      \
  hipLaunchKernelGGL((topk_logits_kernel<D_, G_>), ga, dim3(TOPK_A_THREADS), 0, st,              \
                     (const bf16_t*)q, (const bf16_t*)lmks, raw, L, N, h_kv, G, per_qhead, sm_scale)
  if (D == 64) {
    if (G <= 4) TOPK_A_CALL(64, 4); else TOPK_A_CALL(64, 16);
  } else {
    if (G <= 4) TOPK_A_CALL(128, 4); else TOPK_A_CALL(128, 16);
  }
#undef TOPK_A_CALL
  const long rows = (long)B * L * h_kv;
  const size_t smem = (size_t)N * sizeof(float);
#define TOPK_B_REG(G_, E_)                                                                         \
  hipLaunchKernelGGL((topk_select_reg_kernel<G_, E_>), dim3((unsigned)rows), dim3(TOPK_B_THREADS),  \
                     smem, st, raw, lse_swa, bias, gumbel, drop_mask, indices, (bf16_t*)scores,     \
                     lse_total, sel_logits, L, N, h_kv, G, topk, block_size, window_size, causal,   \
                     q_offset)
  if (N <= 256 * 8) {
    if (G <= 4) TOPK_B_REG(4, 8); else TOPK_B_REG(16, 8);
  } else if (N <= 256 * 16 && G <= 4) {
    TOPK_B_REG(4, 16);
  } else {
    static HilsLdsReserve reserved;
    if (int rc = hils_reserve_lds(&reserved, (const void*)topk_select_kernel, smem, "hils_topk_fwd")) return rc;
    hipLaunchKernelGGL(topk_select_kernel, dim3((unsigned)rows), dim3(TOPK_B_THREADS), smem, st, raw,
                       lse_swa, bias, gumbel, drop_mask, indices, (bf16_t*)scores, lse_total,
                       sel_logits, L, N, h_kv, G, topk, block_size, window_size, causal, q_offset);
  }
#undef TOPK_B_REG
  return HILS_OK;
}

// weights_fused: the row kernel also writes the inter-chunk softmax (set to 1 when it did)
static int topk_fwd_impl(const void* q, const void* lmks, const float* lse_swa,
                         const float* bias, const float* gumbel, const int32_t* drop_mask,
                         int32_t* indices, void* scores, float* lse_total, float* sel_logits,
                         void* workspace, size_t workspace_bytes, void* weights, const float* prior_b,
                         int* weights_fused, int B, int L, int N,
                         int h_kv, int G, int D, int topk, int block_size, int window_size,
                         int causal, int q_offset, int per_qhead, float sm_scale, void* stream,
                         int lse_bf16 = 0) {
  HILS_REQUIRE(q && lmks && lse_swa && indices && scores, "hils_topk_fwd: null pointer");
  HILS_REQUIRE(B > 0 && L > 0 && N > 0 && h_kv > 0 && G > 0 && D > 0, "hils_topk_fwd: sizes must be positive");
  HILS_REQUIRE(topk >= 1 && topk <= TOPK_MAXK, "hils_topk_fwd: topk (%d) must be in 1..%d", topk, TOPK_MAXK);
  HILS_REQUIRE(G <= 16, "hils_topk_fwd: group size %d not supported (max 16)", G);
  HILS_REQUIRE(block_size > 0, "hils_topk_fwd: block_size must be positive");
  HILS_REQUIRE(h_kv <= 65535 && B <= 65535, "hils_topk_fwd: h_kv/B too large for the grid");
  HILS_REQUIRE(!workspace || workspace_bytes >= hils_topk_fwd_workspace(B, L, N, h_kv, G),
               "hils_topk_fwd: workspace of %zu bytes is shorter than the %zu bytes hils_topk_fwd_workspace "
               "returns for this shape", workspace_bytes, hils_topk_fwd_workspace(B, L, N, h_kv, G));
  hipStream_t st = (hipStream_t)stream;
  HILS_REQUIRE(!lse_bf16 || hils_topk_lse16_covers(B, L, N, h_kv, G, D, topk),
               "hils_topk_fwd_weights_lse16: shape not taken by the one-pass prefill kernel "
               "(ask hils_topk_lse16_covers and pass lse_swa in fp32 otherwise)");
  // few queries per (batch, KV head) (decode, short continuations): one workgroup per row whenever
  // there are enough rows to occupy the machine, however many more there are
  // (with a bias the row kernel's inter-chunk softmax adds that same bias to the winners' scores:
  // it writes the weights only when the caller's prior bias is this bias)
  if ((topk_use_split(B, L, N, h_kv) || L <= 4) &&
      topk_use_row((long)B * L * h_kv, N, G, D, per_qhead, !gumbel && !drop_mask, bias != nullptr)) {
    const bool w_here = weights != nullptr && prior_b == bias;
    *weights_fused = w_here;
    if (int rc2 = topk_fwd_row(q, lmks, lse_swa, bias, indices, scores, lse_total, sel_logits, w_here ? weights : nullptr,
                               B, L, N, h_kv, G, D, topk, block_size, window_size, causal, q_offset, sm_scale, st,
                               nullptr, 0, 0, 0, 0, per_qhead))
      return rc2;
    HILS_CHECK_LAUNCH("hils_topk_fwd");
    return HILS_OK;
  }
  if (workspace && (D == 64 || D == 128) && topk_use_split(B, L, N, h_kv) &&
      (long)B * L <= 2147483647L / h_kv) {
    if (int rc2 = topk_fwd_split(q, lmks, lse_swa, bias, gumbel, drop_mask, indices, scores, lse_total,
                                 sel_logits, (float*)workspace, B, L, N, h_kv, G, D, topk, block_size,
                                 window_size, causal, q_offset, per_qhead, sm_scale, st))
      return rc2;
    HILS_CHECK_LAUNCH("hils_topk_fwd");
    return HILS_OK;
  }
  // the one-pass kernel with one chunk key per query head (a wavefront per head for the logits, G = 3..8),
  // or with more than four query heads on shared keys (two wavefronts per four queries)
  if ((per_qhead || G > 4) && workspace && hils_topk_group_covers(N, G, D, topk, per_qhead, !gumbel && !drop_mask)) {  // (G = 2..8 / 5..8)
    const int nblk16 = (N + 15) / 16;
    const int h_lmk = per_qhead ? h_kv * G : h_kv;
    const long total = (long)B * h_lmk * nblk16 * (D / 32) * 64;
    hipLaunchKernelGGL(topk_pack_lmk_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                       (const bf16_t*)lmks, (uint4*)workspace, N, h_lmk, D, nblk16, total);
    if (int rc2 = hils_topk_group_launch(q, workspace, lse_swa, bias, indices, scores, lse_total, sel_logits, B, L, N,
                                         h_kv, G, D, topk, block_size, window_size, causal, q_offset, sm_scale,
                                         lse_bf16, per_qhead ? 1 : 0, stream))
      return rc2;
    HILS_CHECK_LAUNCH("hils_topk_fwd");
    return HILS_OK;
  }
  // one chunk key per query head outside that kernel's envelope (more than 512 chunks, more than 32
  // winners, noise, a drop mask), or five to eight query heads on shared keys: the two-pass MFMA kernel,
  // 16 queries a wavefront, head by head
  if ((per_qhead || G > 4) && workspace && G <= 8 && (D == 64 || D == 128)) {
    const int nblk16 = (N + 15) / 16;
    const int h_lmk = per_qhead ? h_kv * G : h_kv;
    const long total = (long)B * h_lmk * nblk16 * (D / 32) * 64;
    hipLaunchKernelGGL(topk_pack_lmk_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                       (const bf16_t*)lmks, (uint4*)workspace, N, h_lmk, D, nblk16, total);
    const int segw = topk_rows_segw(N);
    const int NQ = 16;
    int pool_floats = NQ * (segw + 16);
    if (pool_floats < NQ * G * topk / 2) pool_floats = NQ * G * topk / 2;  // bf16 score staging
    pool_floats = (pool_floats + 3) & ~3;
    const size_t smem = sizeof(float) * ((size_t)pool_floats + 128 + (size_t)2 * NQ * topk + (size_t)G * NQ);
    dim3 grid_r((L + NQ - 1) / NQ, h_kv, B);
    const float* bias_pk = topk_pack_bias(bias, workspace, B, N, h_kv, G, st);
#define HILS_TOPK_ROWS_Q(KS_, PL_, BO_)                                                             \
  hipLaunchKernelGGL((topk_fwd_rows_kernel<1, KS_, PL_, true, true, BO_>), grid_r, dim3(64), smem, st, \
                     (const bf16_t*)q, (const bf16_t*)lmks, lse_swa, bias, gumbel, drop_mask,       \
                     indices, (bf16_t*)scores, lse_total, sel_logits, L, N, h_kv, G, topk,          \
                     block_size, window_size, causal, q_offset, sm_scale, segw, pool_floats,        \
                     (const uint4*)workspace, bias_pk, per_qhead ? G : 1)
    const bool plain = !bias && !gumbel && !drop_mask && !sel_logits;
    const bool bias_only = bias_pk && !gumbel && !drop_mask && !sel_logits;
    if (D == 64) {
      if (plain) HILS_TOPK_ROWS_Q(2, true, false); else if (bias_only) HILS_TOPK_ROWS_Q(2, false, true); else HILS_TOPK_ROWS_Q(2, false, false);
    } else {
      if (plain) HILS_TOPK_ROWS_Q(4, true, false); else if (bias_only) HILS_TOPK_ROWS_Q(4, false, true); else HILS_TOPK_ROWS_Q(4, false, false);
    }
#undef HILS_TOPK_ROWS_Q
    HILS_CHECK_LAUNCH("hils_topk_fwd");
    return HILS_OK;
  }
  if (!per_qhead && G <= 4 && (D == 64 || D == 128)) {
    const int segw = topk_rows_segw(N);
    const int NQ = (G == 1) ? 16 : 8;                                 // queries per wavefront
    const int GM = (G == 1) ? 1 : (G == 2 ? 2 : 4);
    int pool_floats = NQ * (segw + 16);                               // pooled scores of NQ queries
    if (pool_floats < NQ * GM * topk / 2) pool_floats = NQ * GM * topk / 2;  // bf16 score staging
    pool_floats = (pool_floats + 3) & ~3;
    const size_t smem = sizeof(float) * ((size_t)pool_floats + 128 + (size_t)2 * NQ * topk);
    dim3 grid_r((L + NQ - 1) / NQ, h_kv, B);
    // with a workspace the chunk keys are first repacked into MFMA operand order
    const uint4* packed = nullptr;
    if (workspace) {
      const int nblk16 = (N + 15) / 16;
      const long total = (long)B * h_kv * nblk16 * (D / 32) * 64;
      hipLaunchKernelGGL(topk_pack_lmk_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                         (const bf16_t*)lmks, (uint4*)workspace, N, h_kv, D, nblk16, total);
      packed = (const uint4*)workspace;
      // up to 512 chunks and 32 winners, nothing added to the logits: the one-pass kernel
      if (hils_topk_group_covers(N, G, D, topk, per_qhead, !gumbel && !drop_mask)) {
        if (int rc2 = hils_topk_group_launch(q, packed, lse_swa, bias, indices, scores, lse_total, sel_logits, B, L, N,
                                             h_kv, G, D, topk, block_size, window_size, causal, q_offset,
                                             sm_scale, lse_bf16, 0, stream))
          return rc2;
        HILS_CHECK_LAUNCH("hils_topk_fwd");
        return HILS_OK;
      }
    }
    const float* bias_pk = topk_pack_bias(bias, workspace, B, N, h_kv, G, st);
#define HILS_TOPK_ROWS_P(G_, KS_, PL_, PK_, BO_)                                                    \
  hipLaunchKernelGGL((topk_fwd_rows_kernel<G_, KS_, PL_, PK_, false, BO_>), grid_r, dim3(64), smem, st, \
                     (const bf16_t*)q, (const bf16_t*)lmks, lse_swa, bias, gumbel, drop_mask,       \
                     indices, (bf16_t*)scores, lse_total, sel_logits, L, N, h_kv, G, topk,          \
                     block_size, window_size, causal, q_offset, sm_scale, segw, pool_floats, packed, bias_pk, 1)
#define HILS_TOPK_ROWS(G_, KS_)                                                                     \
  do {                                                                                             \
    if (plain) {                                                                                   \
      if (packed) HILS_TOPK_ROWS_P(G_, KS_, true, true, false); else HILS_TOPK_ROWS_P(G_, KS_, true, false, false);   \
    } else if (bias_only) {                                                                        \
      HILS_TOPK_ROWS_P(G_, KS_, false, true, true);                                                \
    } else {                                                                                       \
      if (packed) HILS_TOPK_ROWS_P(G_, KS_, false, true, false); else HILS_TOPK_ROWS_P(G_, KS_, false, false, false); \
    }                                                                                              \
  } while (0)
    const bool plain = !bias && !gumbel && !drop_mask && !sel_logits;
    const bool bias_only = packed && bias_pk && !gumbel && !drop_mask && !sel_logits;
    if (G == 1) {
      if (D == 64) HILS_TOPK_ROWS(1, 2); else HILS_TOPK_ROWS(1, 4);
    } else if (G == 2) {
      if (D == 64) HILS_TOPK_ROWS(2, 2); else HILS_TOPK_ROWS(2, 4);
    } else {
      if (D == 64) HILS_TOPK_ROWS(4, 2); else HILS_TOPK_ROWS(4, 4);
    }
#undef HILS_TOPK_ROWS_P
#undef HILS_TOPK_ROWS
    HILS_CHECK_LAUNCH("hils_topk_fwd");
    return HILS_OK;
  }
  dim3 grid((L + TOPK_QT - 1) / TOPK_QT, h_kv, B);
  int rc;
#define HILS_TOPK_ARGS                                                                             \
  D, grid, st, (const bf16_t*)q, (const bf16_t*)lmks, lse_swa, bias, gumbel, drop_mask, indices,  \
      (bf16_t*)scores, lse_total, sel_logits, L, N, h_kv, G, topk, block_size, window_size, causal, \
      q_offset, per_qhead, sm_scale
  if (G == 1) rc = launch_topk<1>(HILS_TOPK_ARGS);
  else if (G == 2) rc = launch_topk<2>(HILS_TOPK_ARGS);
  else if (G <= 4) rc = launch_topk<4>(HILS_TOPK_ARGS);
  else if (G <= 8) rc = launch_topk<8>(HILS_TOPK_ARGS);
  else rc = launch_topk<16>(HILS_TOPK_ARGS);
#undef HILS_TOPK_ARGS
  if (rc) return rc;
  HILS_CHECK_LAUNCH("hils_topk_fwd");
  return HILS_OK;
}

extern "C" int hils_topk_fwd(const void* q, const void* lmks, const float* lse_swa,
                             const float* bias, const float* gumbel, const int32_t* drop_mask,
                             int32_t* indices, void* scores, float* lse_total, float* sel_logits,
                             void* workspace, size_t workspace_bytes, int B, int L, int N, int h_kv, int G,
                             int D, int topk, int block_size, int window_size, int causal, int q_offset,
                             int per_qhead, float sm_scale, void* stream) {
  int fused = 0;
  return topk_fwd_impl(q, lmks, lse_swa, bias, gumbel, drop_mask, indices, scores, lse_total, sel_logits,
                       workspace, workspace_bytes, nullptr, nullptr, &fused, B, L, N, h_kv, G, D, topk, block_size, window_size,
                       causal, q_offset, per_qhead, sm_scale, stream);
}

extern "C" int hils_topk_fwd_weights(const void* q, const void* lmks, const float* lse_swa,
                                     const float* bias, const float* prior_b, const float* gumbel,
                                     const int32_t* drop_mask,
                                     int32_t* indices, void* scores, void* weights, void* workspace,
                                     size_t workspace_bytes, int B, int L, int N, int h_kv, int G, int D, int topk,
                                     int block_size, int window_size, int causal, int q_offset,
                                     int per_qhead, float sm_scale, void* stream) {
  HILS_REQUIRE(weights, "hils_topk_fwd_weights: null pointer");
  int fused = 0;
  if (int rc = topk_fwd_impl(q, lmks, lse_swa, bias, gumbel, drop_mask, indices, scores, nullptr, nullptr,
                             workspace, workspace_bytes, weights, prior_b, &fused, B, L, N, h_kv, G, D, topk, block_size,
                             window_size, causal, q_offset, per_qhead, sm_scale, stream))
    return rc;
  if (fused) return HILS_OK;
  return hils_chunk_weights(scores, lse_swa, 0, prior_b, indices, weights, B, L, h_kv * G, h_kv, N, topk, 0,
                            stream);
}

extern "C" int hils_topk_fwd_weights_lse16(const void* q, const void* lmks, const void* lse_swa_bf16,
                                           const float* bias, const float* prior_b, int32_t* indices, void* scores, void* weights, void* workspace,
                                           size_t workspace_bytes, int B, int L, int N, int h_kv, int G, int D,
                                           int topk, int block_size, int window_size, int causal, int q_offset,
                                           float sm_scale, void* stream) {
  HILS_REQUIRE(weights && workspace, "hils_topk_fwd_weights_lse16: null pointer");
  int fused = 0;
  if (int rc = topk_fwd_impl(q, lmks, (const float*)lse_swa_bf16, bias, nullptr, nullptr, indices, scores,
                             nullptr, nullptr, workspace, workspace_bytes, weights, prior_b, &fused, B, L, N, h_kv, G, D,
                             topk, block_size, window_size, causal, q_offset, 0, sm_scale, stream, 1))
    return rc;
  if (fused) return HILS_OK;
  return hils_chunk_weights(scores, lse_swa_bf16, 1, prior_b, indices, weights, B, L, h_kv * G, h_kv, N, topk, 0,
                            stream);
}

// Decode over paged chunk keys (page = chunk = 64 tokens): lmk_pages (num_pages, h_kv, D) bf16 holds
// the pooled key of every page, page_table (B, max_pages) maps chunk c of batch element b to its
// page.  Selection + inter-chunk softmax as hils_topk_fwd_weights; one workgroup per (query, KV head).
extern "C" int hils_topk_fwd_weights_paged(const void* q, const void* lmk_pages, const int32_t* page_table,
                                           const float* lse_swa, const float* bias_pages, int32_t* indices, void* scores, void* weights,
                                           float* lse_total, float* sel_logits, int B, int L, int N, int h_kv,
                                           int G, int D, int topk, int block_size, int window_size, int q_offset,
                                           int max_pages, int num_pages, float sm_scale, int per_qhead, void* stream) {
  HILS_REQUIRE(q && lmk_pages && page_table && lse_swa && indices && scores && weights,
               "hils_topk_fwd_weights_paged: null pointer");
  HILS_REQUIRE(B > 0 && L > 0 && N > 0 && h_kv > 0 && max_pages >= N && num_pages > 0,
               "hils_topk_fwd_weights_paged: sizes must be positive and the page table must cover N chunks");
  HILS_REQUIRE(G >= 1 && G <= 8 && (D == 64 || D == 128) && N <= TOPK_R_MAXN && topk >= 1 && topk <= TOPK_MAXK &&
                   block_size > 0,
               "hils_topk_fwd_weights_paged: needs G <= 8, D in {64, 128}, N <= %d, topk <= %d", TOPK_R_MAXN,
               TOPK_MAXK);
  HILS_REQUIRE((long)B * L * h_kv <= 2147483647L, "hils_topk_fwd_weights_paged: grid too large");
  int paged_inplace;
  HILS_REQUIRE(topk_row_fits(N, G, D, true, bias_pages != nullptr, 8, &paged_inplace),
               "hils_topk_fwd_weights_paged: too many chunks (%d) for the logits (and the bias) of the row's heads in LDS", N);
  if (int rc = topk_fwd_row(q, lmk_pages, lse_swa, bias_pages, indices, scores, lse_total, sel_logits, weights, B, L,
                            N, h_kv, G, D, topk, block_size, window_size, 1, q_offset, sm_scale,
                            (hipStream_t)stream, page_table, max_pages, num_pages, 0, 0, per_qhead))
    return rc;
  HILS_CHECK_LAUNCH("hils_topk_fwd_weights_paged");
  return HILS_OK;
}

// ---------------------------------------------------------------------------
// hils_topk_fwd for callers that cannot allocate: the workspace is a file-scope device array.
// Every GPU the library runs on holds its own copy of the array until the process ends; in host
// code the array's name is only a stand-in, so its device address is looked up once per device
// (with that device current) and that pointer is what the kernels get.
// ---------------------------------------------------------------------------
#define HILS_TOPK_SCRATCH_BYTES ((size_t)8 << 20)
static __device__ __align__(256) unsigned char scratch[HILS_TOPK_SCRATCH_BYTES];
static std::atomic<void*> g_scratch_ptr[HILS_LDS_RESERVE_DEVICES];

static int topk_scratch_address(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= HILS_LDS_RESERVE_DEVICES) {
    (void)hipGetLastError();
    hils_set_error("hils_topk_fwd_noalloc: no current GPU (device ordinal %d)", dev);
    return HILS_ERR_LAUNCH;
  }
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();
      hils_set_error("hils_topk_fwd_noalloc: hipGetSymbolAddress failed on device %d: %s", dev,
                     hipGetErrorString(e));
      return HILS_ERR_LAUNCH;
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // the same address from whichever thread asks
  }
  *out = p;
  return HILS_OK;
}

extern "C" size_t hils_topk_fwd_noalloc_max_workspace(void) { return HILS_TOPK_SCRATCH_BYTES; }

extern "C" int hils_topk_fwd_noalloc(const void* q, const void* lmks, const float* lse_swa,
                                     const float* bias, const float* gumbel, const int32_t* drop_mask,
                                     int32_t* indices, void* scores, float* lse_total, float* sel_logits,
                                     int B, int L, int N, int h_kv, int G, int D, int topk,
                                     int block_size, int window_size, int causal, int q_offset,
                                     int per_qhead, float sm_scale, void* stream) {
  HILS_REQUIRE(B > 0 && L > 0 && N > 0 && h_kv > 0 && G > 0, "hils_topk_fwd_noalloc: sizes must be positive");
  const size_t need = hils_topk_fwd_workspace(B, L, N, h_kv, G);
  HILS_REQUIRE(need <= HILS_TOPK_SCRATCH_BYTES,
               "hils_topk_fwd_noalloc: this shape needs %zu bytes of scratch, the built-in buffer holds %zu; "
               "use hils_topk_fwd with a caller-allocated workspace",
               need, (size_t)HILS_TOPK_SCRATCH_BYTES);
  void* ws = nullptr;
  if (need > 0)
    if (int rc = topk_scratch_address(&ws)) return rc;
  // every byte a kernel of this call reads from the buffer is written earlier in the same call
  // (repacked chunk keys, or the logits parked between the two decode kernels): nothing to clear
  int fused = 0;
  return topk_fwd_impl(q, lmks, lse_swa, bias, gumbel, drop_mask, indices, scores, lse_total, sel_logits,
                       ws, HILS_TOPK_SCRATCH_BYTES, nullptr, nullptr, &fused, B, L, N, h_kv, G, D, topk, block_size, window_size, causal,
                       q_offset, per_qhead, sm_scale, stream);
}

// ---------------------------------------------------------------------------
// backward of the score gather: scores[b,t,h,g,k] = sm_scale * <q[b,t,h,g], lmk[b,idx,h(,g)]>
// ---------------------------------------------------------------------------
// One block per (b, t, hk); thread d owns one feature column.
__global__ void topk_bwd_kernel(const bf16_t* __restrict__ gs, const bf16_t* __restrict__ q,
                                const bf16_t* __restrict__ lmks, const int32_t* __restrict__ indices,
                                bf16_t* __restrict__ dq, float* __restrict__ dlmk, int L, int N,
                                int h_kv, int G, int D, int topk, int per_qhead, float sm_scale) {
  extern __shared__ float sm[];  // G*topk scaled grads, then topk indices
  float* gsc = sm;
  int* idx = (int*)(sm + G * topk);
  const long row = blockIdx.x;  // (b*L + t)*h_kv + hk
  const int hk = (int)(row % h_kv);
  const long bt = row / h_kv;
  const long b = bt / L;
  const int lmk_h = per_qhead ? h_kv * G : h_kv;
  for (int i = threadIdx.x; i < G * topk; i += blockDim.x) gsc[i] = bf2f(gs[row * G * topk + i]) * sm_scale;
  for (int i = threadIdx.x; i < topk; i += blockDim.x) idx[i] = indices[row * topk + i];
  __syncthreads();
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    for (int g = 0; g < G; ++g) {
      float a = 0.f;
      for (int k = 0; k < topk; ++k) {
        const int c = idx[k];
        if (c >= 0 && c < N)
          a += gsc[g * topk + k] * bf2f(lmks[((b * N + c) * (long)lmk_h + (per_qhead ? hk * G + g : hk)) * D + d]);
      }
      dq[(row * G + g) * D + d] = f2bf(a);
    }
    for (int k = 0; k < topk; ++k) {
      const int c = idx[k];
      if (c < 0 || c >= N) continue;
      if (per_qhead) {
        for (int g = 0; g < G; ++g) {
          const float v = gsc[g * topk + k] * bf2f(q[(row * G + g) * D + d]);
          if (v != 0.f) atomicAdd(dlmk + ((b * N + c) * (long)lmk_h + hk * G + g) * D + d, v);
        }
      } else {
        float v = 0.f;
        for (int g = 0; g < G; ++g) v += gsc[g * topk + k] * bf2f(q[(row * G + g) * D + d]);
        if (v != 0.f) atomicAdd(dlmk + ((b * N + c) * (long)lmk_h + hk) * D + d, v);
      }
    }
  }
}

// ---- backward without atomics (workspace given) ----
// dq: a thread owns 8 consecutive features of one (query, head): sum over the K slots of
// grad * chunk key (chunk keys stay in L2).
__global__ void __launch_bounds__(256)
topk_bwd_dq_kernel(const bf16_t* __restrict__ gs, const bf16_t* __restrict__ lmks,
                   const int32_t* __restrict__ indices, bf16_t* __restrict__ dq, long rows_g, int L, int N,
                   int h_kv, int G, int D, int topk, int per_qhead, float sm_scale) {
  const int pieces = D / 8;
  const long item = (long)blockIdx.x * 256 + threadIdx.x;  // (row, g, piece)
  if (item >= rows_g * pieces) return;
  const int pc = (int)(item % pieces);
  const long rg = item / pieces;      // (b*L + t)*h_kv + hk)*G + g
  const int g = (int)(rg % G);
  const long row = rg / G;
  const int hk = (int)(row % h_kv);
  const long b = row / h_kv / L;
  const int lmk_h = per_qhead ? h_kv * G : h_kv;
  const int lh = per_qhead ? hk * G + g : hk;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  for (int k = 0; k < topk; ++k) {
    const int c = indices[row * topk + k];
    if (c < 0 || c >= N) continue;
    const float gv = bf2f(gs[rg * topk + k]) * sm_scale;
    float f[8];
    unpack8(*(const uint4*)(lmks + ((b * N + c) * (long)lmk_h + lh) * D + pc * 8), f);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = fmaf(gv, f[e], acc[e]);
  }
  uint4 o;
  o.x = pack_bf2(acc[0], acc[1]);
  o.y = pack_bf2(acc[2], acc[3]);
  o.z = pack_bf2(acc[4], acc[5]);
  o.w = pack_bf2(acc[6], acc[7]);
  *(uint4*)(dq + rg * D + pc * 8) = o;
}

// dlmk: one workgroup per (batch, chunk-key head, chunk) sums grad * q over the (query, slot)
// pairs of the chunk from the inverse index; 16-byte pieces across lanes, pairs across lane groups.
__global__ void __launch_bounds__(256)
topk_bwd_dlmk_kernel(const bf16_t* __restrict__ gs, const bf16_t* __restrict__ q,
                     const int* __restrict__ offsets, const uint32_t* __restrict__ pairs,
                     float* __restrict__ dlmk, int L, int N, int h_kv, int G, int D, int topk,
                     int per_qhead, float sm_scale) {
  __shared__ float red[256 * 8];
  const int c = blockIdx.x, lh = blockIdx.y;  // chunk-key head
  const long b = blockIdx.z;
  const int lmk_h = per_qhead ? h_kv * G : h_kv;
  const int hk = per_qhead ? lh / G : lh;
  const int g_lo = per_qhead ? lh % G : 0, g_n = per_qhead ? 1 : G;
  const long cell = (b * h_kv + hk) * (long)N + c;
  const int p_lo = offsets[cell], p_hi = offsets[cell + 1];
  const int pieces = D / 8;
  const int pc = threadIdx.x % pieces, grp = threadIdx.x / pieces, ngrp = 256 / pieces;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  const long n_items = (long)(p_hi - p_lo) * g_n;
  // four items per round: their pair entries, then their gradient and query loads, are in flight
  // together (an item past the end re-reads the round's first item and counts for nothing)
  constexpr int U = 4;
  typedef unsigned tk_u32x4 __attribute__((ext_vector_type(4)));
  for (long it = grp; it < n_items; it += (long)ngrp * U) {
    uint32_t pk[U];
    long itu[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const long i2 = it + (long)u * ngrp;
      itu[u] = i2 < n_items ? i2 : it;
      pk[u] = pairs[p_lo + itu[u] / g_n];
    }
    bf16_t gr[U];
    tk_u32x4 qx[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int g = g_lo + (int)(itu[u] % g_n);
      const long rg = (((b * L + (pk[u] >> 8)) * h_kv + hk) * (long)G + g);
      gr[u] = gs[rg * topk + (pk[u] & 255)];
      qx[u] = *(const tk_u32x4*)(q + rg * D + pc * 8);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float gv = (it + (long)u * ngrp < n_items) ? bf2f(gr[u]) * sm_scale : 0.f;
      float f[8];
      unpack8(make_uint4(qx[u].x, qx[u].y, qx[u].z, qx[u].w), f);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = fmaf(gv, f[e], acc[e]);
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red[(grp * pieces + pc) * 8 + e] = acc[e];
  __syncthreads();
  for (int i = threadIdx.x; i < D; i += 256) {
    const int p2 = i / 8, e = i % 8;
    float x = 0.f;
    for (int g2 = 0; g2 < ngrp; ++g2) x += red[(g2 * pieces + p2) * 8 + e];
    if (p_hi > p_lo) dlmk[((b * N + c) * (long)lmk_h + lh) * D + i] += x;
  }
}

// ---- backward as two small dense products per query block ----
// The gradient of the gathered scores is a sparse (rows x chunks) matrix A with topk entries per
// row: dq = sm_scale * A LMK and dlmk = sm_scale * A^T Q.  A workgroup owns TD_R consecutive rows
// (queries x the heads that share the chunk keys) of one (batch, chunk-key head), scatters their
// gradients into a dense bf16 tile of A in LDS (128 chunks at a time), and runs both products on
// 16x16x32 MFMAs with the chunk keys and the query rows staged transposed beside it: no inverse
// index, every input read once and coalesced.  dlmk tiles of the query blocks are added with
// float atomics (the summation order over query blocks is not fixed).  The chunk indices of one
// row must be distinct (they are when they come from the selection).
#define TD_R 128        // rows per workgroup
#define TD_NC 128       // chunks per tile (== TD_R: one thread-to-piece split serves rows and chunk keys)
#define TD_THREADS 512
#define TD_STRIDE 136   // elements per LDS row: 128 + 8, so that 16-byte operand reads of 16 rows hit 64 banks

template <int D>
__global__ void __launch_bounds__(TD_THREADS)
topk_bwd_dense_kernel(const bf16_t* __restrict__ gs, const bf16_t* __restrict__ q,
                      const bf16_t* __restrict__ lmks, const int32_t* __restrict__ indices,
                      bf16_t* __restrict__ dq, float* __restrict__ dlmk, int L, int N, int h_kv, int G,
                      int topk, int per_qhead, float sm_scale) {
  constexpr int DT = D / 16, PPR = D / 8;
  extern __shared__ __align__(16) bf16_t td_sm[];
  bf16_t* A_s = td_sm;                        // [TD_R][TD_STRIDE]   A, row-major
  bf16_t* At_s = A_s + TD_R * TD_STRIDE;      // [TD_NC][TD_STRIDE]  A transposed
  bf16_t* Lt_s = At_s + TD_NC * TD_STRIDE;    // [D][TD_STRIDE]      chunk keys of the tile, feature-major
  bf16_t* Qt_s = Lt_s + D * TD_STRIDE;        // [D][TD_STRIDE]      query rows, feature-major
  __shared__ int cmax_s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, j = lane >> 4;
  // grid order (chunk-key head, batch) fastest, query block slowest: the workgroups in flight at
  // one time add their dlmk tiles to different (batch, head) slices instead of all to the same one
  const int lh = blockIdx.x;  // chunk-key head
  const long b = blockIdx.y;
  const int lmk_h = per_qhead ? h_kv * G : h_kv;
  const int hk = per_qhead ? lh / G : lh;
  const int g_lo = per_qhead ? lh % G : 0, g_n = per_qhead ? 1 : G;
  const int TQ = TD_R / g_n;
  const int t0 = blockIdx.z * TQ;
  auto row_rg = [&](int row) -> long {  // row of gs / q / dq of a block row (valid rows only)
    return ((b * L + t0 + row / g_n) * h_kv + hk) * (long)G + g_lo + row % g_n;
  };
  if (tid == 0) cmax_s = -1;
  // Every global load of the first tile is issued before anything waits (clamped addresses, no
  // branches around the loads): query pieces, chunk-key pieces, and the first NI (row, slot)
  // entries of every thread with their gradients.
  constexpr int NP = TD_R * PPR / TD_THREADS;  // 16-byte pieces per thread (rows and chunk keys alike)
  constexpr int NI = 8;                        // (row, slot) entries per thread and batch
  const int n_item = TD_R * topk;              // entries of the block, row-major like gs
  uint4 qx[NP], lx[NP];
#pragma unroll
  for (int u = 0; u < NP; ++u) {
    const int i = tid + u * TD_THREADS;
    const int row = i / PPR, pc = i % PPR;     // the pieces of a row sit in neighbouring lanes
    const int rc = (t0 + row / g_n < L) ? row : 0;  // row 0 of a block always exists
    qx[u] = *(const uint4*)(q + row_rg(rc) * D + pc * 8);
    const int cc = row < N ? row : N - 1;      // TD_NC == TD_R: the same split serves the chunk keys
    lx[u] = *(const uint4*)(lmks + ((b * N + cc) * (long)lmk_h + lh) * D + pc * 8);
  }
  auto item_load = [&](int i, int& c, bf16_t& val) {  // entry i of the block (any i: clamped)
    const int ic = i < n_item ? i : 0;
    const int row = ic / topk, slot = ic - row * topk;
    const bool ok = i < n_item && t0 + row / g_n < L;
    const int rc = ok ? row : 0;
    c = indices[((b * L + t0 + rc / g_n) * h_kv + hk) * (long)topk + slot];
    val = gs[row_rg(rc) * topk + slot];
    if (!ok || c >= N) c = -1;
  };
  int ci[NI];
  bf16_t gv[NI];
#pragma unroll
  for (int u = 0; u < NI; ++u) item_load(tid + u * TD_THREADS, ci[u], gv[u]);
#pragma unroll
  for (int u = 0; u < NP; ++u) {
    const int i = tid + u * TD_THREADS;
    const int row = i / PPR, pc = i % PPR;
    const bool ok = t0 + row / g_n < L;
    const bf16_t* xs = (const bf16_t*)&qx[u];
#pragma unroll
    for (int e = 0; e < 8; ++e) Qt_s[(pc * 8 + e) * TD_STRIDE + row] = ok ? xs[e] : (bf16_t)0;
  }
  f32x4_t acc_q[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) acc_q[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  int cmax = 0;
  for (int c0 = 0; c0 <= cmax; c0 += TD_NC) {
    // clear both copies of A (the rows of At beyond the tile's chunks stay zero)
    for (int i = tid; i < (TD_R + TD_NC) * TD_STRIDE / 8; i += TD_THREADS) ((uint4*)A_s)[i] = make_uint4(0, 0, 0, 0);
    // chunk keys of the tile, feature-major
#pragma unroll
    for (int u = 0; u < NP; ++u) {
      const int i = tid + u * TD_THREADS;
      const int cl = i / PPR, pc = i % PPR;
      if (c0 > 0) {
        const int cc = c0 + cl < N ? c0 + cl : N - 1;
        lx[u] = *(const uint4*)(lmks + ((b * N + cc) * (long)lmk_h + lh) * D + pc * 8);
      }
      const bool ok = c0 + cl < N;
      const bf16_t* xs = (const bf16_t*)&lx[u];
#pragma unroll
      for (int e = 0; e < 8; ++e) Lt_s[(pc * 8 + e) * TD_STRIDE + cl] = ok ? xs[e] : (bf16_t)0;
    }
    __syncthreads();
    int my_max = -1;
    for (int i0 = 0; i0 < n_item; i0 += NI * TD_THREADS) {
      if (i0 > 0 || c0 > 0) {
#pragma unroll
        for (int u = 0; u < NI; ++u) item_load(i0 + tid + u * TD_THREADS, ci[u], gv[u]);
      }
#pragma unroll
      for (int u = 0; u < NI; ++u) {
        const int c = ci[u];
        my_max = c > my_max ? c : my_max;
        if (c >= c0 && c < c0 + TD_NC) {
          const int row = (i0 + tid + u * TD_THREADS) / topk;
          A_s[row * TD_STRIDE + (c - c0)] = gv[u];
          At_s[(c - c0) * TD_STRIDE + row] = gv[u];
        }
      }
    }
    if (c0 == 0) {  // largest chunk index of the block: how many tiles there are
#pragma unroll
      for (int o2 = 32; o2 >= 1; o2 >>= 1) {
        const int y = __shfl_xor(my_max, o2, 64);
        my_max = y > my_max ? y : my_max;
      }
      if (lane == 0 && my_max >= 0) atomicMax(&cmax_s, my_max);
    }
    __syncthreads();
    cmax = cmax_s;
    if (cmax >= c0) {  // (the first tile of a block with no valid entry has nothing to add)
      // dq rows of this wavefront's row tile += A LMK
#pragma unroll
      for (int kc = 0; kc < TD_NC / 32; ++kc) {
        const uint4 a = *(const uint4*)(A_s + (wave * 16 + col) * TD_STRIDE + kc * 32 + j * 8);
#pragma unroll
        for (int t = 0; t < DT; ++t) {
          const uint4 bb = *(const uint4*)(Lt_s + (t * 16 + col) * TD_STRIDE + kc * 32 + j * 8);
          acc_q[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&a, *(const bf16x8_t*)&bb, acc_q[t], 0, 0, 0);
        }
      }
      // dlmk of this wavefront's chunk tile = A^T Q
      const int c_tile = c0 + wave * 16;
      if (c_tile <= cmax) {
        f32x4_t acc_l[DT];
#pragma unroll
        for (int t = 0; t < DT; ++t) acc_l[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kr = 0; kr < TD_R / 32; ++kr) {
          const uint4 a = *(const uint4*)(At_s + (wave * 16 + col) * TD_STRIDE + kr * 32 + j * 8);
#pragma unroll
          for (int t = 0; t < DT; ++t) {
            const uint4 bb = *(const uint4*)(Qt_s + (t * 16 + col) * TD_STRIDE + kr * 32 + j * 8);
            acc_l[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&a, *(const bf16x8_t*)&bb, acc_l[t], 0, 0, 0);
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int c = c_tile + 4 * j + i;
          if (c < N) {
            float* dst = dlmk + ((b * N + c) * (long)lmk_h + lh) * D + col;
#pragma unroll
            for (int t = 0; t < DT; ++t) {
              const float v = acc_l[t][i] * sm_scale;
              if (v != 0.f) unsafeAtomicAdd(dst + t * 16, v);
            }
          }
        }
      }
    }
    __syncthreads();  // the tile is no longer read
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = wave * 16 + 4 * j + i;
    if (t0 + row / g_n < L) {
      bf16_t* dst = dq + row_rg(row) * D + col;
#pragma unroll
      for (int t = 0; t < DT; ++t) dst[t * 16] = f2bf(acc_q[t][i] * sm_scale);
    }
  }
}

static bool topk_bwd_dense_covers(int G, int D, int per_qhead) {
  const int g_n = per_qhead ? 1 : G;
  return (D == 64 || D == 128) && g_n >= 1 && g_n <= TD_R && TD_R % g_n == 0;
}

template <int D>
static int topk_bwd_dense_launch(dim3 grid, hipStream_t st, const bf16_t* gs, const bf16_t* q, const bf16_t* lmks,
                                 const int32_t* indices, bf16_t* dq, float* dlmk, int L, int N, int h_kv, int G,
                                 int topk, int per_qhead, float sm_scale) {
  const size_t smem = (size_t)(TD_R + TD_NC + 2 * D) * TD_STRIDE * sizeof(bf16_t);
  auto kern = topk_bwd_dense_kernel<D>;
  static HilsLdsReserve reserved;  // per instantiation
  if (int rc = hils_reserve_lds(&reserved, (const void*)kern, smem, "hils_topk_bwd")) return rc;
  hipLaunchKernelGGL(kern, grid, dim3(TD_THREADS), smem, st, gs, q, lmks, indices, dq, dlmk, L, N, h_kv, G, topk,
                     per_qhead, sm_scale);
  return HILS_OK;
}

void hils_build_chunk_index(const int32_t* indices, int* counts, int* offsets, int* cursor, uint32_t* pairs,
                            int B, int L, int H, int K, int nchunk, void* stream);

static size_t topk_bwd_round(size_t n) { return (n + 255) & ~(size_t)255; }

extern "C" size_t hils_topk_bwd_workspace(int B, int L, int N, int h_kv, int G, int D, int topk) {
  if (D % 8 != 0 || D > 2048 || topk > 256 || N > 12288 || L >= (1 << 24)) return 0;
  if (topk_bwd_dense_covers(G, D, 0)) return 0;  // the dense kernel needs no scratch (and covers per-head keys too)
  const size_t cells = (size_t)B * h_kv * N;
  return 3 * topk_bwd_round((cells + 1) * 4) + topk_bwd_round((size_t)B * L * h_kv * topk * 4);
}

extern "C" int hils_topk_bwd(const void* g_scores, const void* q, const void* lmks,
                             const int32_t* indices, void* dq, float* dlmk, void* workspace,
                             size_t workspace_bytes, int B, int L, int N, int h_kv, int G, int D, int topk,
                             int per_qhead, float sm_scale, void* stream) {
  HILS_REQUIRE(g_scores && q && lmks && indices && dq && dlmk, "hils_topk_bwd: null pointer");
  HILS_REQUIRE(!workspace || workspace_bytes >= hils_topk_bwd_workspace(B, L, N, h_kv, G, D, topk),
               "hils_topk_bwd: workspace of %zu bytes is shorter than the %zu bytes hils_topk_bwd_workspace "
               "returns for this shape", workspace_bytes, hils_topk_bwd_workspace(B, L, N, h_kv, G, D, topk));
  HILS_REQUIRE(B > 0 && L > 0 && N > 0 && h_kv > 0 && G > 0 && D > 0 && topk > 0, "hils_topk_bwd: sizes must be positive");
  const long rows = (long)B * L * h_kv;
  HILS_REQUIRE(rows <= 2147483647L, "hils_topk_bwd: grid too large");
  hipStream_t st = (hipStream_t)stream;
  if (topk_bwd_dense_covers(G, D, per_qhead) && B <= 65535 &&
      (L + TD_R / (per_qhead ? 1 : G) - 1) / (TD_R / (per_qhead ? 1 : G)) <= 65535) {
    const int g_n = per_qhead ? 1 : G, TQ = TD_R / g_n;
    const int lmk_h = per_qhead ? h_kv * G : h_kv;
    dim3 grid(lmk_h, B, (unsigned)((L + TQ - 1) / TQ));
    int rc;
    if (D == 64)
      rc = topk_bwd_dense_launch<64>(grid, st, (const bf16_t*)g_scores, (const bf16_t*)q, (const bf16_t*)lmks, indices,
                                     (bf16_t*)dq, dlmk, L, N, h_kv, G, topk, per_qhead, sm_scale);
    else
      rc = topk_bwd_dense_launch<128>(grid, st, (const bf16_t*)g_scores, (const bf16_t*)q, (const bf16_t*)lmks, indices,
                                      (bf16_t*)dq, dlmk, L, N, h_kv, G, topk, per_qhead, sm_scale);
    if (rc) return rc;
    HILS_CHECK_LAUNCH("hils_topk_bwd");
    return HILS_OK;
  }
  if (workspace && hils_topk_bwd_workspace(B, L, N, h_kv, G, D, topk) > 0 && h_kv * G <= 65535 && B <= 65535) {
    const size_t cells = (size_t)B * h_kv * N;
    char* ws = (char*)workspace;
    int* counts = (int*)ws;
    int* offsets = (int*)(ws + topk_bwd_round((cells + 1) * 4));
    int* cursor = (int*)(ws + 2 * topk_bwd_round((cells + 1) * 4));
    uint32_t* pairs = (uint32_t*)(ws + 3 * topk_bwd_round((cells + 1) * 4));
    const long rows_g = rows * G;
    const long items = rows_g * (D / 8);
    hipLaunchKernelGGL(topk_bwd_dq_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, st,
                       (const bf16_t*)g_scores, (const bf16_t*)lmks, indices, (bf16_t*)dq, rows_g, L, N, h_kv,
                       G, D, topk, per_qhead, sm_scale);
    hils_build_chunk_index(indices, counts, offsets, cursor, pairs, B, L, h_kv, topk, N, stream);
    const int lmk_h = per_qhead ? h_kv * G : h_kv;
    hipLaunchKernelGGL(topk_bwd_dlmk_kernel, dim3(N, lmk_h, B), dim3(256), 0, st, (const bf16_t*)g_scores,
                       (const bf16_t*)q, offsets, pairs, dlmk, L, N, h_kv, G, D, topk, per_qhead, sm_scale);
    HILS_CHECK_LAUNCH("hils_topk_bwd");
    return HILS_OK;
  }
  const int threads = D >= 128 ? 128 : 64;
  size_t smem = ((size_t)G * topk + topk) * sizeof(float);
  hipLaunchKernelGGL(topk_bwd_kernel, dim3((unsigned)rows), dim3(threads), smem, st,
                     (const bf16_t*)g_scores, (const bf16_t*)q, (const bf16_t*)lmks, indices,
                     (bf16_t*)dq, dlmk, L, N, h_kv, G, D, topk, per_qhead, sm_scale);
  HILS_CHECK_LAUNCH("hils_topk_bwd");
  return HILS_OK;
}
