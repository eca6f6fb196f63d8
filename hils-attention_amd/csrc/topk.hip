// Query -> chunk-key scoring with per-(query, KV head) top-k selection.
//
// One workgroup (4 wavefronts) owns 16 consecutive queries of one (batch, KV head).
// The logits of a 16-query x 16-chunk tile come from one chain of 16x16x32 bf16 MFMAs
// per query head g (A = the 16 query rows of head g, B = 16 chunk keys).  Two passes
// over the visible chunks: pass 1 keeps an online log-sum-exp per (query, g); pass 2
// recomputes the logits, forms max_g(logit - lse_total), parks the pooled scores of a
// segment of chunks in LDS and lets one wavefront per query pick the top-k with a
// bitwise threshold search on order-preserving integer keys.  Ties: lower index wins.
#include "decode_rows.h"
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

// One wavefront selects the top-K of (previous candidates) U (segment scores).
// cand_* hold the previous winners in ascending index order (ncand of them, all with
// an index below seg_base); seg holds ns pooled scores of chunks seg_base..seg_base+ns-1.
// With KEYS the segment already holds order-preserving keys instead of floats.
// With seg_idx the chunk index of seg[i] is seg_idx[i] (ascending in i) instead of seg_base + i.
// The winners are written back to cand_* in ascending index order; returns the count.
// The K-th largest key is found bit by bit; the bits all valid keys share are skipped, and
// every count is a per-lane tally plus one DPP reduction (no scalar dependency per slot).
template <bool KEYS = false>
__device__ int wave_select(const float* seg, int ns, int seg_base, float* cand_s, int* cand_i,
                           int ncand, int K, const int* seg_idx = nullptr) {
  const int lane = threadIdx.x & 63;
  uint32_t key[TOPK_SLOTS + 1];
  int cidx = -1;
  key[0] = 0u;
  if (lane < ncand) {
    key[0] = score_key(cand_s[lane]);
    cidx = cand_i[lane];
  }
#pragma unroll
  for (int s = 0; s < TOPK_SLOTS; ++s) {
    const int i = s * 64 + lane;
    key[s + 1] = (i < ns) ? (KEYS ? ((const uint32_t*)seg)[i] : score_key(seg[i])) : 0u;
  }
  const int nslot = (ns + 63) / 64 + 1;
  int tl = 0;
  uint32_t ka = 0xffffffffu, ko = 0u;
#pragma unroll
  for (int s = 0; s <= TOPK_SLOTS; ++s)
    if (key[s] != 0u) { ++tl; ka &= key[s]; ko |= key[s]; }
  const int total = wave_sum_i(tl);
  uint32_t T = 1u;  // every valid key is >= 1
  if (total > K) {
    ka = wave_and_u(ka);
    ko = wave_or_u(ko);
    const uint32_t diff = ka ^ ko;  // bits in which the valid keys differ
    if (diff == 0u) {
      T = ka;
    } else {
      const int top = 31 - __clz((int)diff);
      T = (top == 31) ? 0u : (ka & ~((2u << top) - 1u));  // the shared leading bits
      for (int bit = top; bit >= 0; --bit) {
        const uint32_t c = T | (1u << bit);
        int cl = 0;  // keys of unused slots are 0 and never count
#pragma unroll
        for (int s = 0; s <= TOPK_SLOTS; ++s) cl += (key[s] >= c) ? 1 : 0;
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
  for (int s = 0; s <= TOPK_SLOTS; ++s) gl += (key[s] > T) ? 1 : 0;
  const int gt = wave_sum_i(gl);
  int need = K - gt;  // ties with the threshold still to take, lowest index first
  int pos = 0;
  const unsigned long long lt = (1ull << lane) - 1ull;
#pragma unroll
  for (int s = 0; s <= TOPK_SLOTS; ++s) {
    if (s < nslot) {
      const unsigned long long eq = __ballot(key[s] == T && key[s] != 0u);
      const bool take_eq = (key[s] == T && key[s] != 0u) && (__popcll(eq & lt) < need);
      const bool sel = (key[s] > T) || take_eq;
      const unsigned long long sm = __ballot(sel);
      if (sel) {
        const int o = pos + __popcll(sm & lt);
        cand_s[o] = key_score(key[s]);
        cand_i[o] = (s == 0) ? cidx
                             : (seg_idx ? seg_idx[(s - 1) * 64 + lane] : seg_base + (s - 1) * 64 + lane);
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

  // ---------------- register path: G <= 4 and at most 512 visible chunks ----------------
  // One MFMA pass: wavefront w takes chunk blocks w, w+4, ... (at most 8), the query tile
  // is read from LDS as the A operand, and the 16x16 logit tiles of all G heads stay in
  // registers until the pooled score max_g(logit - lse_total) is written.
  bool use_reg = false;
  if constexpr (GMAX <= 4) {
    use_reg = nblk <= 32;
    if (use_reg) {
      constexpr int QROW = D + 8;  // padded row (bf16 elements) of the staged query tile
      __shared__ bf16_t q_lds[TOPK_QT * GMAX * QROW];
      for (int i = tid; i < TOPK_QT * G * (D / 8); i += TOPK_THREADS) {
        const int rowi = i / (D / 8), d8 = i - rowi * (D / 8);
        const int qi = rowi / G, g = rowi - qi * G;
        const int tq = t0 + qi;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (tq < L) v = *(const uint4*)(q + (((b * L + tq) * h_kv + hk) * (long)G + g) * D + d8 * 8);
        *(uint4*)(q_lds + (qi * GMAX + g) * QROW + d8 * 8) = v;
      }
      if (tid < TOPK_QT) ncand_s[tid] = 0;
      __syncthreads();
      auto load_b = [&](int blk, int g, uint4* dst) {
        const int c = blk * 16 + col;
        const int lh = per_qhead ? hk * G + g : hk;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          dst[ks] = make_uint4(0, 0, 0, 0);
          if (c < N) dst[ks] = *(const uint4*)(lmks + ((b * N + c) * (long)lmk_h + lh) * D + ks * 32 + grp * 8);
        }
      };
      float xs[8][GMAX][4];
      float m4[GMAX][4];
#pragma unroll
      for (int g = 0; g < GMAX; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) m4[g][i] = HILS_NEG_INF;
      uint4 bcur[KS], bnext[KS];
      if (!per_qhead && wave < nblk) load_b(wave, 0, bcur);
#pragma unroll
      for (int bi = 0; bi < 8; ++bi) {
        const int blk = wave + bi * 4;
        if (blk >= nblk) break;
        if (!per_qhead && blk + 4 < nblk) load_b(blk + 4, 0, bnext);
        const int c = blk * 16 + col;
        const bool cvalid = c < N;
#pragma unroll
        for (int g = 0; g < GMAX; ++g) {
          if (g < G) {
            if (per_qhead) load_b(blk, g, bcur);
            f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
              const uint4 av = *(const uint4*)(q_lds + (col * GMAX + g) * QROW + ks * 32 + grp * 8);
              acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&av, *(bf16x8_t*)&bcur[ks], acc, 0, 0, 0);
            }
            float add = 0.f, gum = 0.f;
            if (cvalid && bias) add = bias[((b * N + c) * (long)h_kv + hk) * G + g];
            if (cvalid && gumbel) gum = gumbel[(long)(hk * G + g) * N + c];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              float x = __fmul_rn(acc[i], sm_scale);
              if (bias) x = __fadd_rn(x, add);
              if (gumbel) x = __fadd_rn(x, gum);
              if (!(cvalid && c < lim[i])) x = HILS_NEG_INF;
              xs[bi][g][i] = x;
              m4[g][i] = fmaxf(m4[g][i], x);
            }
          }
        }
        if (!per_qhead) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) bcur[ks] = bnext[ks];
        }
      }
      // log-sum-exp per (query, g): this lane's blocks, the 16 columns of the lane group
      // (one DPP row), then the 4 wavefronts through LDS
#pragma unroll
      for (int g = 0; g < GMAX; ++g) {
        if (g < G) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float m = m4[g][i];
            m = fmaxf(m, __shfl_xor(m, 1, 64));
            m = fmaxf(m, __shfl_xor(m, 2, 64));
            m = fmaxf(m, __shfl_xor(m, 4, 64));
            m = fmaxf(m, __shfl_xor(m, 8, 64));
            float l = 0.f;
            if (m > HILS_NEG_INF) {
#pragma unroll
              for (int bi = 0; bi < 8; ++bi)
                if (wave + bi * 4 < nblk) l += __expf(xs[bi][g][i] - m);
            }
            l = row_sum<16>(l);
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
      __syncthreads();
#pragma unroll
      for (int bi = 0; bi < 8; ++bi) {
        const int blk = wave + bi * 4;
        if (blk >= nblk) break;
        const int c = blk * 16 + col;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int tq = t0 + grp * 4 + i;
          float best = HILS_NEG_INF;
#pragma unroll
          for (int g = 0; g < GMAX; ++g) {
            if (g < G) {
              const float x = xs[bi][g][i];
              if (sel_logits_out && c < N && tq < L)
                sel_logits_out[(((b * L + tq) * (long)h_kv + hk) * G + g) * N + c] = x;
              const float nrm = (x == HILS_NEG_INF) ? HILS_NEG_INF : __fsub_rn(x, lse_tot[g][grp * 4 + i]);
              best = fmaxf(best, nrm);
            }
          }
          if (drop_mask && best > HILS_NEG_INF && tq < L && c < N &&
              drop_mask[(b * L + tq) * (long)N + c] != 0)
            best = HILS_NEG_INF;
          pooled[grp * 4 + i][c] = best;
        }
      }
      __syncthreads();
      const int ns = nblk * 16;
      for (int qi = wave; qi < TOPK_QT; qi += 4) {
        if (t0 + qi < L) {
          const int nc = wave_select(pooled[qi], ns, 0, cand_s[qi], cand_i[qi], 0, topk);
          if (lane == 0) ncand_s[qi] = nc;
        }
      }
      __syncthreads();
    }
  }
  if (!use_reg) {
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

static bool topk_use_split(int B, int L, int N, int h_kv) {
  static int cus = 0;  // looked up once (keeps the query out of HIP graph capture)
  if (cus == 0) {
    int dev = 0, v = 0;
    cus = 256;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      cus = v;
  }
  const long fused_wgs = (long)B * ((L + TOPK_QT - 1) / TOPK_QT) * h_kv;
  return fused_wgs < 2L * cus && N >= 256 && N <= 16384;
}

extern "C" size_t hils_topk_fwd_workspace(int B, int L, int N, int h_kv, int G) {
  if (!topk_use_split(B, L, N, h_kv)) return 0;
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
    if (smem > 64 * 1024) {
      static bool reserved = false;
      if (!reserved) {
        (void)hipFuncSetAttribute((const void*)topk_select_kernel,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024 + 4096);
        reserved = true;
      }
    }
    hipLaunchKernelGGL(topk_select_kernel, dim3((unsigned)rows), dim3(TOPK_B_THREADS), smem, st, raw,
                       lse_swa, bias, gumbel, drop_mask, indices, (bf16_t*)scores, lse_total,
                       sel_logits, L, N, h_kv, G, topk, block_size, window_size, causal, q_offset);
  }
#undef TOPK_B_REG
  return HILS_OK;
}

extern "C" int hils_topk_fwd(const void* q, const void* lmks, const float* lse_swa,
                             const float* bias, const float* gumbel, const int32_t* drop_mask,
                             int32_t* indices, void* scores, float* lse_total, float* sel_logits,
                             void* workspace, int B, int L, int N, int h_kv, int G, int D, int topk,
                             int block_size, int window_size, int causal, int q_offset,
                             int per_qhead, float sm_scale, void* stream) {
  HILS_REQUIRE(q && lmks && lse_swa && indices && scores, "hils_topk_fwd: null pointer");
  HILS_REQUIRE(B > 0 && L > 0 && N > 0 && h_kv > 0 && G > 0 && D > 0, "hils_topk_fwd: sizes must be positive");
  HILS_REQUIRE(topk >= 1 && topk <= TOPK_MAXK, "hils_topk_fwd: topk (%d) must be in 1..%d", topk, TOPK_MAXK);
  HILS_REQUIRE(G <= 16, "hils_topk_fwd: group size %d not supported (max 16)", G);
  HILS_REQUIRE(block_size > 0, "hils_topk_fwd: block_size must be positive");
  HILS_REQUIRE(h_kv <= 65535 && B <= 65535, "hils_topk_fwd: h_kv/B too large for the grid");
  hipStream_t st = (hipStream_t)stream;
  if (workspace && (D == 64 || D == 128) && topk_use_split(B, L, N, h_kv) &&
      (long)B * L <= 2147483647L / h_kv) {
    if (int rc2 = topk_fwd_split(q, lmks, lse_swa, bias, gumbel, drop_mask, indices, scores, lse_total,
                                 sel_logits, (float*)workspace, B, L, N, h_kv, G, D, topk, block_size,
                                 window_size, causal, q_offset, per_qhead, sm_scale, st))
      return rc2;
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

extern "C" int hils_topk_bwd(const void* g_scores, const void* q, const void* lmks,
                             const int32_t* indices, void* dq, float* dlmk, int B, int L, int N,
                             int h_kv, int G, int D, int topk, int per_qhead, float sm_scale,
                             void* stream) {
  HILS_REQUIRE(g_scores && q && lmks && indices && dq && dlmk, "hils_topk_bwd: null pointer");
  HILS_REQUIRE(B > 0 && L > 0 && N > 0 && h_kv > 0 && G > 0 && D > 0 && topk > 0, "hils_topk_bwd: sizes must be positive");
  const long rows = (long)B * L * h_kv;
  HILS_REQUIRE(rows <= 2147483647L, "hils_topk_bwd: grid too large");
  const int threads = D >= 128 ? 128 : 64;
  size_t smem = ((size_t)G * topk + topk) * sizeof(float);
  hipLaunchKernelGGL(topk_bwd_kernel, dim3((unsigned)rows), dim3(threads), smem, (hipStream_t)stream,
                     (const bf16_t*)g_scores, (const bf16_t*)q, (const bf16_t*)lmks, indices,
                     (bf16_t*)dq, dlmk, L, N, h_kv, G, D, topk, per_qhead, sm_scale);
  HILS_CHECK_LAUNCH("hils_topk_bwd");
  return HILS_OK;
}
