// Decode sparse attention, row-streaming MFMA variant (D == Dv in {64, 128}, up to 16 query heads
// per KV head).
//
// The step is bound by reading K and V of the selected chunks once, so everything else is kept
// out of the memory pipeline's way:
//   * every K and V load is a fully coalesced 16-byte lane load (D/8 neighbouring lanes read one
//     2*D-byte token row).  A chunk is a stream of eight groups of 16 tokens (K0..K3, V0..V3) and
//     a wavefront keeps a ring of NR register groups: the group just consumed is re-issued for the
//     one NR places further down the stream, across chunk boundaries alike, so NR-1 groups
//     (4 KiB each at D = 128) per wavefront are always in flight;
//   * a consumed group is written row-major into the wavefront's own LDS staging area (rows padded
//     by 16 bytes, so that the row-wise writes and the column-wise operand reads are both free of
//     bank conflicts) and read back as MFMA operands: S^T = K q^T with the query heads in the 16
//     MFMA columns, O^T += V^T P with V^T read by the transposing LDS load;
//   * the per-chunk softmax runs on the 16 accumulator values a lane holds (token 4j+i of each
//     16-token tile, head = lane & 15), its two cross-row reductions on the row-swap instructions;
//     the chunk weight is folded into P, so the output accumulators are never rescaled.
// The arithmetic is a few hundred instructions per 32 KiB chunk; the wavefronts of a workgroup own
// slots (selected chunks) round-robin and their outputs are summed through LDS at the end.
#pragma once
#include <type_traits>
#include "common.h"
#include "../../include/hils_amd.h"

#define DR_S 64
#define DR_QT 16       // tokens per register group
#define DR_NR 8        // register groups in the ring
#define DR_MAXSLOT 32  // slots a wavefront can own
#define DR_NH 16       // MFMA columns = query heads per KV head the kernel can take

typedef unsigned dr_u4 __attribute__((ext_vector_type(4)));  // a 16-byte piece as a register value
typedef short dr_s4 __attribute__((ext_vector_type(4)));

struct DrDims {
  int L, Lkv, HQ, H, G, K, NW, nchunk, nsplit, mask_last;
  float sm_scale;
  // paged cache (page = chunk = 64 tokens): K and V are (num_pages, H, 64, D), the tokens of a
  // (page, head) contiguous, and chunk c of batch element b lives in page page_table[b][c]
  const int32_t* page_table;
  int max_pages, num_pages;
};

static inline size_t dr_smem_bytes(int D, int G, int nwave) {
  return (size_t)nwave * 32 * (2 * D + 16)             // staging areas: 32 padded token rows
         + (size_t)nwave * G * D * sizeof(float)       // partial outputs
         + (size_t)nwave * DR_MAXSLOT * (sizeof(long) + sizeof(int))  // slot lists
         + (size_t)nwave * DR_MAXSLOT * DR_NH * sizeof(bf16_t);       // slot weights
}

struct DrNoHook {
  __device__ __forceinline__ void operator()() const {}
};

// One (query, KV head) row by a workgroup of NWAVE wavefronts: `split` of dm.nsplit shares of the
// slots, KV head hk, query bt = b * L + t; dr_smem = dr_smem_bytes(D, G, NWAVE) bytes of LDS.
// weights and indices may point into LDS (the one-launch decode step hands the row's selection over
// there: generic loads reach either memory).  `hook` runs once in every wavefront after its first
// chunk's loads have been issued and before it writes the staging areas of dr_smem (that kernel puts
// the barrier there that ends the selection's use of the same LDS).
template <int D, int NWAVE, class Hook = DrNoHook>
__device__ __forceinline__ void decode_rows_body(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                                                 const bf16_t* __restrict__ v, const bf16_t* __restrict__ weights,
                                                 const int32_t* __restrict__ indices, bf16_t* __restrict__ o,
                                                 float* __restrict__ partial, const DrDims& dm, char* dr_smem,
                                                 int split, int hk, long bt, Hook hook = Hook{}) {
  constexpr int LR = D / 8;          // lanes per token row
  constexpr int TPI = 64 / LR;       // token rows per load instruction
  constexpr int GL = DR_QT / TPI;    // load instructions per group
  constexpr int KS = D / 32;         // k-steps of S^T = K q^T
  constexpr int MT = D / 16;         // 16-feature tiles of O^T
  constexpr int NR = DR_NR;
  constexpr int ROWB = 2 * D + 16;   // bytes of a staged token row
  constexpr int STAGE_B = 32 * ROWB;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, j = lane >> 4;
  const int piece = lane % LR, tsub = lane / LR;
  const long b = bt / dm.L;
  const int G = dm.G, K = dm.K;

  char* stage_w = dr_smem + (size_t)wave * STAGE_B;
  float* o_s = (float*)(dr_smem + (size_t)NWAVE * STAGE_B);  // [wave][G][D]
  long* sl_off_all = (long*)(o_s + (size_t)NWAVE * G * D);
  int* sl_id_all = (int*)(sl_off_all + NWAVE * DR_MAXSLOT);
  bf16_t* sl_w_all = (bf16_t*)(sl_id_all + NWAVE * DR_MAXSLOT);
  long* sl_off = sl_off_all + wave * DR_MAXSLOT;
  int* sl_id = sl_id_all + wave * DR_MAXSLOT;
  bf16_t* sl_w = sl_w_all + (size_t)wave * DR_MAXSLOT * DR_NH;

  // query heads as the B operand of S^T = K q^T: lane (head = col, j) holds features ks*32 + j*8 ..
  bf16x8_t qb[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    dr_u4 t = {0u, 0u, 0u, 0u};
    if (col < G) t = *(const dr_u4*)(q + (bt * dm.HQ + hk * G + col) * (long)D + ks * 32 + j * 8);
    qb[ks] = __builtin_bit_cast(bf16x8_t, t);
  }
  const float c2 = dm.sm_scale * HILS_LOG2E;

  // ---- this wavefront's slots (s_begin + wave, + NWAVE, ...): lane i looks at the i-th of them, the
  // ones that hold a mapped chunk are compacted in order (byte offset of the chunk's first row and
  // i go to LDS).  The heads' weights of all of them are loaded alongside the indices, so the
  // stream below starts one memory latency after the kernel ----
  const int per_split = (K + dm.nsplit - 1) / dm.nsplit;
  const int s_begin = split * per_split;
  const int s_end = (s_begin + per_split < K) ? s_begin + per_split : K;
  const int nmine = (s_end - s_begin - wave + NWAVE - 1) / NWAVE;  // slots of this wavefront (may be <= 0)
  int nsl;
  {
    bf16_t wv[DR_MAXSLOT / 4];
#pragma unroll
    for (int p4 = 0; p4 < DR_MAXSLOT / 4; ++p4) {
      wv[p4] = 0;
      if (p4 * 4 < nmine) {  // uniform
        const int i = p4 * 4 + j;
        if (i < nmine && col < G)
          wv[p4] = weights[(bt * dm.HQ + hk * G + col) * (long)dm.NW + s_begin + wave + i * NWAVE];
      }
    }
    const int slot = s_begin + wave + lane * NWAVE;
    bool ok = lane < DR_MAXSLOT && slot < s_end;
    int c = -1;
    if (ok) c = indices[(bt * dm.H + hk) * (long)K + slot];
    ok = ok && c >= 0 && c < dm.nchunk;
    long row0;
    if (dm.page_table) {
      int pg = -1;
      if (ok) pg = dm.page_table[b * dm.max_pages + c];
      ok = ok && pg >= 0 && pg < dm.num_pages;  // an unmapped chunk contributes nothing
      row0 = ((long)pg * dm.H + hk) * DR_S;
    } else {
      row0 = (b * dm.Lkv + (long)c * DR_S) * dm.H + hk;
    }
    const unsigned long long m = __ballot(ok);
    const int pos = __popcll(m & ((1ull << lane) - 1ull));
    nsl = __popcll(m);
    if (ok) {
      sl_off[pos] = row0 * D * 2;  // bytes
      sl_id[pos] = lane;
    }
#pragma unroll
    for (int p4 = 0; p4 < DR_MAXSLOT / 4; ++p4)
      if (p4 * 4 < nmine) sl_w[(p4 * 4 + j) * DR_NH + col] = wv[p4];
  }
  __builtin_amdgcn_wave_barrier();

  // Addresses are a wavefront-uniform 64-bit base (tensor + chunk + group + load number, scalar
  // registers) plus one 32-bit byte offset per lane: no per-load vector address arithmetic.
  const unsigned step_b = (dm.page_table ? (unsigned)D : (unsigned)dm.H * D) * 2u;  // bytes between token rows
  const unsigned lane_b = (unsigned)tsub * step_b + (unsigned)piece * 16u;
  const char* kb = (const char*)k;
  const char* vb = (const char*)v;
  auto chunk_off = [&](int si) __attribute__((always_inline)) -> long {  // byte offset of the chunk's first row
    const long x = sl_off[si];
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)x);
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(x >> 32));
    return (long)(((unsigned long)hi << 32) | lo);
  };
  // stream group s of a chunk: s < 4 tokens 16s.. of K, else tokens 16(s-4).. of V
  auto issue = [&](dr_u4 (&dst)[GL], long coff, int s) __attribute__((always_inline)) {
    const char* base = (s < 4 ? kb : vb) + coff + (size_t)((s & 3) * DR_QT) * step_b;
#pragma unroll
    for (int i = 0; i < GL; ++i) dst[i] = *(const dr_u4*)(base + (size_t)(i * TPI) * step_b + lane_b);
  };
  // per-lane LDS addresses: everything else is an immediate offset
  char* const w_addr = stage_w + tsub * ROWB + piece * 16;                          // row-wise write of a load
  const char* const k_addr = stage_w + col * ROWB + j * 16;                         // K tile as A operand
  const char* const t_addr = stage_w + (4 * j + (col >> 2)) * ROWB + (col & 3) * 8; // transposing read of V
  auto stage = [&](const dr_u4 (&src)[GL], int row0) __attribute__((always_inline)) {
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < GL; ++i) *(dr_u4*)(w_addr + (row0 + i * TPI) * ROWB) = src[i];
    __builtin_amdgcn_wave_barrier();
  };

  f32x4_t S[4], O[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) O[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  bf16x8_t pb[2];  // P of the chunk as B operands: tokens 0..31 and 32..63

  // K group t (tokens 16t ..): one 16-token tile of S^T
  auto consume_k = [&](const dr_u4 (&src)[GL], int t) __attribute__((always_inline)) {
    stage(src, 0);
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const dr_u4 a = *(const dr_u4*)(k_addr + ks * 64);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), qb[ks], acc, 0, 0, 0);
    }
    S[t] = acc;
  };
  // V group t: staged beside its neighbour; after the second of a pair,
  // O^T[feature][head] += V^T[feature][token] P[token][head] over the pair's 32 tokens.  A lane's
  // eight k-slots are tokens 4j..4j+3 of the first and of the second 16-token tile, the order in
  // which the S^T accumulators hold them; the transposing LDS load delivers V^T in that order
  // (a 16-lane group addresses a 4 x 16 block, lane l row l/4 and columns 4(l%4).., and receives
  // column l of it).
  auto consume_v = [&](const dr_u4 (&src)[GL], int t) __attribute__((always_inline)) {
    stage(src, (t & 1) * 16);
    if (!(t & 1)) return;
    typedef short dr_s8 __attribute__((ext_vector_type(8)));
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const dr_s4 a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) dr_s4*)(t_addr + mt * 32));
      const dr_s4 a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) dr_s4*)(t_addr + mt * 32 + 16 * ROWB));
      const dr_s8 a = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
      O[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), pb[t >> 1], O[mt], 0, 0, 0);
    }
  };
  // softmax over the chunk's 64 tokens per head, the chunk weight folded in
  auto softmax = [&](int si) __attribute__((always_inline)) {
    if (dm.mask_last && j == 3) S[3][3] = HILS_NEG_INF;
    float mx = HILS_NEG_INF;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) mx = fmaxf(mx, S[t][i]);
    mx = rows_max(mx);
    const float mc = (mx > HILS_NEG_INF) ? mx * c2 : 0.f;
    float l = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        S[t][i] = __builtin_amdgcn_exp2f(fmaf(S[t][i], c2, -mc));
        l += S[t][i];
      }
    l = rows_sum(l);
    const float wr = (col < G) ? bf2f(sl_w[sl_id[si] * DR_NH + col]) : 0.f;
    const float f = (l > 0.f) ? wr / l : 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      dr_u4 pk;
      pk.x = pack_bf2(S[2 * h][0] * f, S[2 * h][1] * f);
      pk.y = pack_bf2(S[2 * h][2] * f, S[2 * h][3] * f);
      pk.z = pack_bf2(S[2 * h + 1][0] * f, S[2 * h + 1][1] * f);
      pk.w = pack_bf2(S[2 * h + 1][2] * f, S[2 * h + 1][3] * f);
      pb[h] = __builtin_bit_cast(bf16x8_t, pk);
    }
  };

  // One chunk: its eight groups in stream order; ring place s % NR holds group s and is re-issued
  // for the group NR places on (of this chunk or of the next one, at byte offset noff).  The last
  // chunk of the wavefront is a second copy of the code without the next chunk's loads, so that
  // no load is conditional.
  dr_u4 R[NR][GL];
  auto chunk = [&](int si, long coff, long noff, auto more) __attribute__((always_inline)) {
    constexpr bool MORE = decltype(more)::value;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      if (s < 4) consume_k(R[s % NR], s);
      else consume_v(R[s % NR], s - 4);
      if (s == 3) softmax(si);
      if (s + NR < 8) issue(R[s % NR], coff, s + NR);
      else if (MORE) issue(R[s % NR], noff, s + NR - 8);
    }
  };
  if (nsl > 0) {
    long coff = chunk_off(0);
#pragma unroll
    for (int s = 0; s < NR; ++s) issue(R[s], coff, s);
    hook();
    for (int si = 0; si + 1 < nsl; ++si) {
      const long noff = chunk_off(si + 1);
      chunk(si, coff, noff, std::true_type{});
      coff = noff;
    }
    chunk(nsl - 1, coff, 0, std::false_type{});
  } else {
    hook();
  }

  // accumulator register i of tile mt in lane (head = col, j) is feature mt*16 + 4j + i
  if (col < G) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      *(f32x4_t*)&o_s[((size_t)wave * G + col) * D + mt * 16 + 4 * j] = O[mt];
  }
  __syncthreads();
  for (int i = tid; i < G * D; i += NWAVE * 64) {
    const int g = i / D, dv = i - g * D;
    float x = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < NWAVE; ++w2) x += o_s[((size_t)w2 * G + g) * D + dv];
    if (dm.nsplit == 1) o[(bt * dm.HQ + hk * G + g) * (long)D + dv] = f2bf(x);
    else partial[((bt * dm.HQ + hk * G + g) * (long)dm.nsplit + split) * D + dv] = x;
  }
}

