// Decode sparse attention, row-streaming variant (D == Dv, G <= 4).
//
// Every K and V load is a fully coalesced 16-byte lane load: LR = D/8 neighbouring lanes
// read one 2*D-byte token row, 64/LR token rows per instruction.  q.K uses packed bf16
// dot2 instructions plus a DPP reduction over the LR lanes of a row; because K and V rows
// are mapped to lanes the same way, the softmax probabilities of a token already sit in
// the lanes that hold that token's V row, so P V needs no data movement at all.
#include "decode_rows.h"
#include "../../include/hils_amd.h"

#define DR_THREADS 256
#ifndef DR_MINW
#define DR_MINW 4
#endif
#define DR_WAVES (DR_THREADS / 64)
#define DR_S 64
#define DR_MAXSLOT 64  // slots a wavefront can own: K <= 256 over at least 4 wavefronts

struct DrDims {
  int L, Lkv, HQ, H, G, K, NW, nchunk, nsplit, mask_last;
  float sm_scale;
  // paged cache (page = chunk = 64 tokens): K and V are (num_pages, H, 64, D), the tokens of a
  // (page, head) contiguous, and chunk c of batch element b lives in page page_table[b][c]
  const int32_t* page_table;
  int max_pages, num_pages;
};

template <int D, int GMAX, int NWAVE>
__global__ void __launch_bounds__(NWAVE * 64, (NWAVE == 4 ? DR_MINW : 1))
sparse_attn_decode_rows_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                               const bf16_t* __restrict__ v, const bf16_t* __restrict__ weights,
                               const int32_t* __restrict__ indices, bf16_t* __restrict__ o,
                               float* __restrict__ partial, DrDims dm) {
  constexpr int LR = D / 8;        // lanes per token row
  constexpr int TPI = 64 / LR;     // token rows per load instruction
  constexpr int NI = DR_S / TPI;   // load instructions per chunk
  // load instructions per pipelined group: two groups (K and V) are in flight per wavefront, and
  // with four the 128 registers a 16-wavefront workgroup leaves each lane no longer hold them
  constexpr int GI = 2;
  constexpr int NG = NI / GI;      // groups per chunk
  extern __shared__ float o_s[];   // [wave][G][D] partial outputs
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int piece = lane % LR, tsub = lane / LR;
  const int split = blockIdx.x, hk = blockIdx.y;
  const long bt = blockIdx.z;
  const long b = bt / dm.L;
  const int G = dm.G, K = dm.K;

  uint4 qp[GMAX];  // this lane's 8 features of each query head, packed bf16
#pragma unroll
  for (int g = 0; g < GMAX; ++g) {
    qp[g] = make_uint4(0, 0, 0, 0);
    if (g < G) qp[g] = *(const uint4*)(q + (bt * dm.HQ + hk * G + g) * (long)D + piece * 8);
  }
  const float c2 = dm.sm_scale * HILS_LOG2E;
  // running output of this wavefront, kept in its private slice of LDS (lanes < LR own it)
  for (int i = lane; i < G * D; i += 64) o_s[(size_t)wave * G * D + i] = 0.f;

  const int per_split = (K + dm.nsplit - 1) / dm.nsplit;
  const int s_begin = split * per_split;
  const int s_end = (s_begin + per_split < K) ? s_begin + per_split : K;
  // this wavefront's slots (s_begin + wave, + NWAVE, ...) that hold a mapped chunk: first-row element
  // offset and slot number, kept in LDS so that the load of the next group never waits for an index
  long* sl_off = (long*)(o_s + (size_t)NWAVE * G * D) + (size_t)wave * DR_MAXSLOT;
  int* sl_id = (int*)((long*)(o_s + (size_t)NWAVE * G * D) + (size_t)NWAVE * DR_MAXSLOT) + wave * DR_MAXSLOT;
  int nsl = 0;
  long step = (long)TPI * (dm.page_table ? D : dm.H * D);
  for (int slot = s_begin + wave; slot < s_end; slot += NWAVE) {
    const int c = indices[(bt * dm.H + hk) * (long)K + slot];
    if (c < 0 || c >= dm.nchunk) continue;
    long row0;
    if (dm.page_table) {
      const int pg = dm.page_table[b * dm.max_pages + c];
      if (pg < 0 || pg >= dm.num_pages) continue;  // an unmapped chunk contributes nothing
      row0 = ((long)pg * dm.H + hk) * DR_S + tsub;
    } else {
      row0 = (b * dm.Lkv + (long)c * DR_S + tsub) * dm.H + hk;
    }
    // every lane stores its own first row (tsub differs): the list is per lane group in registers
    // of the loop below, so only lane 0's view goes to LDS and tsub is added back on use
    if (lane == 0 && nsl < DR_MAXSLOT) {
      sl_off[nsl] = (row0 - tsub) * D;
      sl_id[nsl] = slot;
    }
    ++nsl;
  }
  __builtin_amdgcn_wave_barrier();
  const long lane_off = (long)tsub * (dm.page_table ? D : dm.H * D) + piece * 8;

  // The (slot, group) units of this wavefront form one stream; the K and V rows of unit u+1 are
  // loaded while unit u is computed (two register buffers), so a load is never waited for right
  // after its issue, across group and slot boundaries alike.
  const int nu = nsl * NG;
  uint4 kr[2][GI], vr[2][GI];
  auto load_unit = [&](int u, uint4 (&kd)[GI], uint4 (&vd)[GI]) {
    const int si = u / NG, grp = u - si * NG;
    const long off = sl_off[si] + lane_off + (long)grp * GI * step;
#pragma unroll
    for (int i = 0; i < GI; ++i) {
      kd[i] = *(const uint4*)(k + off + i * step);
      vd[i] = *(const uint4*)(v + off + i * step);
    }
  };
  float mrun[GMAX], lrun[GMAX], acc[GMAX][8];
  auto compute_unit = [&](int u, const uint4 (&kc)[GI], const uint4 (&vc)[GI]) {
    const int si = u / NG, grp = u - si * NG;
    if (grp == 0) {
#pragma unroll
      for (int g = 0; g < GMAX; ++g) {
        mrun[g] = HILS_NEG_INF;
        lrun[g] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
      }
    }
    // flash-style pass over the chunk in NG groups of GI*TPI tokens; every token sub-group
    // (lanes with the same tsub) keeps its own running max / sum / accumulator
    float sc[GMAX][GI];
#pragma unroll
    for (int i = 0; i < GI; ++i)
#pragma unroll
      for (int g = 0; g < GMAX; ++g)
        if (g < G) {
          float s = row_sum<LR>(dot8_bf16(qp[g], kc[i], 0.f));
          if (dm.mask_last && grp == NG - 1 && i == GI - 1 && tsub == TPI - 1) s = HILS_NEG_INF;
          sc[g][i] = s;
        }
#pragma unroll
    for (int g = 0; g < GMAX; ++g)
      if (g < G) {
        float mn = mrun[g];
#pragma unroll
        for (int i = 0; i < GI; ++i) mn = fmaxf(mn, sc[g][i]);
        if (mn > HILS_NEG_INF) {
          const float corr = __builtin_amdgcn_exp2f((mrun[g] - mn) * c2);
          lrun[g] *= corr;
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[g][e] *= corr;
#pragma unroll
          for (int i = 0; i < GI; ++i) {
            sc[g][i] = __builtin_amdgcn_exp2f((sc[g][i] - mn) * c2);
            lrun[g] += sc[g][i];
          }
          mrun[g] = mn;
        } else {
#pragma unroll
          for (int i = 0; i < GI; ++i) sc[g][i] = 0.f;
        }
      }
#pragma unroll
    for (int i = 0; i < GI; ++i) {
      float vf[8];
      unpack8(vc[i], vf);
#pragma unroll
      for (int g = 0; g < GMAX; ++g)
        if (g < G) {
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[g][e] = fmaf(sc[g][i], vf[e], acc[g][e]);
        }
    }
    if (grp != NG - 1) return;
    // merge the token sub-groups, normalise, weight and add to the running output
    const int slot = sl_id[si];
#pragma unroll
    for (int g = 0; g < GMAX; ++g)
      if (g < G) {
        float m = mrun[g];
#pragma unroll
        for (int off = LR; off < 64; off <<= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
        const float sc2 = (mrun[g] > HILS_NEG_INF) ? __builtin_amdgcn_exp2f((mrun[g] - m) * c2) : 0.f;
        float l = lrun[g] * sc2;
#pragma unroll
        for (int off = LR; off < 64; off <<= 1) l += __shfl_xor(l, off, 64);
        const float wr = bf2f(weights[(bt * dm.HQ + hk * G + g) * (long)dm.NW + slot]);
        const float f = (l > 0.f) ? sc2 * wr / l : 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float x = acc[g][e] * f;
#pragma unroll
          for (int off = LR; off < 64; off <<= 1) x += __shfl_xor(x, off, 64);
          if (lane < LR) o_s[((size_t)wave * G + g) * D + lane * 8 + e] += x;
        }
      }
  };
  if (nu > 0) load_unit(0, kr[0], vr[0]);
  for (int u = 0; u < nu; u += 2) {
    if (u + 1 < nu) load_unit(u + 1, kr[1], vr[1]);
    compute_unit(u, kr[0], vr[0]);
    if (u + 1 < nu) {
      if (u + 2 < nu) load_unit(u + 2, kr[0], vr[0]);
      compute_unit(u + 1, kr[1], vr[1]);
    }
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

// (a wavefront keeps a list of at most DR_MAXSLOT slots: K <= 1024 covers every split the launcher picks)
bool hils_decode_rows_covers(int D, int Dv, int G, int K) {
  return D == Dv && (D == 64 || D == 128) && G <= 4 && K <= 16 * DR_MAXSLOT;
}

void hils_sparse_attn_decode_rows(const void* q, const void* k, const void* v, const void* weights,
                                  const int32_t* indices, void* o, void* workspace, int nsplit,
                                  int B, int L, int Lkv, int HQ, int H, int D, int K, int NW,
                                  float sm_scale, int mask_last, const int32_t* page_table, int max_pages,
                                  int num_pages, hipStream_t st) {
  const int G = HQ / H;
  DrDims dm{L, Lkv, HQ, H, G, K, NW, page_table ? max_pages : Lkv / DR_S, nsplit, mask_last, sm_scale,
            page_table, max_pages, num_pages};
  dim3 grid(nsplit, H, (unsigned)((long)B * L));
  // nsplit == 1 with many slots: one workgroup of 16 wavefronts per (query, KV head), no partial sums
  const int nwave = (nsplit == 1 && K >= 16) ? 16 : DR_WAVES;
  // partial outputs [wave][G][D] + the wavefronts' slot lists (row offsets, slot numbers)
  const size_t smem = (size_t)nwave * G * D * sizeof(float) + (size_t)nwave * DR_MAXSLOT * (sizeof(long) + sizeof(int));
#define DR_CALL_W(D_, G_, W_)                                                                    \
  hipLaunchKernelGGL((sparse_attn_decode_rows_kernel<D_, G_, W_>), grid, dim3(W_ * 64), smem, st, \
                     (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, (const bf16_t*)weights, \
                     indices, (bf16_t*)o, (float*)workspace, dm)
#define DR_CALL(D_, G_)                                                                          \
  do {                                                                                           \
    if (nwave == 16) DR_CALL_W(D_, G_, 16); else DR_CALL_W(D_, G_, DR_WAVES);                    \
  } while (0)
  if (D == 64) {
    if (G == 1) DR_CALL(64, 1); else if (G == 2) DR_CALL(64, 2); else DR_CALL(64, 4);
  } else {
    if (G == 1) DR_CALL(128, 1); else if (G == 2) DR_CALL(128, 2); else DR_CALL(128, 4);
  }
#undef DR_CALL_W
#undef DR_CALL
}
