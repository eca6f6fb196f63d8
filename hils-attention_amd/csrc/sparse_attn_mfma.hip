// Sparse attention forward on bf16 MFMA for prefill-sized query counts.
//
// The work is regrouped by chunk, not by query.  One workgroup owns T consecutive queries
// of one (batch, KV head).  It sorts the T*K (query, slot) pairs by chunk index in LDS, so
// that all queries of the block that selected chunk c sit next to each other ("a visit").
// A wavefront takes up to 16/G queries of a visit (16 rows: queries x the G heads of the
// KV head), loads the chunk's K rows and the gathered query rows straight into MFMA
// operands, forms S^T = K Q^T (tokens x rows) with 16x16x32 MFMAs, does the per-chunk
// softmax along the accumulator registers, and feeds P back as the A operand of
// O = P V without leaving registers (the contraction order over tokens is permuted to
// the accumulator layout; V is pre-transposed per chunk in the same order).  The
// (rows x Dv) partial outputs are summed into a fixed-point output tile in LDS with integer
// LDS atomics, which is what lets rows of different visits be arbitrary subsets of the block.
#include "common.h"
#include "../../include/hils_amd.h"

#define GA_THREADS 512
#ifndef GA_THREADS_NARROW
#define GA_THREADS_NARROW 768  // D = Dv = 64
#endif
#define GA_WAVES (GA_THREADS / 64)
#define GA_S 64                 // chunk size this kernel is built for
#define GA_MAXP 16              // (query, slot) pairs of a block per thread
#define GA_KEY_INVALID 0xFFFFFFFFu
#define GA_PAIR_BITS 12

// ---------------------------------------------------------------------------
// Operand packing.  Each 64-token chunk of K and V of a (batch, KV head) is rewritten once
// into the exact register order of the 16x16x32 MFMA operands the forward kernel needs, so
// that every operand load of a wavefront is one contiguous 1 KiB burst (8 full cache lines)
// instead of 16 half-used lines at a 2*H*D-byte stride:
//   kp[chunk][mt][ks][lane][8] = K[token mt*16 + (lane&15)][d = ks*32 + (lane>>4)*8 + e]
//   vp[chunk][dt][s][lane][8]  = V[token tok(s, lane>>4, e)][dv = dt*16 + (lane&15)]
// with tok(s, j, e) = 32*s + 16*(e/4) + 4*j + e%4, the order in which an accumulator-layout
// P supplies tokens when it is fed back as the A operand of O = P V.
// Also records max|V| of every chunk (it bounds the fixed-point output accumulation).
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
pack_kv_kernel(const bf16_t* __restrict__ k, const bf16_t* __restrict__ v, bf16_t* __restrict__ kp,
               bf16_t* __restrict__ vp, float* __restrict__ vmax, int Lkv, int H, int D, int Dv,
               int nchunk) {
  extern __shared__ bf16_t tile[];  // 64 x (max(D, Dv) + 2)
  __shared__ float red[32];
  const int c = blockIdx.x, h = blockIdx.y;
  const long b = blockIdx.z;
  const long chunk = (b * H + h) * (long)nchunk + c;
  // ---- K: rows are already contiguous along d; only the order of 16-byte pieces changes
  {
    const int pieces = D / 8;  // 16-byte pieces per token row
    bf16_t* out = kp + chunk * (long)GA_S * D;
    for (int i = threadIdx.x; i < GA_S * pieces; i += 256) {
      // destination order: ((mt * KS + ks) * 64 + lane)
      const int lane = i & 63, blk = i >> 6;
      const int KS = D / 32;
      const int mt = blk / KS, ks = blk - mt * KS;
      const int tok = mt * 16 + (lane & 15), d = ks * 32 + (lane >> 4) * 8;
      const uint4 x = *(const uint4*)(k + ((b * Lkv + (long)c * GA_S + tok) * H + h) * D + d);
      *(uint4*)(out + (long)i * 8) = x;
    }
  }
  // ---- V: transposed through LDS
  const int DP = Dv + 2;
  const int d8n = Dv / 8;
  float mx = 0.f;
  for (int i = threadIdx.x; i < GA_S * d8n; i += 256) {
    const int s = i / d8n, d8 = i - s * d8n;
    uint4 x = *(const uint4*)(v + ((b * Lkv + (long)c * GA_S + s) * H + h) * Dv + d8 * 8);
    const bf16_t* xs = (const bf16_t*)&x;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      tile[s * DP + d8 * 8 + e] = xs[e];
      mx = fmaxf(mx, fabsf(bf2f(xs[e])));
    }
  }
  mx = block_max(mx, red);  // contains the barrier that orders the tile writes
  if (threadIdx.x == 0) vmax[chunk] = mx;
  if (!vp) return;  // only max|V| wanted
  bf16_t* out = vp + chunk * (long)GA_S * Dv;
  for (int i = threadIdx.x; i < Dv * 8; i += 256) {
    // destination order: ((dt * 2 + s) * 64 + lane)
    const int lane = i & 63, blk = i >> 6;
    const int dt = blk >> 1, s = blk & 1;
    const int dv = dt * 16 + (lane & 15), j = lane >> 4;
    bf16_t y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int tok = 32 * s + 16 * (e >> 2) + 4 * j + (e & 3);
      y[e] = tile[tok * DP + dv];
    }
    *(uint4*)(out + (long)i * 8) = *(uint4*)y;
  }
}

// Fixed point by accumulator bias: a product accumulated onto GA_FX_BIAS = 1.5 * 2^23 comes out
// as a float whose unit in the last place is 1, so (bits - bits of the bias) is the sum rounded
// to an integer, for |sum| < 2^22.  The kernel adds the raw bits and counts the adds of every
// output row; the biases leave in the epilogue (all of it modulo 2^32).
#define GA_FX_BIAS 12582912.0f
#define GA_FX_BIAS_BITS 0x4B400000
#define GA_FX_LOG2_MAX 21  // sums are scaled below 2^21: one bit of head room for the rounding of P

struct GaDims {
  int L, Lkv, HQ, H, B, K, NW, T, nblk, nchunk, mask_last;
  float sm_scale;
  // indices (and weights) are shared by q_block consecutive queries (T % q_block == 0); weights
  // have WH = HQ or H heads; sm_n * exp(-max) joins every chunk's softmax denominator
  int q_block, WH;
  float sm_n;
  int merge_col;  // with a local-branch output given: the weight column that scales it
  uint32_t k_magic, qb_magic;  // hils_udiv_magic of K and q_block (pair index < 2^16, query index < 2^24)
};

// Power-of-two fixed-point scale for sums bounded by `bound`: bound * scale < 2^GA_FX_LOG2_MAX.
__device__ __forceinline__ float ga_fx_scale(float bound) {
  if (!(bound > 0.f && bound < 3.0e38f)) return 1.f;
  int e2 = GA_FX_LOG2_MAX - 1 - ilogbf(bound);
  e2 = e2 > 90 ? 90 : (e2 < -90 ? -90 : e2);
  return ldexpf(1.f, e2);
}

// ---- explicit operand loads --------------------------------------------------------------
// The tile stream below keeps several global loads in flight across loop iterations (the next
// tile's query rows, the next visit's K and V).  Which of them are outstanding at a use depends on
// wavefront-uniform branches (does the chunk change?), and the compiler's wait-count insertion
// merges such paths to "wait for nearly everything", which exposed one full memory latency per
// tile.  So the loads of the stream are issued by inline assembly, which that pass does not track,
// and the kernel waits itself: vector-memory loads return in issue order, so
// `s_waitcnt vmcnt(N)` with N = the loads issued after the wanted one (a lower bound is always
// safe; stores are never counted) guarantees it has landed.  A register that a load is still
// writing must not be read or copied before its wait: the waits are followed by empty asm
// statements that "modify" the registers, which orders every use behind the wait.
typedef unsigned ga_u32x4 __attribute__((ext_vector_type(4)));

template <int OFF>
__device__ __forceinline__ void ga_load128(ga_u32x4& dst, unsigned voff, const void* sbase) {
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "+v"(dst) : "v"(voff), "s"(sbase), "n"(OFF));
}
__device__ __forceinline__ void ga_load16(unsigned& dst, unsigned voff, const void* sbase) {
  asm volatile("global_load_ushort %0, %1, %2" : "+v"(dst) : "v"(voff), "s"(sbase));
}
template <int N>
__device__ __forceinline__ void ga_vmwait() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N));
}
__device__ __forceinline__ void ga_pin(ga_u32x4& a) { asm volatile("" : "+v"(a)); }
__device__ __forceinline__ void ga_pin(unsigned& a) { asm volatile("" : "+v"(a)); }
__device__ __forceinline__ bf16x8_t ga_bf(const ga_u32x4& x) { return __builtin_bit_cast(bf16x8_t, x); }

// One tile of the stream a wavefront works through: up to 16/G (query, slot) pairs of a visit.
template <int KS>
struct GaTile {
  ga_u32x4 bq[KS];  // gathered query rows (B operand of S^T = K Q^T), this lane's pieces
  unsigned wbits;   // this lane's row: its weight (bf16 bits)
  float rs;         // ... and the fixed-point scale of its output row
  int pk;           // ... and its pair (query of the block << 8 | slot)
  int n;            // real pairs in the tile
  int orow[4];      // output-tile element offsets of this lane's four accumulator rows
};

// Output tiles are accumulated in LDS as 32-bit fixed point: integer LDS atomics run at
// full rate on this hardware (float LDS atomics do not), and integer addition is
// associative, so the result does not depend on the order in which wavefronts add.
// The scale is chosen per output row from bound = sum_k |w_row,k| * max_visited|V|, which
// bounds every element of the row because each P row is a convex combination: a row keeps
// 20 bits below its own bound however small its weights are beside its neighbours'.
template <int D, int DV, int G, bool SLOPE, int NT>
__global__ void __launch_bounds__(NT)
sparse_attn_fwd_gather(const bf16_t* __restrict__ q, bf16_t* qp, const bf16_t* __restrict__ kp,
                       const bf16_t* __restrict__ vp, const float* __restrict__ vmax,
                       const bf16_t* __restrict__ weights, const int32_t* __restrict__ indices,
                       const float* __restrict__ slope, const bf16_t* __restrict__ swa_o,
                       bf16_t* __restrict__ o, float* __restrict__ lse, GaDims dm) {
  constexpr int KS = D / 32;    // k-steps of S^T = K Q^T
  constexpr int DT = DV / 16;   // 16-wide output column tiles
  constexpr int QT = 16 / G;    // queries per 16-row tile
  constexpr int MAXP = GA_MAXP;  // pairs per thread: T*K <= MAXP * GA_THREADS
  typedef GaTile<KS> Tile;
  extern __shared__ __align__(16) int smem_i[];
  const int R = dm.T * G;
  int* o_acc = smem_i;                       // R x DV fixed point
  int* cur = o_acc + (size_t)R * DV;         // nchunk: histogram -> running ends
  int* pairs = cur + dm.nchunk;              // T*K pairs (query << 8 | slot) grouped by chunk
  int* nadd = pairs + dm.T * dm.K;           // R: tiles added to each output row
  float* rscale = (float*)(nadd + R);        // R: sum_k |w| of the row, then its fixed-point scale
  __shared__ float red[32];
  __shared__ int scan_s[NT / 64];
  __shared__ int next_s;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  // XCD-aware order: hardware hands consecutive workgroup ids to the 8 XCDs in turn, so
  // id -> (xcd, slot); each XCD walks one contiguous share of the (batch, head, block)
  // list, latest query blocks first, and its L2 sees one head's K/V at a time.
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
  const long LB = dm.L / dm.q_block;          // rows of indices / weights per batch element
  const bool w_per_q = dm.WH == dm.HQ;        // weights per query head (else per KV head)

  // ---- prologue.  All global loads of the block set-up are issued before anything waits:
  // the query rows to repack, the selected chunk indices, and the weight rows.
  // (0) Packed copy of this block's query rows: within the G heads of a (query, KV head) the
  // 16-byte pieces are interleaved head-minor, [piece][head][8], so that the B-operand loads
  // of the G lanes that hold the heads of one query are contiguous (whole cache lines; read in
  // place, a row's four lanes would touch half a line each).  Only this workgroup reads what it
  // writes here (made visible by the barriers below).
  constexpr int PPR = D / 8;
  constexpr int QPK = 10;  // pieces per thread in flight (a 72-query block of 4 heads, D = 128, has 9)
  const int npiece = dm.T * G * PPR;
  uint4 qtmp[QPK];
#pragma unroll
  for (int e = 0; e < QPK; ++e) {
    const int i = tid + e * NT;
    const int ql = i / (G * PPR), rem = i - ql * (G * PPR);
    const int g2 = rem / PPR, pc = rem - g2 * PPR;
    const bool ok = i < npiece && t0 + ql < dm.L;
    const long blk_e = ((b * dm.L + (ok ? t0 + ql : t0)) * (long)dm.HQ + hk * G) * D;  // t0 < L always
    // relaxed atomic loads: the compiler keeps them here, ahead of the loads below, instead of
    // moving them next to their use behind the weight loop (a second exposed latency)
    const unsigned long long* src = (const unsigned long long*)(q + blk_e + g2 * D + pc * 8);
    const unsigned long long lo = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    const unsigned long long hi = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    qtmp[e] = make_uint4((unsigned)lo, (unsigned)(lo >> 32), (unsigned)hi, (unsigned)(hi >> 32));
  }
  // (1) selected chunk of every (query, slot) pair of the block
  int creg[MAXP], preg[MAXP];
#pragma unroll
  for (int e = 0; e < MAXP; ++e) {
    const int i = tid + e * NT;
    int c = -1;
    preg[e] = 0;
    if (i < npair) {
      const int ql = (int)hils_udiv((uint32_t)i, (uint32_t)K, dm.k_magic), slot = i - ql * K;
      preg[e] = (ql << 8) | slot;
      if (t0 + ql < dm.L) c = indices[((b * LB + (long)hils_udiv((uint32_t)(t0 + ql), (uint32_t)dm.q_block, dm.qb_magic)) * dm.H + hk) * (long)K + slot];
    }
    creg[e] = c;
  }
  // (2) weight rows, for the bound of the fixed-point scale: a row's sum of |w| over the K slots
  // (aligned dword loads, all in flight together)
  for (int row = tid; row < R; row += NT) {
    const int ql = row / G, g = row - ql * G;
    float a = 0.f;
    if (t0 + ql < dm.L) {
      const long e0 = ((b * LB + (long)hils_udiv((uint32_t)(t0 + ql), (uint32_t)dm.q_block, dm.qb_magic)) * (long)dm.WH + (w_per_q ? hk * G + g : hk)) *
                      dm.NW;  // first element
      a = hils_abs_row_sum_bf16(weights, e0, K, (long)dm.B * LB * dm.WH * dm.NW);
    }
    rscale[row] = a;  // only this thread touches the entry until the barrier behind the scan
  }
  // The packed copy goes through LDS (the output tile is not in use yet): pieces arrive in the
  // order of the source rows and leave in packed order, so that loads and stores are both
  // contiguous 1 KiB per wavefront instruction.  The staged pieces fit the output tile: a row has
  // D / 8 pieces of 16 bytes against DV * 4 bytes of accumulators (D <= 2 * DV).
  static_assert(D <= 2 * DV, "the staged query pieces must fit inside the output tile");
  uint4* stage = (uint4*)o_acc;
#pragma unroll
  for (int e = 0; e < QPK; ++e) {
    const int i = tid + e * NT;
    const int ql = i / (G * PPR), rem = i - ql * (G * PPR);
    const int g2 = rem / PPR, pc = rem - g2 * PPR;
    if (i < npiece) stage[ql * (G * PPR) + pc * G + g2] = qtmp[e];
  }
  for (int i = QPK * NT + tid; i < npiece; i += NT) {  // blocks with more pieces (rare shapes)
    const int ql = i / (G * PPR), rem = i - ql * (G * PPR);
    const int g2 = rem / PPR, pc = rem - g2 * PPR;
    const long blk_e = ((b * dm.L + (t0 + ql < dm.L ? t0 + ql : t0)) * (long)dm.HQ + hk * G) * D;
    stage[ql * (G * PPR) + pc * G + g2] = *(const uint4*)(q + blk_e + g2 * D + pc * 8);
  }
  for (int i = tid; i < dm.nchunk; i += NT) cur[i] = 0;
  for (int i = tid; i < R; i += NT) nadd[i] = 0;
  if (tid == 0) next_s = 0;
  lds_barrier();
  for (int i = tid; i < npiece; i += NT) {
    const int ql = i / (G * PPR);
    const uint4 x = stage[i];
    stage[i] = make_uint4(0, 0, 0, 0);  // this thread's share of clearing the output tile
    if (t0 + ql < dm.L)
      *(uint4*)(qp + ((b * dm.L + t0 + ql) * (long)dm.HQ + hk * G) * D + (i - ql * (G * PPR)) * 8) = x;
  }
  for (int i = npiece * 4 + tid; i < R * DV; i += NT) o_acc[i] = 0;  // the rest of the tile
  // (LDS-only barriers up to the last one of the prologue: the packed-query stores above stay in
  // flight behind the sort instead of being waited for here)
  lds_barrier();
  // histogram of the selected chunks
#pragma unroll
  for (int e = 0; e < MAXP; ++e) {
    int c = creg[e];
    if (c < -1 || c >= dm.nchunk) c = -1;
    if (c < 0 && lse) {
      const int i = tid + e * NT;
      const int ql = (int)hils_udiv((uint32_t)i, (uint32_t)K, dm.k_magic), slot = i - ql * K;
      if (i < npair && t0 + ql < dm.L) {
#pragma unroll
        for (int g = 0; g < G; ++g)
          lse[((b * dm.L + t0 + ql) * dm.HQ + hk * G + g) * (long)K + slot] = HILS_NEG_INF;
      }
    }
    creg[e] = c;
    if (c >= 0) atomicAdd(&cur[c], 1);
  }
  lds_barrier();  // histogram complete
  // max |V| over the visited chunks; exclusive scan of the histogram on the way
  float vm = 0.f;
  const int per_thr = (dm.nchunk + NT - 1) / NT;
  const int c_lo = tid * per_thr;
  int local = 0;
  for (int c = c_lo; c < c_lo + per_thr && c < dm.nchunk; ++c) {
    const int h = cur[c];
    if (h > 0) vm = fmaxf(vm, vmax[(b * dm.H + hk) * (long)dm.nchunk + c]);
    local += h;
  }
  int incl = local;
#pragma unroll
  for (int o2 = 1; o2 < 64; o2 <<= 1) {
    const int x = __shfl_up(incl, o2, 64);
    if (lane >= o2) incl += x;
  }
  if (lane == 63) scan_s[wave] = incl;
  vm = block_max_lds(vm, red);  // barrier: scan_s visible, all histogram reads done
  int base = incl - local;
  for (int w2 = 0; w2 < wave; ++w2) base += scan_s[w2];
  for (int c = c_lo; c < c_lo + per_thr && c < dm.nchunk; ++c) {
    const int h = cur[c];
    cur[c] = base;
    base += h;
  }
  for (int row = tid; row < R; row += NT) rscale[row] = ga_fx_scale(rscale[row] * vm);
  lds_barrier();
#pragma unroll
  for (int e = 0; e < MAXP; ++e)
    if (creg[e] >= 0) pairs[atomicAdd(&cur[creg[e]], 1)] = preg[e];
  __syncthreads();  // now chunk c owns pairs[cur[c-1] .. cur[c])

  const float c2 = dm.sm_scale * HILS_LOG2E;
  const int qs = r / G, g = r - qs * G;  // this lane's row of a tile: query slot, head
  const int hq = hk * G + g;
  const float sl = SLOPE ? slope[hq] : 0.f;
  // rows of a tile are addressed from the block's first query with 32-bit byte offsets into the
  // packed copy, in which the G heads of a query are interleaved per 16-byte piece: the lanes of
  // one query read contiguous bytes
  const char* qb = (const char*)(qp + ((b * dm.L + t0) * (long)dm.HQ + hk * G) * D);
  const bf16_t* wb = weights + ((b * LB + t0 / dm.q_block) * (long)dm.WH + (w_per_q ? hk * G : hk)) * dm.NW;
  float* lse_blk = lse ? lse + (b * dm.L + t0) * (long)dm.HQ * K : nullptr;  // the block's first row
  const unsigned q_lane = (unsigned)((j * G + g) * 8) * 2u, w_lane = w_per_q ? (unsigned)(g * dm.NW) : 0u;
  const unsigned q_step = (unsigned)dm.HQ * D * 2u;  // bytes per query of the block
  const int w_step = dm.WH * dm.NW;                  // elements per group of q_block queries

  // ---- visits: a wavefront takes chunks from a shared counter; a visit is all pairs of the
  // block on one chunk, processed as tiles of up to QT pairs.  The tile stream of a wavefront
  // is software-pipelined so that no operand load is waited for right after it is issued:
  //   step i:  issue Q(i+1);  O += P(i-1) V  [then V(chunk i) replaces V in place];
  //            S(i) = K Q(i)^T  [then K(chunk i+1) replaces K in place];  softmax -> P(i).
  // K and V of a chunk are reloaded only when the next tile belongs to another chunk.  Two tile
  // records alternate between "current" and "next / previous", so nothing is copied per step.
  ga_u32x4 ka[4][KS], vb[DT][2];
  constexpr int NK = 4 * KS;   // loads of a K reload
  constexpr int NV = 2 * DT;   // loads of a V reload
  constexpr int NA = KS + 1;   // loads of a tile issue (query pieces + weight)
  // operand loads: a wavefront-uniform 64-bit base plus this lane's 32-bit byte offset; the
  // instruction's immediate offset reaches 4 KiB, so a chunk is addressed from 4 KiB-spaced bases
  const unsigned lane_b = lane * 16;
  const char* kp_unit = (const char*)(kp + (b * dm.H + hk) * (long)dm.nchunk * GA_S * D);
  const char* vp_unit = (const char*)(vp + (b * dm.H + hk) * (long)dm.nchunk * GA_S * DV);
  auto load_k_all = [&](int c) {
    const char* kbase = kp_unit + (long)c * (GA_S * D * 2);
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        constexpr int dummy = 0; (void)dummy;
        const int piece = mt * KS + ks;  // 1 KiB pieces
        const char* sb = kbase + (piece / 4) * 4096;
        switch (piece % 4) {
          case 0: ga_load128<0>(ka[mt][ks], lane_b, sb); break;
          case 1: ga_load128<1024>(ka[mt][ks], lane_b, sb); break;
          case 2: ga_load128<2048>(ka[mt][ks], lane_b, sb); break;
          default: ga_load128<3072>(ka[mt][ks], lane_b, sb); break;
        }
      }
  };
  auto load_v_half = [&](int c, int d0, int nd) {  // column tiles d0 .. d0+nd-1
    const char* vbase = vp_unit + (long)c * (GA_S * DV * 2);
#pragma unroll
    for (int u = 0; u < nd; ++u)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const int piece = (d0 + u) * 2 + s2;
        const char* sb = vbase + (piece / 4) * 4096;
        switch (piece % 4) {
          case 0: ga_load128<0>(vb[d0 + u][s2], lane_b, sb); break;
          case 1: ga_load128<1024>(vb[d0 + u][s2], lane_b, sb); break;
          case 2: ga_load128<2048>(vb[d0 + u][s2], lane_b, sb); break;
          default: ga_load128<3072>(vb[d0 + u][s2], lane_b, sb); break;
        }
      }
  };
  auto pin_k = [&]() {
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ga_pin(ka[mt][ks]);
  };
  auto pin_v = [&]() {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      ga_pin(vb[dt][0]);
      ga_pin(vb[dt][1]);
    }
  };
  const int npair_valid = cur[dm.nchunk - 1];  // pairs with a valid chunk
  // next non-empty visit: chunk id (or -1) and its pair range
  auto grab = [&](int& vs_o, int& ve_o) -> int {
    for (;;) {
      int c = 0;
      if (lane == 0) c = atomicAdd(&next_s, 1);
      c = __builtin_amdgcn_readfirstlane(c);
      if (c >= dm.nchunk) return -1;
      vs_o = c ? cur[c - 1] : 0;
      if (vs_o >= npair_valid) return -1;  // every pair lies in an earlier chunk
      ve_o = cur[c];
      if (vs_o != ve_o) return c;
    }
  };
  // tile after (c, p, ve)
  auto advance = [&](int& c, int& p, int& ve) {
    if (p + QT < ve) { p += QT; return; }
    int vs2, ve2;
    c = grab(vs2, ve2);
    p = vs2;
    ve = ve2;
  };
  // A tile's gathered query rows (B operands), weight, row scale: NA loads.  Padding rows of a
  // visit's last tile repeat the tile's last pair with weight 0: their P is exactly 0 and is
  // added to that pair's output rows.
  const char* wb_c = (const char*)wb;
  auto issue_tile = [&](Tile& t, int p, int ve) {
    t.n = (ve - p < QT) ? ve - p : QT;
    const int last = t.n - 1;
    t.pk = pairs[p + (qs < last ? qs : last)];
    const unsigned ql = (unsigned)t.pk >> 8;
    const unsigned qoff = __umul24(ql, q_step) + q_lane;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      switch (ks) {
        case 0: ga_load128<0>(t.bq[ks], qoff, qb); break;
        case 1: ga_load128<4 * G * 16>(t.bq[ks], qoff, qb); break;
        case 2: ga_load128<2 * 4 * G * 16>(t.bq[ks], qoff, qb); break;
        default: ga_load128<3 * 4 * G * 16>(t.bq[ks], qoff, qb); break;
      }
    }
    const unsigned woff =
        (__umul24(dm.q_block == 1 ? ql : ql / (unsigned)dm.q_block, (unsigned)w_step) + w_lane + (t.pk & 255)) * 2u;
    ga_load16(t.wbits, woff, wb_c);
    t.rs = rscale[ql * G + g];
  };
  auto pin_tile = [&](Tile& t) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ga_pin(t.bq[ks]);
    ga_pin(t.wbits);
  };
  // output rows 4j .. 4j+3 of a tile starting at pair p (element offsets of this lane's column)
  auto tile_rows = [&](Tile& t, int p) {
    const int last = t.n - 1;
    if constexpr (G >= 4) {  // the four rows are consecutive heads of one query
      const int qsl = (4 * j) / G;
      const int pk = pairs[p + (qsl < last ? qsl : last)];
      const int base = ((pk >> 8) * G + (4 * j) % G) * DV + r;
#pragma unroll
      for (int i = 0; i < 4; ++i) t.orow[i] = base + i * DV;
    } else {
      int pk_o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int qsl = (4 * j + i) / G;
        pk_o[i] = pairs[p + (qsl < last ? qsl : last)];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int rr = 4 * j + i;
        t.orow[i] = ((pk_o[i] >> 8) * G + rr % G) * DV + r;
      }
    }
  };
  bf16x8_t ap[2];   // P of the previous tile (A operand of O = P V)
  // S = K Q^T of tile t (its operands have landed), softmax, P -> ap; K(c_next) replaces K when asked
  auto score_stage = [&](Tile& t, bool reload, int c_next) {
    // four independent accumulation chains (token tiles), interleaved so that a chain's next
    // MFMA is issued only after three others
    f32x4_t st[4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) st[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
        st[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ga_bf(ka[mt][ks]), ga_bf(t.bq[ks]), st[mt], 0, 0, 0);
    if (reload) load_k_all(c_next);
    if (SLOPE) {
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int dist = GA_S - 2 - (mt * 16 + j * 4 + i);
          st[mt][i] -= sl * (float)(dist > 0 ? dist : 0);
        }
    }
    if (dm.mask_last && j == 3) st[3][3] = HILS_NEG_INF;  // token 63 = tile 3, lane group 3, register 3
    // (this file is compiled without NaN handling: the maxima are bare v_max3 instructions)
    float m = fmaxf(fmaxf(st[0][0], st[0][1]), st[0][2]);
    m = fmaxf(fmaxf(m, st[0][3]), st[1][0]);
    m = fmaxf(fmaxf(m, st[1][1]), st[1][2]);
    m = fmaxf(fmaxf(m, st[1][3]), st[2][0]);
    m = fmaxf(fmaxf(m, st[2][1]), st[2][2]);
    m = fmaxf(fmaxf(m, st[2][3]), st[3][0]);
    m = fmaxf(fmaxf(m, st[3][1]), st[3][2]);
    m = rows_max(fmaxf(m, st[3][3]));
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
    sum = rows_sum(sum);
    if (dm.sm_n != 0.f) sum += dm.sm_n * __builtin_amdgcn_exp2f(-mc);
    if (lse && qs < t.n && j == 0) {
      const int ql = t.pk >> 8, slot = t.pk & 255;
      lse_blk[(ql * dm.HQ + hq) * K + slot] = mc + __builtin_amdgcn_logf(sum);
    }
    if (j == 0) atomicAdd(&nadd[(t.pk >> 8) * G + g], 1);  // padding rows count on the row they are added to
    const float w_row = qs < t.n ? __uint_as_float(t.wbits << 16) : 0.f;
    const float f = w_row * t.rs * __builtin_amdgcn_rcpf(sum);  // fixed-point scale (a power of two) folded into P
    // P as the A operand of O = P V: k-step s takes tokens of accumulator tiles 2s, 2s+1
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      uint4 x;
      x.x = pack_bf2(st[2 * s][0] * f, st[2 * s][1] * f);
      x.y = pack_bf2(st[2 * s][2] * f, st[2 * s][3] * f);
      x.z = pack_bf2(st[2 * s + 1][0] * f, st[2 * s + 1][1] * f);
      x.w = pack_bf2(st[2 * s + 1][2] * f, st[2 * s + 1][3] * f);
      ap[s] = *(bf16x8_t*)&x;
    }
  };
  // O += P V for the tile whose rows are `orow` (V has landed); V(c_next) replaces V when asked
  const f32x4_t fx_bias = {GA_FX_BIAS, GA_FX_BIAS, GA_FX_BIAS, GA_FX_BIAS};
  auto output_stage = [&](const int* orow, bool reload, int c_next) {
    // four column tiles at a time: their eight MFMAs interleaved (two-deep chains), then the
    // operand reload, then the fixed-point adds
#pragma unroll
    for (int d0 = 0; d0 < DT; d0 += 4) {
      f32x4_t acc[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[u] = fx_bias;
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int u = 0; u < 4; ++u)
          acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ap[s2], ga_bf(vb[d0 + u][s2]), acc[u], 0, 0, 0);
      if (reload) load_v_half(c_next, d0, 4);
      if constexpr (G >= 4) {
        // the lane's four rows are consecutive heads of one query: one address, the rest are offsets
        // the instruction carries
        int* o0 = o_acc + orow[0];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) atomicAdd(o0 + i * DV + (d0 + u) * 16, __float_as_int(acc[u][i]));
      } else {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            atomicAdd(&o_acc[orow[i] + (d0 + u) * 16], __float_as_int(acc[u][i]));
      }
    }
  };

  // ---- the stream.  Issue order of a step i (x_i = "tile i is on another chunk than tile i-1"):
  //   A_i: query rows + weight of tile i+1 (NA loads, when there is a tile i+1)
  //   B_i: V of tile i's chunk (NV loads, when x_i), behind the MFMAs of O += P(i-1) V
  //   C_i: K of tile i+1's chunk (NK loads, when x_{i+1}), behind the MFMAs of S(i)
  // O += P(i-1) V needs B_{i-1}: the loads behind it are C_{i-1} (NK when x_i) and A_i;
  // S(i) needs C_{i-1} and A_{i-1}: the loads behind C_{i-1} are A_i and B_i (NV when x_i).
  // Without a tile i+1 there is no A_i and the step simply waits for everything.
  int c_cur, p_cur = 0, ve_cur = 0;
  c_cur = grab(p_cur, ve_cur);
  if (c_cur >= 0) {
    Tile ta, tb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) { ta.bq[ks] = (ga_u32x4){0, 0, 0, 0}; tb.bq[ks] = (ga_u32x4){0, 0, 0, 0}; }
    ta.wbits = tb.wbits = 0;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ka[mt][ks] = (ga_u32x4){0, 0, 0, 0};
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vb[dt][0] = vb[dt][1] = (ga_u32x4){0, 0, 0, 0};
    // step 0 (no previous tile): A_{-1} = tile 0, C_{-1} = K(c_0), then A_0, B_0 = V(c_0)
    issue_tile(ta, p_cur, ve_cur);
    tile_rows(ta, p_cur);
    load_k_all(c_cur);
    int c_nxt = c_cur, p_nxt = p_cur, ve_nxt = ve_cur;
    advance(c_nxt, p_nxt, ve_nxt);
    if (c_nxt >= 0) {
      issue_tile(tb, p_nxt, ve_nxt);
      tile_rows(tb, p_nxt);
    }
    load_v_half(c_cur, 0, DT);
    if (c_nxt >= 0) ga_vmwait<NA + NV>(); else ga_vmwait<NV>();
    pin_k();
    pin_tile(ta);
    score_stage(ta, c_nxt >= 0 && c_nxt != c_cur, c_nxt);
    int c_prev = c_cur;
    // one step: `cu` is the tile whose scores are due (its loads were issued a step ago), `nx`
    // holds the previous tile's output rows until the output stage is through, then the tile
    // after `cu`.
    auto step = [&](Tile& cu, Tile& nx) {
      c_cur = c_nxt; p_cur = p_nxt; ve_cur = ve_nxt;
      advance(c_nxt, p_nxt, ve_nxt);
      const bool more = c_nxt >= 0;
      const bool x = c_cur != c_prev;
      if (more) issue_tile(nx, p_nxt, ve_nxt);  // A_i; leaves nx.orow alone
      if (!more) ga_vmwait<0>(); else if (x) ga_vmwait<NA + NK>(); else ga_vmwait<NA>();
      pin_v();
      output_stage(nx.orow, x, c_cur);          // B_i
      if (more) tile_rows(nx, p_nxt);
      if (!more) ga_vmwait<0>(); else if (x) ga_vmwait<NA + NV>(); else ga_vmwait<NA>();
      pin_k();
      pin_tile(cu);
      score_stage(cu, more && c_nxt != c_cur, c_nxt);  // C_i
      c_prev = c_cur;
    };
    // the stream: tile 0 = ta (scored above), tile 1 = tb, tile 2 -> ta, ...
    bool last_is_a = true;
    while (c_nxt >= 0) {
      step(tb, ta);
      last_is_a = false;
      if (c_nxt < 0) break;
      step(ta, tb);
      last_is_a = true;
    }
    int orow_last[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) orow_last[i] = last_is_a ? ta.orow[i] : tb.orow[i];
    ga_vmwait<0>();
    pin_v();
    output_stage(orow_last, false, 0);
  }
  __syncthreads();
  constexpr int C8 = DV / 8;
  const int wcol = dm.merge_col;
  for (int i = tid; i < R * C8; i += NT) {
    const int row = i / C8, c8 = i - row * C8;
    const int ql = row / G, g2 = row - ql * G;
    const int t = t0 + ql;
    if (t < dm.L) {
      const int* src = o_acc + (size_t)row * DV + c8 * 8;
      const unsigned bias = (unsigned)nadd[row] * (unsigned)GA_FX_BIAS_BITS;  // wraps like the sums did
      const float fx_inv = 1.f / rscale[row];  // a power of two: exact
      float f[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = (float)(int)((unsigned)src[e] - bias) * fx_inv;
      const long orow_g = ((b * dm.L + t) * (long)dm.HQ + hk * G + g2) * DV + c8 * 8;
      if (swa_o) {  // o = remote branch + local branch * its inter-chunk weight, rounded once
        const float wl = bf2f(weights[((b * LB + (long)hils_udiv((uint32_t)t, (uint32_t)dm.q_block, dm.qb_magic)) * (long)dm.WH + (w_per_q ? hk * G + g2 : hk)) *
                                          dm.NW + wcol]);
        float sv[8];
        unpack8(*(const uint4*)(swa_o + orow_g), sv);
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = fmaf(sv[e], wl, f[e]);
      }
      uint4 x;
      x.x = pack_bf2(f[0], f[1]);
      x.y = pack_bf2(f[2], f[3]);
      x.z = pack_bf2(f[4], f[5]);
      x.w = pack_bf2(f[6], f[7]);
      *(uint4*)(o + orow_g) = x;
    }
  }
}

template <int D, int DV, int G, bool SLOPE>
static int ga_launch_s(dim3 grid, size_t smem, hipStream_t st, const bf16_t* q, bf16_t* qp, const bf16_t* k,
                       const bf16_t* vt, const float* vmax, const bf16_t* w, const int32_t* idx,
                       const float* slope, const bf16_t* swa_o, bf16_t* o, float* lse, const GaDims& dm) {
  static_assert(D % 32 == 0 && DV % 16 == 0 && 16 % G == 0, "tile shapes of the MFMA forward");
  // Narrow heads leave the wavefronts under 168 registers: twelve of them per workgroup (one workgroup
  // per compute unit, its size is what sets the occupancy) instead of eight.
  constexpr int NT = (D <= 64 && DV <= 64) ? GA_THREADS_NARROW : GA_THREADS;
  auto kern = sparse_attn_fwd_gather<D, DV, G, SLOPE, NT>;
  static HilsLdsReserve reserved;  // per instantiation
  if (int rc = hils_reserve_lds(&reserved, (const void*)kern, smem, "hils_sparse_attn_fwd")) return rc;
  hipLaunchKernelGGL(kern, grid, dim3(NT), smem, st, q, qp, k, vt, vmax, w, idx, slope, swa_o, o, lse, dm);
  return HILS_OK;
}

template <int D, int DV, int G>
static int ga_launch(dim3 grid, size_t smem, hipStream_t st, const bf16_t* q, bf16_t* qp, const bf16_t* k,
                     const bf16_t* vt, const float* vmax, const bf16_t* w, const int32_t* idx,
                     const float* slope, const bf16_t* swa_o, bf16_t* o, float* lse, const GaDims& dm) {
  if (slope) return ga_launch_s<D, DV, G, true>(grid, smem, st, q, qp, k, vt, vmax, w, idx, slope, swa_o, o, lse, dm);
  return ga_launch_s<D, DV, G, false>(grid, smem, st, q, qp, k, vt, vmax, w, idx, slope, swa_o, o, lse, dm);
}

template <int D, int DV>
static int ga_dispatch_g(int G, dim3 grid, size_t smem, hipStream_t st, const bf16_t* q, bf16_t* qp,
                         const bf16_t* k, const bf16_t* vt, const float* vmax, const bf16_t* w,
                         const int32_t* idx, const float* slope, const bf16_t* swa_o, bf16_t* o, float* lse,
                         const GaDims& dm) {
  switch (G) {
    case 1: return ga_launch<D, DV, 1>(grid, smem, st, q, qp, k, vt, vmax, w, idx, slope, swa_o, o, lse, dm);
    case 2: return ga_launch<D, DV, 2>(grid, smem, st, q, qp, k, vt, vmax, w, idx, slope, swa_o, o, lse, dm);
    case 4: return ga_launch<D, DV, 4>(grid, smem, st, q, qp, k, vt, vmax, w, idx, slope, swa_o, o, lse, dm);
    case 8: return ga_launch<D, DV, 8>(grid, smem, st, q, qp, k, vt, vmax, w, idx, slope, swa_o, o, lse, dm);
    case 16: return ga_launch<D, DV, 16>(grid, smem, st, q, qp, k, vt, vmax, w, idx, slope, swa_o, o, lse, dm);
  }
  return -1;
}

static size_t ga_vt_bytes(int B, int H, int nchunk, int Dv) {  // one packed tensor (K or V)
  size_t n = (size_t)B * H * nchunk * Dv * GA_S * sizeof(bf16_t);
  return (n + 255) & ~(size_t)255;
}

static size_t ga_vmax_bytes(int B, int H, int nchunk) {
  return ((size_t)B * H * nchunk * sizeof(float) + 255) & ~(size_t)255;
}

// Tile sizes: the largest T (queries per workgroup, a multiple of q_block and of 8 when it can be)
// such that the fixed-point output tile, the chunk histogram, the pair list and the add counts
// fit in the LDS of a compute unit, with at most GA_MAXP pairs per thread.  The more rows share a
// visit, the fewer bytes of K and V the block pulls per row.  Returns 0 when nothing fits.
#define GA_SMEM_MAX (160 * 1024 - 512)  // dynamic LDS beside the kernel's static arrays
static int ga_pick_T(int L, int G, int Dv, int K, int nchunk, int q_block, size_t* smem_out) {
  // per query: G output rows, K pairs, G add counts, G row scales
  const size_t per_q = (size_t)G * Dv * 4 + (size_t)K * 4 + (size_t)G * 4 + (size_t)G * 4;
  const size_t fixed = (size_t)nchunk * 4;
  if (fixed + per_q > GA_SMEM_MAX) return 0;
  long T = (long)((GA_SMEM_MAX - fixed) / per_q);
  if (T * K > GA_MAXP * GA_THREADS) T = (GA_MAXP * GA_THREADS) / K;
  if (T > L) T = L;
  if (T >= 8 && q_block <= 8 && 8 % q_block == 0) T &= ~7L;
  else T -= T % q_block;
  if (T < 1) return 0;
  *smem_out = fixed + (size_t)T * per_q;
  return (int)T;
}

// Workspace the MFMA path needs (the per-chunk transposed copy of V and the per-chunk max|V|),
// 0 if the shape is not covered by it.
size_t hils_ga_workspace_bytes(int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K, int S,
                               int q_block, int WH, float sm_n) {
  if (H <= 0 || HQ % H != 0) return 0;
  const int G = HQ / H;
  const bool ok = S == GA_S && (D == 64 || D == 128) && (Dv == 64 || Dv == 128) &&
                  (G == 1 || G == 2 || G == 4 || G == 8 || G == 16) && q_block >= 1 &&
                  L % q_block == 0 && (WH == HQ || WH == H) && sm_n >= 0.f && L >= 64 && Lkv >= S &&
                  K >= 1 && K <= 256 && (long)L * q_block < (1L << 31);  // hils_udiv by q_block stays exact
  if (!ok) return 0;
  size_t smem;
  const int T = ga_pick_T(L, G, Dv, K, Lkv / S, q_block, &smem);
  if (T == 0 || T % q_block != 0) return 0;  // a query block holds whole index-sharing groups
  const int nchunk = Lkv / S;
  return ga_vt_bytes(B, H, nchunk, Dv) + ga_vt_bytes(B, H, nchunk, D) + ga_vmax_bytes(B, H, nchunk) +
         (size_t)B * L * HQ * D * sizeof(bf16_t);  // packed V, packed K, per-chunk max|V|, packed Q
}

// Returns HILS_OK and sets *handled = 1 when the MFMA path ran.
int hils_sparse_attn_fwd_mfma(const void* q, const void* k, const void* v, const void* weights,
                              const int32_t* indices, const float* slope, const void* swa_o, int merge_col,
                              void* o, float* lse, void* workspace, int workspace_ready, int B, int L,
                              int Lkv, int HQ, int H, int D, int Dv, int K, int NW, int S, float sm_scale,
                              int mask_last, int q_block, int WH, float sm_n, void* stream,
                              int* handled) {
  *handled = 0;
  const int G = HQ / H;
  const int nchunk = Lkv / S;
  hipStream_t st = (hipStream_t)stream;
  size_t smem;
  const int T = ga_pick_T(L, G, Dv, K, nchunk, q_block, &smem);
  if (T == 0 || T % q_block != 0 || H > 65535 || B > 65535) return HILS_OK;
  const int nblk = (L + T - 1) / T;
  const long total = (long)nblk * H * B;
  if (total > (1L << 30)) return HILS_OK;
  bf16_t* vpk = (bf16_t*)workspace;
  bf16_t* kpk = (bf16_t*)((char*)workspace + ga_vt_bytes(B, H, nchunk, Dv));
  float* vmax = (float*)((char*)kpk + ga_vt_bytes(B, H, nchunk, D));
  bf16_t* qpk = (bf16_t*)((char*)vmax + ga_vmax_bytes(B, H, nchunk));
  if (!workspace_ready) {
    const int dmax = D > Dv ? D : Dv;
    hipLaunchKernelGGL(pack_kv_kernel, dim3(nchunk, H, B), dim3(256),
                       (size_t)GA_S * (dmax + 2) * sizeof(bf16_t), st, (const bf16_t*)k,
                       (const bf16_t*)v, kpk, vpk, vmax, Lkv, H, D, Dv, nchunk);
  }
  GaDims dm{L, Lkv, HQ, H, B, K, NW, T, nblk, nchunk, mask_last, sm_scale, q_block, WH, sm_n, merge_col,
            hils_udiv_magic((uint32_t)K), hils_udiv_magic((uint32_t)q_block)};
  const long per_xcd = (total + 7) / 8;
  dim3 grid((unsigned)(per_xcd * 8));
  int rc = -1;
#define GA_CALL(D_, DV_)                                                                       \
  rc = ga_dispatch_g<D_, DV_>(G, grid, smem, st, (const bf16_t*)q, qpk, kpk, vpk, vmax,        \
                              (const bf16_t*)weights, indices, slope, (const bf16_t*)swa_o, (bf16_t*)o, lse, dm)
  if (D == 64 && Dv == 64) GA_CALL(64, 64);
  else if (D == 128 && Dv == 128) GA_CALL(128, 128);
  else if (D == 64 && Dv == 128) GA_CALL(64, 128);
  else if (D == 128 && Dv == 64) GA_CALL(128, 64);
#undef GA_CALL
  if (rc != HILS_OK) return rc < 0 ? HILS_OK : rc;
  *handled = 1;
  return HILS_OK;
}

// Launches the packing kernel on explicit buffers: ap = a in A-operand order, bp = b in the
// transposed B-operand order, bmax = max|b| per chunk (also used by the backward kernels).
void hils_ga_pack_launch(const void* a, const void* b, void* ap, void* bp, float* bmax, int B, int Lkv,
                         int H, int Da, int Db, void* stream) {
  const int nchunk = Lkv / GA_S;
  const int dmax = Da > Db ? Da : Db;
  hipLaunchKernelGGL(pack_kv_kernel, dim3(nchunk, H, B), dim3(256),
                     (size_t)GA_S * (dmax + 2) * sizeof(bf16_t), (hipStream_t)stream, (const bf16_t*)a,
                     (const bf16_t*)b, (bf16_t*)ap, (bf16_t*)bp, bmax, Lkv, H, Da, Db, nchunk);
}

extern "C" int hils_pack_kv_chunks(const void* k, const void* v, void* workspace, size_t workspace_bytes,
                                   int B, int Lkv, int H, int D, int Dv, void* stream) {
  HILS_REQUIRE(k && v && workspace, "hils_pack_kv_chunks: null pointer");
  HILS_REQUIRE(B > 0 && Lkv >= GA_S && H > 0 && (D == 64 || D == 128) && (Dv == 64 || Dv == 128),
               "hils_pack_kv_chunks: bad sizes (Lkv >= 64, D and Dv in {64, 128})");
  HILS_REQUIRE(H <= 65535 && B <= 65535, "hils_pack_kv_chunks: H/B too large for the grid");
  const int nchunk = Lkv / GA_S;
  {
    const size_t need = ga_vt_bytes(B, H, nchunk, Dv) + ga_vt_bytes(B, H, nchunk, D) + ga_vmax_bytes(B, H, nchunk);
    HILS_REQUIRE(workspace_bytes >= need,
                 "hils_pack_kv_chunks: workspace of %zu bytes is shorter than the %zu bytes the packed K, V and "
                 "per-chunk maxima of this shape take", workspace_bytes, need);
  }
  bf16_t* vpk = (bf16_t*)workspace;
  bf16_t* kpk = (bf16_t*)((char*)workspace + ga_vt_bytes(B, H, nchunk, Dv));
  float* vmax = (float*)((char*)kpk + ga_vt_bytes(B, H, nchunk, D));
  const int dmax = D > Dv ? D : Dv;
  hipLaunchKernelGGL(pack_kv_kernel, dim3(nchunk, H, B), dim3(256),
                     (size_t)GA_S * (dmax + 2) * sizeof(bf16_t), (hipStream_t)stream,
                     (const bf16_t*)k, (const bf16_t*)v, kpk, vpk, vmax, Lkv, H, D, Dv, nchunk);
  HILS_CHECK_LAUNCH("hils_pack_kv_chunks");
  return HILS_OK;
}
