// Sliding-window attention of the local branch: every query attends causally to the keys from
// the start of the chunk that holds (query - window + 1) up to itself (or from query - window + 1
// exactly), optionally without the landmark key of every chunk; outputs o and the natural-log LSE.
//
// A wavefront owns 32 score rows (query x head of the group), held as matrix B operands; the keys
// and values of the window pass through LDS in 64-token tiles: K row-major (A operand of the
// transposed scores K Q^T), V as the B operand of O += P V, whose contraction runs over the tokens.
// With the rows as matrix columns a row's 64 scores lie in 16 registers of 4 lanes (in-lane softmax
// plus one row-swap reduction) and the probabilities are already the A operand of the second product.
#include <type_traits>
#include "stream_tiles.h"
#include "../../include/hils_amd.h"

struct SwaDims {
  int Lq, Lk, HQ, H, window, chunk, mask_lmk, expand, kv_start, chunk_pow2;
  float sm_scale;
};

// Workgroup order.  Neighbouring blocks of a head read the same key / value (or query) tiles, and the
// hardware hands consecutive workgroup ids to the 8 XCDs in turn: with the block index in the grid's
// fastest dimension every tile was fetched from HBM by as many XCDs (L2s) as blocks share it.  The grids
// here are one-dimensional, id -> (xcd, slot), and each XCD walks one contiguous share of the
// (batch, head, block) list.  False for the padding ids of the last share.
__device__ __forceinline__ bool swa_xcd_unit(int n_blk, int H, int B, int& blk, int& hk, long& b) {
  const int total = n_blk * H * B;
  const int per_xcd = (total + 7) / 8;
  const int vid = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
  if (vid >= total) return false;
  const int unit = vid / n_blk;
  blk = vid - unit * n_blk;
  hk = unit % H;
  b = unit / H;
  return true;
}
static dim3 swa_xcd_grid(int n_blk, int H, int B) { return dim3((unsigned)(((long)n_blk * H * B + 7) / 8 * 8)); }

// Forward.  A workgroup of NWV wavefronts owns NWV*32/G consecutive queries of one KV head: 32 score
// rows (query x head of the group) per wavefront, held as matrix B operands.  The keys and values the
// block can see (its queries' windows: two or three 64-token tiles at window 64) are loaded once, all
// loads in flight together, and stay in LDS row-major (rows padded by 16 bytes); a longer window is
// worked through in phases of RES resident tiles.  S^T = K Q^T takes K rows as A operands, O += P V takes V
// through the transposing LDS load, in the token order in which the S^T accumulators hold P.  A
// wavefront skips the tiles none of its rows can see and masks only the tiles that straddle a row's
// window start, its diagonal, the end of the keys or a landmark; running max / sum per row as in
// flash attention.
// Two shapes of workgroup.  Wide: eight wavefronts, four resident tiles (139 KiB of LDS at D = Dv =
// 128, one workgroup per compute unit: its load, compute and store phases follow each other with
// nothing to overlap them).  Narrow: four wavefronts, two resident tiles (70 KiB), two workgroups per
// compute unit, one loading while the other computes; taken when no block of 128/G queries needs more
// than two tiles (window <= 64 at chunk 64), at the price of every tile being staged by twice as many
// workgroups (L2 hits).
#define SWA_FWD_RT 2   // 16-row tiles per wavefront
#define SWA_LAZY 6.f   // log2 of the growth of a row's maximum that moves its reference point

template <int D, int DV, int NWV, int RES>
static size_t swa_fwd_smem() {
  const size_t tiles = (size_t)RES * 64 * ((2 * D + 16) + (2 * DV + 16));
  const size_t outs = (size_t)NWV * 16 * SWA_FWD_RT * (2 * DV + 16);
  return (tiles > outs ? tiles : outs) + (size_t)NWV * SWA_FWD_RT * 16 * sizeof(float);
}

template <int D, int DV, int G, int NWV, int RES>
__global__ void __launch_bounds__(NWV * 64) __attribute__((amdgpu_waves_per_eu(2)))
swa_fwd_blk(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
            bf16_t* __restrict__ o, float* __restrict__ lse, SwaDims dm, int n_qt, int n_b) {
  constexpr int RT = SWA_FWD_RT, NT = NWV * 64;
  constexpr int KS = D / 32, DT = DV / 16;
  constexpr int QW = 16 * RT / G > 0 ? 16 * RT / G : 1;  // queries per wavefront (G <= 16: >= 2)
  constexpr int QB = NWV * 16 * RT / G;                  // queries per workgroup
  constexpr int KP = D * 2 + 16, VP = DV * 2 + 16;       // bytes per staged row
  constexpr int KSEG = D / 8, VSEG = DV / 8;
  constexpr int KPT = 64 * KSEG / NT, VPT = 64 * VSEG / NT;  // 16-byte pieces per thread and tile
  static_assert(KPT >= 1 && VPT >= 1 && KPT * NT == 64 * KSEG && VPT * NT == 64 * VSEG,
                "every thread stages whole pieces of a tile");
  constexpr int TILE_B = 64 * KP + 64 * VP;
  constexpr int OP = DV * 2 + 16;  // bytes per staged output row
  typedef unsigned swa_u32x4 __attribute__((ext_vector_type(4)));
  typedef short swa_s4 __attribute__((ext_vector_type(4)));
  typedef short swa_s8 __attribute__((ext_vector_type(8)));
  extern __shared__ __align__(16) unsigned char swa_dyn[];
  constexpr size_t TILES_B = (size_t)RES * TILE_B;
  constexpr size_t OUTS_B = (size_t)NWV * 16 * RT * OP;
  float* bc_all = (float*)(swa_dyn + (TILES_B > OUTS_B ? TILES_B : OUTS_B));  // [wave][rt][16] row factors
  const int tid = threadIdx.x, lane = tid & 63;
  // in a scalar register: what is derived from it (the wavefront's key range, "does this tile need
  // masks") then steers scalar branches instead of lane masks
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, j = lane >> 4;
  float* bc_s = bc_all + wave * RT * 16;
  int qt, hk;
  long b;
  if (!swa_xcd_unit(n_qt, dm.H, n_b, qt, hk, b)) return;
  qt = n_qt - 1 - qt;
  const int tq0 = qt * QB;
  const int t0 = tq0 + wave * QW;
  const int q_off = dm.kv_start + dm.Lk - dm.Lq;  // absolute position of query 0

  bf16x8_t qa[RT][KS];
  int qabs[RT], cstart[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = rt * 16 + col;
    const int t = t0 + row / G, g = row % G;
    const int tc = t < dm.Lq ? t : dm.Lq - 1;
    qabs[rt] = t < dm.Lq ? q_off + t : -2147483647;  // dead rows see nothing
    const int left = q_off + tc - dm.window + 1;
    cstart[rt] = dm.expand ? floordiv(left, dm.chunk) * dm.chunk : left;
    const bf16_t* qp = q + ((b * dm.Lq + tc) * (long)dm.HQ + hk * G + g) * D + j * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qa[rt][ks] = *(const bf16x8_t*)(qp + ks * 32);
  }
  // visible key positions of this lane's rows as [vlo, vlo + vspan]; a row that sees nothing gets a
  // start no position reaches
  int vlo[RT];
  unsigned vspan[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int last = dm.kv_start + dm.Lk - 1;
    const int hi = qabs[rt] < last ? qabs[rt] : last;
    const bool some = hi >= cstart[rt];
    vlo[rt] = some ? cstart[rt] : 0x7fffffff;
    vspan[rt] = some ? (unsigned)(hi - cstart[rt]) : 0u;
  }
  auto win_lo = [&](int t) -> int {  // first raw key index query t can see (may be negative)
    const int left = q_off + t - dm.window + 1;
    return (dm.expand ? floordiv(left, dm.chunk) * dm.chunk : left) - dm.kv_start;
  };
  // key range of the workgroup and of this wavefront (raw indices into k / v)
  int tile_lo, tile_hi;
  {
    int tq1 = tq0 + QB - 1;
    if (tq1 > dm.Lq - 1) tq1 = dm.Lq - 1;
    int lo = win_lo(tq0), hi = q_off + tq1 - dm.kv_start + 1;
    lo = lo < 0 ? 0 : lo;
    hi = hi > dm.Lk ? dm.Lk : hi;
    tile_lo = lo / 64;
    tile_hi = (hi + 63) / 64;  // may be <= tile_lo: nothing visible
  }
  int w_lo, w_hi, w_in_lo, w_in_hi;  // the wavefront's visible range and the part of it no row masks
  {
    const int ta = t0 < dm.Lq ? t0 : dm.Lq - 1;
    int tb = t0 + (16 * RT - 1) / G;
    tb = tb < dm.Lq ? tb : dm.Lq - 1;
    w_lo = win_lo(ta);
    w_hi = q_off + tb - dm.kv_start + 1;
    w_in_lo = win_lo(tb);                     // every row sees keys from here ...
    w_in_hi = q_off + ta - dm.kv_start + 1;   // ... up to (excluding) here
    if (w_in_hi > dm.Lk) w_in_hi = dm.Lk;
    if (t0 >= dm.Lq) w_hi = w_lo;             // a wavefront of dead rows
  }
  const float c2 = dm.sm_scale * HILS_LOG2E;

  f32x4_t acc[RT][DT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[rt][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run[RT], l_run[RT];  // running max (raw score units) and sum, per row (lane & 15)
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    m_run[rt] = HILS_NEG_INF;
    l_run[rt] = 0.f;
  }

  // one resident tile: scores, masks where a row needs them, running softmax, O += P V
  auto tile_step = [&](int tile, const unsigned char* k_s, const unsigned char* v_s) __attribute__((always_inline)) {
    f32x4_t p[RT][4];  // scores, then probabilities: accumulator tiles (token tt*16 + 4j + i, row lane & 15)
    bool rescale = false;
    {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) p[rt][tt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int tt = 0; tt < 4; ++tt)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8_t a = *(const bf16x8_t*)(k_s + (tt * 16 + col) * KP + ks * 64 + j * 16);
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            p[rt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qa[rt][ks], p[rt][tt], 0, 0, 0);
          // (keeps the operand reads of later steps from being hoisted here: registers)
          if (ks == KS - 1 && (tt & 1)) __builtin_amdgcn_sched_barrier(0);
        }
      const bool inner = !dm.mask_lmk && tile * 64 >= w_in_lo && tile * 64 + 64 <= w_in_hi;  // uniform
      if (!inner) {
        // a token at absolute position ta is visible to a row iff vlo <= ta <= vhi (window start, the
        // query itself or the last key): one unsigned compare of ta - vlo against vhi - vlo, no branches
        const int tok_abs0 = dm.kv_start + tile * 64 + 4 * j;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          const unsigned base = (unsigned)(tok_abs0 - vlo[rt]);
#pragma unroll
          for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              p[rt][tt][i] = (base + (unsigned)(tt * 16 + i) <= vspan[rt]) ? p[rt][tt][i] : HILS_NEG_INF;
        }
        // landmarks (the last position of every chunk) in a pass of their own behind a uniform branch:
        // the test does not depend on the row, and the common call masks none
        if (dm.mask_lmk) {
#pragma unroll
          for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int ta = tok_abs0 + tt * 16 + i + 1;
              const bool lm = dm.chunk_pow2 ? ((ta & (dm.chunk - 1)) == 0) : (ta % dm.chunk == 0);
#pragma unroll
              for (int rt = 0; rt < RT; ++rt) p[rt][tt][i] = lm ? HILS_NEG_INF : p[rt][tt][i];
            }
        }
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        float mx = HILS_NEG_INF;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
          for (int i = 0; i < 4; ++i) mx = fmaxf(mx, p[rt][tt][i]);
        mx = rows_max(mx);
        // The reference point of the exponentials follows the running maximum only when that grows by
        // more than 2^SWA_LAZY (or when the row has nothing accumulated yet): until then probabilities
        // up to 2^SWA_LAZY enter sum and output alike, which the final division cancels, and the
        // output accumulators need no rescaling (most tiles: the branch below is wavefront-uniform).
        const bool fresh = l_run[rt] == 0.f;
        const bool move = fresh | ((mx - m_run[rt]) * c2 > SWA_LAZY);
        const float m_new = move ? fmaxf(m_run[rt], mx) : m_run[rt];
        const bool any = m_new > HILS_NEG_INF;
        const float corr = (move & any & !fresh) ? __builtin_amdgcn_exp2f((m_run[rt] - m_new) * c2) : 1.f;
        const float mc = any ? m_new * c2 : 0.f;
        rescale |= corr != 1.f;
        float sum = 0.f;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float e = __builtin_amdgcn_exp2f(fmaf(p[rt][tt][i], c2, -mc));  // masked: exp2(-inf) = 0
            p[rt][tt][i] = e;
            sum += e;
          }
        sum = rows_sum(sum);
        l_run[rt] = l_run[rt] * corr + sum;
        m_run[rt] = m_new;
        if (j == 0) bc_s[rt * 16 + col] = corr;
      }
    }
    __builtin_amdgcn_wave_barrier();
    // rescale the output accumulators: their rows are 4j+i, the factors live per lane & 15
    if (__any(rescale)) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const float4 c4 = *(const float4*)&bc_s[rt * 16 + 4 * j];
        const float cf[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[rt][dt][i] *= cf[i];
      }
    }
    __builtin_amdgcn_wave_barrier();
    // O += P V: a lane's eight k-slots are tokens 4j..4j+3 of two neighbouring 16-token tiles; the
    // transposing load (a 16-lane group addresses a 4 x 16 block, lane l row l/4 and columns 4(l%4)..,
    // and receives column l of it) delivers V in that order
    const unsigned char* t_addr = v_s + (4 * j + (col >> 2)) * VP + (col & 3) * 8;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      bf16x8_t a[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        swa_u32x4 u;
        u.x = pack_bf2(p[rt][2 * h][0], p[rt][2 * h][1]);
        u.y = pack_bf2(p[rt][2 * h][2], p[rt][2 * h][3]);
        u.z = pack_bf2(p[rt][2 * h + 1][0], p[rt][2 * h + 1][1]);
        u.w = pack_bf2(p[rt][2 * h + 1][2], p[rt][2 * h + 1][3]);
        a[rt] = __builtin_bit_cast(bf16x8_t, u);
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const unsigned char* p0 = t_addr + (2 * h * 16) * VP + dt * 32;
        const swa_s4 b0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) swa_s4*)p0);
        const swa_s4 b1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) swa_s4*)(p0 + 16 * VP));
        const swa_s8 bb = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          acc[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt], __builtin_bit_cast(bf16x8_t, bb), acc[rt][dt], 0, 0, 0);
        if ((dt & 3) == 3) __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // loads of a phase of N resident tiles, two tiles in flight (tokens past the end read the last row:
  // their scores are masked); one copy of the code per N, so no load is conditional
  auto phase = [&](int tile0, auto n_const) __attribute__((always_inline)) {
    constexpr int N = decltype(n_const)::value;
    swa_u32x4 kr[2][KPT], vr[2][VPT];  // two tiles' loads in flight
    auto issue = [&](int ti, swa_u32x4 (&kd)[KPT], swa_u32x4 (&vd)[VPT]) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        const int pc = tid + NT * i;
        int tok = (tile0 + ti) * 64 + pc / KSEG;
        tok = tok < dm.Lk ? tok : dm.Lk - 1;
        kd[i] = *(const swa_u32x4*)(k + ((b * dm.Lk + tok) * (long)dm.H + hk) * D + (pc % KSEG) * 8);
      }
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int pc = tid + NT * i;
        int tok = (tile0 + ti) * 64 + pc / VSEG;
        tok = tok < dm.Lk ? tok : dm.Lk - 1;
        vd[i] = *(const swa_u32x4*)(v + ((b * dm.Lk + tok) * (long)dm.H + hk) * DV + (pc % VSEG) * 8);
      }
    };
    auto stash = [&](int ti, const swa_u32x4 (&kd)[KPT], const swa_u32x4 (&vd)[VPT]) __attribute__((always_inline)) {
      unsigned char* k_s = swa_dyn + (size_t)ti * TILE_B;
      unsigned char* v_s = k_s + 64 * KP;
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        const int pc = tid + NT * i;
        *(swa_u32x4*)(k_s + (pc / KSEG) * KP + (pc % KSEG) * 16) = kd[i];
      }
#pragma unroll
      for (int i = 0; i < VPT; ++i) {
        const int pc = tid + NT * i;
        *(swa_u32x4*)(v_s + (pc / VSEG) * VP + (pc % VSEG) * 16) = vd[i];
      }
    };
    issue(0, kr[0], vr[0]);
    if (N > 1) issue(1, kr[1], vr[1]);
#pragma unroll
    for (int ti = 0; ti < N; ++ti) {
      stash(ti, kr[ti & 1], vr[ti & 1]);
      if (ti + 2 < N) issue(ti + 2, kr[ti & 1], vr[ti & 1]);
    }
  };
  for (int tile0 = tile_lo; tile0 < tile_hi; tile0 += RES) {
    if (tile0 != tile_lo) __syncthreads();  // the previous phase's tiles are no longer read
    const int n = tile_hi - tile0 < RES ? tile_hi - tile0 : RES;
    if (RES >= 4 && n == 4) phase(tile0, std::integral_constant<int, RES >= 4 ? 4 : 1>{});
    else if (RES >= 3 && n == 3) phase(tile0, std::integral_constant<int, RES >= 3 ? 3 : 1>{});
    else if (n == 2) phase(tile0, std::integral_constant<int, 2>{});
    else phase(tile0, std::integral_constant<int, 1>{});
    __syncthreads();
    for (int ti = 0; ti < n; ++ti) {  // one copy of the tile code
      const int tile = tile0 + ti;
      if (tile * 64 < w_hi && tile * 64 + 64 > w_lo) {  // uniform: some row of the wavefront sees the tile
        const unsigned char* k_s = swa_dyn + (size_t)ti * TILE_B;
        tile_step(tile, k_s, k_s + 64 * KP);
      }
    }
  }
  // ---- finalize: o = acc / l, lse = ln(l) + max * scale ----
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float inv = l_run[rt] > 0.f ? 1.f / l_run[rt] : 0.f;
    if (j == 0) bc_s[rt * 16 + col] = inv;
    const int row = rt * 16 + col;
    const int t = t0 + row / G, g = row % G;
    if (j == 0 && t < dm.Lq)
      lse[(b * dm.Lq + t) * (long)dm.HQ + hk * G + g] =
          l_run[rt] > 0.f ? (m_run[rt] * c2 + __builtin_amdgcn_logf(l_run[rt])) * HILS_LN2 : HILS_NEG_INF;
  }
  __syncthreads();  // every wavefront is through with the tiles: their LDS becomes the output stage
  // Each wavefront parks its normalised rows as bf16 and writes them out as 16-byte pieces (a query's
  // heads are contiguous).
  unsigned char* ob = swa_dyn + (size_t)wave * (16 * RT) * OP;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float4 c4 = *(const float4*)&bc_s[rt * 16 + 4 * j];
    const float cf[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        *(bf16_t*)(ob + (rt * 16 + 4 * j + i) * OP + (dt * 16 + col) * 2) = f2bf(acc[rt][dt][i] * cf[i]);
  }
  __builtin_amdgcn_wave_barrier();
  constexpr int OSEG = DV / 8;
#pragma unroll
  for (int pp = 0; pp < 16 * RT * OSEG / 64; ++pp) {
    const int pc = pp * 64 + lane;
    const int row = pc / OSEG, seg = pc % OSEG;
    const int t = t0 + row / G, g = row % G;
    if (t < dm.Lq)
      *(uint4*)(o + ((b * dm.Lq + t) * (long)dm.HQ + hk * G + g) * DV + seg * 8) = *(const uint4*)(ob + row * OP + seg * 16);
  }
}

// ---- backward (training: Lq == Lk, kv_start == 0) -------------------------------------------
//   P = exp(s - lse),  dP = dO V^T,  delta = sum_d o*dO - d_lse,  dS = P (dP - delta) * scale
//   dQ = dS K,  dK = dS^T Q,  dV = P^T dO.
// Same split as the forward: one side owned by a wavefront in registers, the other streamed
// through LDS in 64-row tiles (row-major for the score-like products, transposed for the
// gradient products).

// visibility bits of this lane's landmark test for the 16 tokens tt*16 + 4j + i of a 64-token tile
__device__ __forceinline__ unsigned swa_lmk_bits(const SwaDims& dm, int tok0) {
  if (!dm.mask_lmk) return 0xffffu;
  unsigned ok = 0u;
#pragma unroll
  for (int tt = 0; tt < 4; ++tt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ta = tok0 + tt * 16 + i + 1;
      const bool lm = dm.chunk_pow2 ? ((ta & (dm.chunk - 1)) == 0) : (ta % dm.chunk == 0);
      ok |= lm ? 0u : (1u << (tt * 4 + i));
    }
  return ok;
}

// 16-row tiles per wavefront of the backward kernels: two for narrow heads; one for wide heads, whose two
// tiles need more than 256 registers (one wavefront per SIMD, nothing to overlap a wait with)
constexpr int swa_dq_rt(int D, int DV) { return (D <= 64 && DV <= 64) ? 2 : 1; }

// dQ (and delta): a wavefront owns 16 * RT score rows; K (row-major and transposed) and V stream.
template <int D, int DV, int G>
// (the hint keeps the accumulators out of accumulation registers; wide heads with their one tile per
// wavefront are held to 168 registers, five spilled dwords, for three wavefronts per SIMD: 52 KiB of LDS
// let three workgroups share a compute unit)
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((D > 64 && DV > 64) ? 3 : 2)))
swa_bwd_dq_mfma(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
                const bf16_t* __restrict__ o, const float* __restrict__ lse,
                const bf16_t* __restrict__ d_o, const float* __restrict__ d_lse,
                bf16_t* __restrict__ dq, float* __restrict__ delta_out, SwaDims dm, int n_qt, int n_b) {
  constexpr int RT = swa_dq_rt(D, DV);
  constexpr int KS = D / 32, VS = DV / 32, DT = D / 16;
  constexpr int QW = 16 * RT / G > 0 ? 16 * RT / G : 1, QB = 4 * 16 * RT / G;
  constexpr int PITCH = D * 2 + 16, VPITCH = DV * 2 + 16;
  constexpr int KSEG = D / 8, KPPP = 256 / KSEG, KPASS = 32 / KPPP;
  constexpr int VSEG = DV / 8, VPASS = 64 * VSEG / 256;
  __shared__ __align__(16) unsigned char k_s[64 * PITCH];
  __shared__ __align__(16) unsigned char kt_s[D * LZM_PT];
  __shared__ __align__(16) unsigned char v_s[64 * VPITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, j = lane >> 4;
  int qt, hk;
  long b;
  if (!swa_xcd_unit(n_qt, dm.H, n_b, qt, hk, b)) return;
  qt = n_qt - 1 - qt;
  const int t0 = qt * QB + wave * QW;
  const int L = dm.Lq;

  bf16x8_t qa[RT][KS], doa[RT][VS];
  int qabs[RT], cstart[RT];
  float lse2[RT], delta[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = rt * 16 + col;
    const int t = t0 + row / G, g = row % G;
    const int tc = t < L ? t : L - 1;
    const long rix = (b * L + tc) * (long)dm.HQ + hk * G + g;
    const float ls = lse[rix];
    const bool live = t < L && ls > -1e30f;  // rows that saw no key have no gradient
    qabs[rt] = live ? t : -2147483647;
    const int left = tc - dm.window + 1;
    cstart[rt] = dm.expand ? floordiv(left, dm.chunk) * dm.chunk : left;
    lse2[rt] = live ? ls * HILS_LOG2E : 0.f;
    const bf16_t* qp = q + rix * D + j * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qa[rt][ks] = *(const bf16x8_t*)(qp + ks * 32);
    float part = 0.f;
#pragma unroll
    for (int vs = 0; vs < VS; ++vs) {
      const uint4 dv4 = *(const uint4*)(d_o + rix * DV + vs * 32 + j * 8);
      const uint4 ov4 = *(const uint4*)(o + rix * DV + vs * 32 + j * 8);
      doa[rt][vs] = *(const bf16x8_t*)&dv4;
      float a[8], c[8];
      unpack8(dv4, a);
      unpack8(ov4, c);
#pragma unroll
      for (int e = 0; e < 8; ++e) part = fmaf(a[e], c[e], part);
    }
    part = rows_sum(part);
    delta[rt] = part - (d_lse ? d_lse[rix] : 0.f);
    if (j == 0 && t < L) delta_out[rix] = delta[rt];
  }
  int vlo[RT];
  unsigned vspan[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const bool some = qabs[rt] >= cstart[rt];
    vlo[rt] = some ? cstart[rt] : 0x7fffffff;
    vspan[rt] = some ? (unsigned)(qabs[rt] - cstart[rt]) : 0u;
  }
  int tile_lo, tile_hi;
  {
    const int tq0 = qt * QB;
    int tq1 = tq0 + QB - 1;
    if (tq1 > L - 1) tq1 = L - 1;
    const int left_abs = tq0 - dm.window + 1;
    int lo = dm.expand ? floordiv(left_abs, dm.chunk) * dm.chunk : left_abs;
    lo = lo < 0 ? 0 : lo;
    tile_lo = lo / 64;
    tile_hi = tq1 / 64 + 1;
  }
  const float c2 = dm.sm_scale * HILS_LOG2E;

  // prefetch registers as in the forward kernel: native vectors, loads without branches, tokens
  // past the end read the last row (their probabilities are masked to 0)
  typedef unsigned swa_u32x4 __attribute__((ext_vector_type(4)));
  swa_u32x4 kr[KPASS][2], vr[VPASS];
  auto as_uint4 = [](const swa_u32x4& x) { return make_uint4(x.x, x.y, x.z, x.w); };
  auto fetch = [&](int tile) {
#pragma unroll
    for (int i = 0; i < KPASS; ++i)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        int tok = tile * 64 + 2 * (tid / KSEG + KPPP * i) + h;
        tok = tok < L ? tok : L - 1;
        kr[i][h] = *(const swa_u32x4*)(k + ((b * L + tok) * (long)dm.H + hk) * D + (tid % KSEG) * 8);
      }
#pragma unroll
    for (int i = 0; i < VPASS; ++i) {
      const int p = tid + 256 * i;
      int tok = tile * 64 + p / VSEG;
      tok = tok < L ? tok : L - 1;
      vr[i] = *(const swa_u32x4*)(v + ((b * L + tok) * (long)dm.H + hk) * DV + (p % VSEG) * 8);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < KPASS; ++i)
      lzm_stash_pair<PITCH>(k_s, kt_s, 2 * (tid / KSEG + KPPP * i), tid % KSEG, as_uint4(kr[i][0]), as_uint4(kr[i][1]));
#pragma unroll
    for (int i = 0; i < VPASS; ++i) {
      const int p = tid + 256 * i;
      *(swa_u32x4*)(v_s + (p / VSEG) * VPITCH + (p % VSEG) * 16) = vr[i];
    }
  };
  f32x4_t acc[RT][DT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[rt][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  fetch(tile_lo);
  stash();
  __syncthreads();
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    fetch(tile + 1 < tile_hi ? tile + 1 : tile);
    float ds[RT][4][4];
    {
      f32x4_t st[RT][4], dp[RT][4];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
          st[rt][tt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
          dp[rt][tt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8_t a = *(const bf16x8_t*)(k_s + (tt * 16 + col) * PITCH + ks * 64 + j * 16);
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            st[rt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qa[rt][ks], st[rt][tt], 0, 0, 0);
        }
#pragma unroll
        for (int vs = 0; vs < VS; ++vs) {
          const bf16x8_t a = *(const bf16x8_t*)(v_s + (tt * 16 + col) * VPITCH + vs * 64 + j * 16);
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            dp[rt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, doa[rt][vs], dp[rt][tt], 0, 0, 0);
        }
      }
      // token ta is visible to a row iff window start <= ta <= query: one unsigned compare of
      // ta - start against query - start (a dead row has a start no token reaches)
      const int tok0 = tile * 64 + 4 * j;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const unsigned base = (unsigned)(tok0 - vlo[rt]);
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const bool vis = base + (unsigned)(tt * 16 + i) <= vspan[rt];
            const float pv = vis ? __builtin_amdgcn_exp2f(st[rt][tt][i] * c2 - lse2[rt]) : 0.f;
            ds[rt][tt][i] = pv * (dp[rt][tt][i] - delta[rt]) * dm.sm_scale;
          }
      }
      if (dm.mask_lmk) {  // landmarks in a pass of their own behind a uniform branch (row-independent)
        const unsigned lmk_ok = swa_lmk_bits(dm, tok0);
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const bool ok = ((lmk_ok >> (tt * 4 + i)) & 1u) != 0u;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) ds[rt][tt][i] = ok ? ds[rt][tt][i] : 0.f;
          }
      }
    }
    lzm_grad_product<D, RT>(kt_s, ds, acc, col, j);
    __syncthreads();
    stash();
    __syncthreads();
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = rt * 16 + 4 * j + i;
      const int t = t0 + row / G, g = row % G;
      if (t >= L) continue;
      bf16_t* out = dq + ((b * L + t) * (long)dm.HQ + hk * G + g) * D + col;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) out[dt * 16] = f2bf(acc[rt][dt][i]);
    }
}

// dK, dV: a workgroup owns 64 * TT tokens of one KV head (TT 16-token tiles per wavefront, as matrix B
// operands: two for narrow heads, one for wide heads, whose two tiles need more than 256 registers); the
// score rows (query x head) that can see them stream in tiles of 64 rows, Q and dO both row-major
// and transposed, with the rows' lse, delta and window start beside them.
template <int D, int DV, int G>
// (the hint gives two wavefronts per SIMD and keeps the accumulators out of accumulation registers)
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
swa_bwd_dkdv_mfma(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                  const bf16_t* __restrict__ v, const float* __restrict__ lse,
                  const bf16_t* __restrict__ d_o, const float* __restrict__ delta_in,
                  bf16_t* __restrict__ dk, bf16_t* __restrict__ dv, SwaDims dm, int n_kb, int n_b) {
  constexpr int TT = swa_dq_rt(D, DV);
  constexpr int KS = D / 32, VS = DV / 32, DT = D / 16, DVT = DV / 16;
  constexpr int QT = 64 / G;
  constexpr int PITCH = D * 2 + 16, VPITCH = DV * 2 + 16;
  constexpr int QSEG = D / 8, QPPP = 256 / QSEG, QPASS = 32 / QPPP;
  constexpr int OSEG = DV / 8, OPPP = 256 / OSEG, OPASS = 32 / OPPP;
  extern __shared__ __align__(16) unsigned char dyn[];
  unsigned char* q_s = dyn;                       // 64 * PITCH
  unsigned char* qt_s = q_s + 64 * PITCH;         // D * LZM_PT
  unsigned char* do_s = qt_s + D * LZM_PT;        // 64 * VPITCH
  unsigned char* dot_s = do_s + 64 * VPITCH;      // DV * LZM_PT
  float* lse_s = (float*)(dot_s + DV * LZM_PT);   // 64
  float* del_s = lse_s + 64;                      // 64
  int* cs_s = (int*)(del_s + 64);                 // 64: window start of the row (INT_MAX: dead row)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, j = lane >> 4;
  int kb, hk;
  long b;
  if (!swa_xcd_unit(n_kb, dm.H, n_b, kb, hk, b)) return;
  const int L = dm.Lq;
  const int j0 = kb * (64 * TT);
  const int tok_w = j0 + wave * (16 * TT);  // first owned token of the wavefront

  bf16x8_t ka[TT][KS], va[TT][VS];
  unsigned lmk_ok = 0u;  // bit tt: owned token tt*16 + col is not a landmark
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
    const int tok = tok_w + tt * 16 + col;
    const int tc = tok < L ? tok : L - 1;  // tokens past the end are never visible
    const bf16_t* kp = k + ((b * L + tc) * (long)dm.H + hk) * D + j * 8;
    const bf16_t* vp = v + ((b * L + tc) * (long)dm.H + hk) * DV + j * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ka[tt][ks] = *(const bf16x8_t*)(kp + ks * 32);
#pragma unroll
    for (int vs = 0; vs < VS; ++vs) va[tt][vs] = *(const bf16x8_t*)(vp + vs * 32);
    const bool lm = dm.mask_lmk && (dm.chunk_pow2 ? (((tok + 1) & (dm.chunk - 1)) == 0) : ((tok + 1) % dm.chunk == 0));
    if (!lm && tok < L) lmk_ok |= 1u << tt;
  }
  // owned token of this lane per tile, or a position far below every window for a landmark / a
  // token past the end
  int tokv[TT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) tokv[tt] = ((lmk_ok >> tt) & 1u) ? tok_w + tt * 16 + col : -(1 << 30);
  // queries that can see a token of [j0, j1]: j0 <= t <= (last window that starts at or before j1)
  int j1 = j0 + 64 * TT - 1;
  if (j1 > L - 1) j1 = L - 1;
  long t_hi = dm.expand ? ((long)(j1 / dm.chunk) + 1) * dm.chunk + dm.window - 2 : (long)j1 + dm.window - 1;
  if (t_hi > L - 1) t_hi = L - 1;
  const int tile0 = j0 / QT;
  const int n_tiles = (int)(t_hi / QT) + 1;
  const float c2 = dm.sm_scale * HILS_LOG2E;

  uint4 qr[QPASS][2], dor[OPASS][2];
  float r_lse = 0.f, r_del = 0.f;
  int r_cs = 2147483647;
  auto fetch = [&](int tile) {
#pragma unroll
    for (int i = 0; i < QPASS; ++i)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int row = 2 * (tid / QSEG + QPPP * i) + h;
        int t = tile * QT + row / G;
        if (t > L - 1) t = L - 1;
        qr[i][h] = *(const uint4*)(q + ((b * L + t) * (long)dm.HQ + hk * G + row % G) * D + (tid % QSEG) * 8);
      }
#pragma unroll
    for (int i = 0; i < OPASS; ++i)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int row = 2 * (tid / OSEG + OPPP * i) + h;
        int t = tile * QT + row / G;
        if (t > L - 1) t = L - 1;
        dor[i][h] = *(const uint4*)(d_o + ((b * L + t) * (long)dm.HQ + hk * G + row % G) * DV + (tid % OSEG) * 8);
      }
    if (tid < 64) {
      const int t = tile * QT + tid / G;
      const int tc = t < L ? t : L - 1;
      const long rix = (b * L + tc) * (long)dm.HQ + hk * G + tid % G;
      r_lse = lse[rix];  // raw: what a dead row gets is decided in stash(), nothing waits for a load here
      r_del = delta_in[rix];
      const int left = tc - dm.window + 1;
      r_cs = t < L ? (dm.expand ? floordiv(left, dm.chunk) * dm.chunk : left) : 2147483647;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < QPASS; ++i)
      lzm_stash_pair<PITCH>(q_s, qt_s, 2 * (tid / QSEG + QPPP * i), tid % QSEG, qr[i][0], qr[i][1]);
#pragma unroll
    for (int i = 0; i < OPASS; ++i)
      lzm_stash_pair<VPITCH>(do_s, dot_s, 2 * (tid / OSEG + OPPP * i), tid % OSEG, dor[i][0], dor[i][1]);
    if (tid < 64) {
      const bool live = r_lse > -1e30f;  // rows with an empty window have lse = -inf
      lse_s[tid] = live ? r_lse * HILS_LOG2E : 0.f;
      del_s[tid] = r_del;
      cs_s[tid] = live ? r_cs : 2147483647;
    }
  };
  f32x4_t acck[TT][DT], accv[TT][DVT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acck[tt][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt) accv[tt][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  fetch(tile0);
  stash();
  __syncthreads();
  for (int tile = tile0; tile < n_tiles; ++tile) {
    fetch(tile + 1 < n_tiles ? tile + 1 : tile);
    float p[TT][4][4], ds[TT][4][4];  // [owned token tile][streamed row tile][row 4j+i]
    {
      f32x4_t st[TT][4], dp[TT][4];
#pragma unroll
      for (int tt = 0; tt < TT; ++tt)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          st[tt][rr] = f32x4_t{0.f, 0.f, 0.f, 0.f};
          dp[tt][rr] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8_t a = *(const bf16x8_t*)(q_s + (rr * 16 + col) * PITCH + ks * 64 + j * 16);
#pragma unroll
          for (int tt = 0; tt < TT; ++tt)
            st[tt][rr] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, ka[tt][ks], st[tt][rr], 0, 0, 0);
        }
#pragma unroll
        for (int vs = 0; vs < VS; ++vs) {
          const bf16x8_t a = *(const bf16x8_t*)(do_s + (rr * 16 + col) * VPITCH + vs * 64 + j * 16);
#pragma unroll
          for (int tt = 0; tt < TT; ++tt)
            dp[tt][rr] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, va[tt][vs], dp[tt][rr], 0, 0, 0);
        }
      }
      const int tq0 = tile * QT;
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const float4 l4 = *(const float4*)&lse_s[rr * 16 + 4 * j];
        const float4 d4 = *(const float4*)&del_s[rr * 16 + 4 * j];
        const int4 c4 = *(const int4*)&cs_s[rr * 16 + 4 * j];
        const float ls[4] = {l4.x, l4.y, l4.z, l4.w}, dl[4] = {d4.x, d4.y, d4.z, d4.w};
        const int cs[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // window start <= token <= query as one unsigned compare of query - token against
          // query - start + 1 (0 for a dead row, whose start no query reaches)
          const int t = tq0 + (rr * 16 + 4 * j + i) / G;
          const unsigned span1 = t >= cs[i] ? (unsigned)(t - cs[i]) + 1u : 0u;
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) {
            const bool vis = (unsigned)(t - tokv[tt]) < span1;
            const float pv = vis ? __builtin_amdgcn_exp2f(st[tt][rr][i] * c2 - ls[i]) : 0.f;
            p[tt][rr][i] = pv;
            ds[tt][rr][i] = pv * (dp[tt][rr][i] - dl[i]) * dm.sm_scale;
          }
        }
      }
    }
    lzm_grad_product<DV, TT>(dot_s, p, accv, col, j);
    lzm_grad_product<D, TT>(qt_s, ds, acck, col, j);
    __syncthreads();
    stash();
    __syncthreads();
  }
#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tok = tok_w + tt * 16 + 4 * j + i;
      if (tok >= L) continue;
      bf16_t* outk = dk + ((b * L + tok) * (long)dm.H + hk) * D + col;
      bf16_t* outv = dv + ((b * L + tok) * (long)dm.H + hk) * DV + col;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) outk[dt * 16] = f2bf(acck[tt][dt][i]);
#pragma unroll
      for (int dt = 0; dt < DVT; ++dt) outv[dt * 16] = f2bf(accv[tt][dt][i]);
    }
}

template <int D, int DV, int G, int NWV, int RES>
static int swa_fwd_launch_shape(int B, hipStream_t st, const bf16_t* q, const bf16_t* k, const bf16_t* v,
                                bf16_t* o, float* lse, const SwaDims& dm) {
  const size_t smem = swa_fwd_smem<D, DV, NWV, RES>();
  auto kern = swa_fwd_blk<D, DV, G, NWV, RES>;
  static HilsLdsReserve reserved;  // per instantiation
  if (int rc = hils_reserve_lds(&reserved, (const void*)kern, smem, "hils_swa_fwd")) return rc;
  const int QB = NWV * 16 * SWA_FWD_RT / G;  // queries of a workgroup (>= 8: G <= 16)
  const int n_qt = (dm.Lq + QB - 1) / QB;
  hipLaunchKernelGGL(kern, swa_xcd_grid(n_qt, dm.H, B), dim3(NWV * 64), smem, st, q, k, v, o, lse, dm, n_qt, B);
  return HILS_OK;
}

// The most 64-token tiles a block of QB queries reads (over the last blocks: the first ones are
// clipped at key 0, and the pattern repeats with the alignment of blocks, chunks and tiles).
static int swa_fwd_block_tiles(const SwaDims& dm, int QB) {
  const int n_qt = (dm.Lq + QB - 1) / QB;
  const long q_off = (long)dm.kv_start + dm.Lk - dm.Lq;
  int most = 0;
  for (int qt = n_qt - 1; qt >= 0 && qt >= n_qt - 256; --qt) {
    const long tq0 = (long)qt * QB;
    long tq1 = tq0 + QB - 1;
    if (tq1 > dm.Lq - 1) tq1 = dm.Lq - 1;
    const long left = q_off + tq0 - dm.window + 1;
    long lo = dm.expand ? (left >= 0 ? left / dm.chunk : -((-left + dm.chunk - 1) / dm.chunk)) * dm.chunk : left;
    lo -= dm.kv_start;
    long hi = q_off + tq1 - dm.kv_start + 1;
    if (lo < 0) lo = 0;
    if (hi > dm.Lk) hi = dm.Lk;
    const int n = (int)((hi + 63) / 64 - lo / 64);
    if (n > most) most = n;
  }
  return most;
}

template <int D, int DV, int G>
static int swa_fwd_launch(int B, hipStream_t st, const bf16_t* q, const bf16_t* k, const bf16_t* v,
                          bf16_t* o, float* lse, const SwaDims& dm) {
  const int tiles = swa_fwd_block_tiles(dm, 4 * 16 * SWA_FWD_RT / G);
  if (tiles <= 2) return swa_fwd_launch_shape<D, DV, G, 4, 2>(B, st, q, k, v, o, lse, dm);
  // narrow heads: four resident tiles are 72 KiB, and two 4-wavefront workgroups fit a compute unit
  // where one 8-wavefront workgroup does (150 registers: three wavefronts per SIMD)
  if constexpr (D <= 64 && DV <= 64)
    if (tiles <= 4) return swa_fwd_launch_shape<D, DV, G, 4, 4>(B, st, q, k, v, o, lse, dm);
  return swa_fwd_launch_shape<D, DV, G, 8, 4>(B, st, q, k, v, o, lse, dm);
}

template <int D, int DV>
static int swa_launch_g(int G, int B, hipStream_t st, const bf16_t* q, const bf16_t* k,
                        const bf16_t* v, bf16_t* o, float* lse, const SwaDims& dm) {
  switch (G) {
    case 1: return swa_fwd_launch<D, DV, 1>(B, st, q, k, v, o, lse, dm);
    case 2: return swa_fwd_launch<D, DV, 2>(B, st, q, k, v, o, lse, dm);
    case 4: return swa_fwd_launch<D, DV, 4>(B, st, q, k, v, o, lse, dm);
    case 8: return swa_fwd_launch<D, DV, 8>(B, st, q, k, v, o, lse, dm);
    default: return swa_fwd_launch<D, DV, 16>(B, st, q, k, v, o, lse, dm);
  }
}

extern "C" int hils_swa_fwd(const void* q, const void* k, const void* v, void* o, float* lse, int B,
                            int Lq, int Lk, int HQ, int H, int D, int Dv, int window, int chunk,
                            int mask_lmk, int expand_to_chunk, int kv_start, float sm_scale,
                            void* stream) {
  HILS_REQUIRE(q && k && v && o && lse, "hils_swa_fwd: null pointer");
  HILS_REQUIRE(B > 0 && Lq > 0 && Lk > 0 && HQ > 0 && H > 0, "hils_swa_fwd: sizes must be positive");
  HILS_REQUIRE(Lq <= Lk, "hils_swa_fwd: Lq (%d) must not exceed Lk (%d)", Lq, Lk);
  HILS_REQUIRE(HQ % H == 0, "hils_swa_fwd: HQ (%d) must be a multiple of H (%d)", HQ, H);
  HILS_REQUIRE(window >= 1 && chunk >= 1, "hils_swa_fwd: window and chunk must be positive");
  HILS_REQUIRE(kv_start >= 0, "hils_swa_fwd: kv_start must not be negative");
  const int G = HQ / H;
  HILS_REQUIRE((D == 64 || D == 128) && (Dv == 64 || Dv == 128),
               "hils_swa_fwd: head dims (%d, %d) must be 64 or 128", D, Dv);
  HILS_REQUIRE(G == 1 || G == 2 || G == 4 || G == 8 || G == 16,
               "hils_swa_fwd: group size %d must be 1, 2, 4, 8 or 16", G);
  HILS_REQUIRE(((long)Lq / 8 + 1) * H * B < (1L << 31) - 8, "hils_swa_fwd: B * H * Lq too large for the grid");
  HILS_REQUIRE((long)kv_start + Lk < 2147483647L / 2, "hils_swa_fwd: positions overflow 32 bits");
  SwaDims dm{Lq, Lk, HQ, H, window, chunk, mask_lmk, expand_to_chunk, kv_start,
             (chunk & (chunk - 1)) == 0, sm_scale};
  hipStream_t st = (hipStream_t)stream;
  const bf16_t *qq = (const bf16_t*)q, *kk = (const bf16_t*)k, *vv = (const bf16_t*)v;
  int rc;
  if (D == 64 && Dv == 64) rc = swa_launch_g<64, 64>(G, B, st, qq, kk, vv, (bf16_t*)o, lse, dm);
  else if (D == 128 && Dv == 128) rc = swa_launch_g<128, 128>(G, B, st, qq, kk, vv, (bf16_t*)o, lse, dm);
  else if (D == 64) rc = swa_launch_g<64, 128>(G, B, st, qq, kk, vv, (bf16_t*)o, lse, dm);
  else rc = swa_launch_g<128, 64>(G, B, st, qq, kk, vv, (bf16_t*)o, lse, dm);
  if (rc) return rc;
  HILS_CHECK_LAUNCH("hils_swa_fwd");
  return HILS_OK;
}

template <int D, int DV, int G>
static int swa_bwd_launch(const bf16_t* q, const bf16_t* k, const bf16_t* v, const bf16_t* o,
                          const float* lse, const bf16_t* d_o, const float* d_lse, bf16_t* dq, bf16_t* dk,
                          bf16_t* dv, float* delta, int B, const SwaDims& dm, hipStream_t st) {
  const int QB = 4 * 16 * swa_dq_rt(D, DV) / G;
  const int n_qt = (dm.Lq + QB - 1) / QB;
  hipLaunchKernelGGL((swa_bwd_dq_mfma<D, DV, G>), swa_xcd_grid(n_qt, dm.H, B),
                     dim3(256), 0, st, q, k, v, o, lse, d_o, d_lse, dq, delta, dm, n_qt, B);
  const size_t smem = (size_t)64 * (D * 2 + 16) + (size_t)D * LZM_PT + (size_t)64 * (DV * 2 + 16) +
                      (size_t)DV * LZM_PT + 3 * 64 * sizeof(float);
  auto kern = swa_bwd_dkdv_mfma<D, DV, G>;
  static HilsLdsReserve reserved;  // per instantiation
  if (int rc = hils_reserve_lds(&reserved, (const void*)kern, smem, "hils_swa_bwd")) return rc;
  const int n_kb = (dm.Lq + 64 * swa_dq_rt(D, DV) - 1) / (64 * swa_dq_rt(D, DV));
  hipLaunchKernelGGL(kern, swa_xcd_grid(n_kb, dm.H, B), dim3(256), smem, st, q, k, v, lse, d_o, delta, dk, dv, dm,
                     n_kb, B);
  return HILS_OK;
}

template <int D, int DV>
static int swa_bwd_launch_g(int G, const bf16_t* q, const bf16_t* k, const bf16_t* v, const bf16_t* o,
                            const float* lse, const bf16_t* d_o, const float* d_lse, bf16_t* dq,
                            bf16_t* dk, bf16_t* dv, float* delta, int B, const SwaDims& dm, hipStream_t st) {
  switch (G) {
    case 1: return swa_bwd_launch<D, DV, 1>(q, k, v, o, lse, d_o, d_lse, dq, dk, dv, delta, B, dm, st);
    case 2: return swa_bwd_launch<D, DV, 2>(q, k, v, o, lse, d_o, d_lse, dq, dk, dv, delta, B, dm, st);
    case 4: return swa_bwd_launch<D, DV, 4>(q, k, v, o, lse, d_o, d_lse, dq, dk, dv, delta, B, dm, st);
    case 8: return swa_bwd_launch<D, DV, 8>(q, k, v, o, lse, d_o, d_lse, dq, dk, dv, delta, B, dm, st);
    default: return swa_bwd_launch<D, DV, 16>(q, k, v, o, lse, d_o, d_lse, dq, dk, dv, delta, B, dm, st);
  }
}

extern "C" int hils_swa_bwd(const void* q, const void* k, const void* v, const void* o, const float* lse,
                            const void* d_o, const float* d_lse, void* dq, void* dk, void* dv,
                            float* delta, int B, int L, int HQ, int H, int D, int Dv, int window,
                            int chunk, int mask_lmk, int expand_to_chunk, float sm_scale, void* stream) {
  HILS_REQUIRE(q && k && v && o && lse && d_o && dq && dk && dv && delta, "hils_swa_bwd: null pointer");
  HILS_REQUIRE(B > 0 && L > 0 && HQ > 0 && H > 0, "hils_swa_bwd: sizes must be positive");
  HILS_REQUIRE(HQ % H == 0, "hils_swa_bwd: HQ (%d) must be a multiple of H (%d)", HQ, H);
  HILS_REQUIRE(window >= 1 && chunk >= 1, "hils_swa_bwd: window and chunk must be positive");
  const int G = HQ / H;
  HILS_REQUIRE((D == 64 || D == 128) && (Dv == 64 || Dv == 128),
               "hils_swa_bwd: head dims (%d, %d) must be 64 or 128", D, Dv);
  HILS_REQUIRE(G == 1 || G == 2 || G == 4 || G == 8 || G == 16,
               "hils_swa_bwd: group size %d must be 1, 2, 4, 8 or 16", G);
  HILS_REQUIRE(((long)L / 8 + 1) * H * B < (1L << 31) - 8, "hils_swa_bwd: B * H * L too large for the grid");
  HILS_REQUIRE((long)L + window < 2147483647L / 2, "hils_swa_bwd: positions overflow 32 bits");
  SwaDims dm{L, L, HQ, H, window, chunk, mask_lmk, expand_to_chunk, 0, (chunk & (chunk - 1)) == 0, sm_scale};
  hipStream_t st = (hipStream_t)stream;
  const bf16_t *qq = (const bf16_t*)q, *kk = (const bf16_t*)k, *vv = (const bf16_t*)v,
               *oo = (const bf16_t*)o, *dd = (const bf16_t*)d_o;
  int rc;
  if (D == 64 && Dv == 64)
    rc = swa_bwd_launch_g<64, 64>(G, qq, kk, vv, oo, lse, dd, d_lse, (bf16_t*)dq, (bf16_t*)dk, (bf16_t*)dv, delta, B, dm, st);
  else if (D == 128 && Dv == 128)
    rc = swa_bwd_launch_g<128, 128>(G, qq, kk, vv, oo, lse, dd, d_lse, (bf16_t*)dq, (bf16_t*)dk, (bf16_t*)dv, delta, B, dm, st);
  else if (D == 64)
    rc = swa_bwd_launch_g<64, 128>(G, qq, kk, vv, oo, lse, dd, d_lse, (bf16_t*)dq, (bf16_t*)dk, (bf16_t*)dv, delta, B, dm, st);
  else
    rc = swa_bwd_launch_g<128, 64>(G, qq, kk, vv, oo, lse, dd, d_lse, (bf16_t*)dq, (bf16_t*)dk, (bf16_t*)dv, delta, B, dm, st);
  if (rc) return rc;
  HILS_CHECK_LAUNCH("hils_swa_bwd");
  return HILS_OK;
}
