// Exact per-chunk log Z: log_z[b,t,h,c] = log sum_{j in chunk c} exp(sm_scale * <q_t, k_j>)
// over chunks that lie fully before the query's local window.
#include "common.h"
#include "stream_tiles.h"
#include "../../include/hils_amd.h"

#define LZ_THREADS 256

struct LzDims {
  int L, HQ, H, G, D, S, W, N, mask_lmk;
  float sm_scale;
};

// number of fully-remote chunks of query t: chunk c counts iff t >= (c+1)*S + W - 1
__device__ __forceinline__ int lz_limit(const LzDims& dm, int t) {
  int lm = floordiv(t - dm.W + 1, dm.S);
  return lm < 0 ? 0 : (lm > dm.N ? dm.N : lm);
}

// One block per (b, t, hq); wavefront w takes chunks w, w+4, ...; lanes take tokens.
__global__ void __launch_bounds__(LZ_THREADS)
logz_fwd_simple(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                float* __restrict__ log_z, LzDims dm) {
  extern __shared__ float smem[];
  float* q_s = smem;  // D
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long row = blockIdx.x;  // (b*L + t)*HQ + hq
  const int hq = (int)(row % dm.HQ);
  const long bt = row / dm.HQ;
  const int t = (int)(bt % dm.L);
  const long b = bt / dm.L;
  const int hk = hq / dm.G;
  for (int d = tid; d < dm.D; d += LZ_THREADS) q_s[d] = bf2f(q[row * dm.D + d]);
  __syncthreads();
  const int lim = lz_limit(dm, t);
  float* out = log_z + row * (long)dm.N;
  for (int c = wave; c < dm.N; c += LZ_THREADS / 64) {
    if (c >= lim) {
      if (lane == 0) out[c] = HILS_NEG_INF;
      continue;
    }
    float m = HILS_NEG_INF, l = 0.f;
    for (int s = lane; s < dm.S; s += 64) {
      const int j = c * dm.S + s;
      if (j > t || j >= dm.L) continue;
      if (dm.mask_lmk && ((j + 1) % dm.S) == 0) continue;
      const bf16_t* kr = k + ((b * dm.L + j) * (long)dm.H + hk) * dm.D;
      float a = 0.f;
      for (int d8 = 0; d8 < dm.D / 8; ++d8) {
        float f[8];
        unpack8(*(const uint4*)(kr + d8 * 8), f);
#pragma unroll
        for (int i = 0; i < 8; ++i) a = fmaf(q_s[d8 * 8 + i], f[i], a);
      }
      a *= dm.sm_scale;
      const float mn = fmaxf(m, a);
      l = l * __expf(m - mn) + __expf(a - mn);
      m = mn;
    }
    const float mx = wave_max(m);
    float part = (m > HILS_NEG_INF) ? l * __expf(m - mx) : 0.f;
    part = wave_sum(part);
    if (lane == 0) out[c] = (part > 0.f) ? mx + logf(part) : HILS_NEG_INF;
  }
}

// Matrix-core forward for 64-token chunks.  A workgroup of four wavefronts owns 128/G consecutive
// queries of one KV head (128 score rows: query x head of the group) and walks the chunks that are
// remote for its last query.  The chunk's keys pass through LDS once per workgroup (double
// buffered); each wavefront multiplies them with its 32 rows, computing the TRANSPOSED scores
// K Q^T so that the 64 tokens of one row lie in 16 registers of 4 lanes: the log-sum-exp is an
// in-lane reduction plus one row-swap reduction.
#define LZM_RT 2  // 16-row tiles per wavefront

// Workgroup order of the matrix-core kernels: one-dimensional grids in which all blocks of a
// (batch, KV head) unit run on one XCD (the hardware hands consecutive workgroup ids to the 8 XCDs in
// turn: id -> (xcd, slot); unit = 8 * (slot / n_blk) + xcd), so that the keys (or query rows) the
// unit's workgroups stream are fetched into one L2 once instead of into all eight.  False for the
// padding ids of a unit count that is not a multiple of 8.
__device__ __forceinline__ bool lz_xcd_unit(int n_blk, int n_unit, int& unit, int& blk) {
  const int xcd = (int)(blockIdx.x % 8), slot = (int)(blockIdx.x / 8);
  unit = (slot / n_blk) * 8 + xcd;
  blk = slot % n_blk;
  return unit < n_unit;
}
static dim3 lz_xcd_grid(int n_blk, int n_unit) { return dim3((unsigned)(8 * ((n_unit + 7) / 8) * n_blk)); }
// (the occupancy hint also keeps the score accumulators in ordinary registers: without it the
// compiler, free to use 512 registers at this workgroup size, parks them in accumulation registers
// and copies every score back for the softmax)
template <int D, int G>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3)))
logz_fwd_mfma(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
              float* __restrict__ log_z, LzDims dm, int n_qt, int n_unit) {
  constexpr int KS = D / 32;
  constexpr int QW = 16 * LZM_RT / G;  // queries per wavefront
  constexpr int QB = 4 * QW;           // queries per workgroup
  constexpr int PITCH = D * 2 + 16;    // bytes per staged key row
  constexpr int NP = D / 32;           // 16-byte pieces of a chunk per thread
  __shared__ __align__(16) unsigned char k_s[2][64 * PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, j = lane >> 4;
  int unit, qt;
  if (!lz_xcd_unit(n_qt, n_unit, unit, qt)) return;
  qt = n_qt - 1 - qt;  // longest rows first
  const int hk = unit % dm.H;
  const long b = unit / dm.H;
  const int t0 = qt * QB + wave * QW;

  bf16x8_t qa[LZM_RT][KS];
  int lim[LZM_RT];
  long orow[LZM_RT];
  bool live[LZM_RT];
#pragma unroll
  for (int rt = 0; rt < LZM_RT; ++rt) {
    const int row = rt * 16 + col;
    const int t = t0 + row / G, g = row % G;
    live[rt] = t < dm.L;
    const int tc = live[rt] ? t : dm.L - 1;
    lim[rt] = live[rt] ? lz_limit(dm, t) : 0;
    orow[rt] = ((b * dm.L + tc) * (long)dm.HQ + hk * G + g);
    const bf16_t* qp = q + orow[rt] * D + j * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qa[rt][ks] = *(const bf16x8_t*)(qp + ks * 32);
  }
  int t_last = qt * QB + QB - 1;
  if (t_last > dm.L - 1) t_last = dm.L - 1;
  const int nc = lz_limit(dm, t_last);  // chunks the workgroup walks
  const float sc2 = dm.sm_scale * HILS_LOG2E;

  // (a native vector type: an array of HIP's uint4 struct that lives across the loop's back edge
  // is kept in scratch memory by the compiler)
  typedef unsigned lz_u32x4 __attribute__((ext_vector_type(4)));
  lz_u32x4 kr[NP];
  auto fetch = [&](int c) {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int p = tid + 256 * i;
      const int tok = p / (D / 8), seg = p % (D / 8);
      kr[i] = *(const lz_u32x4*)(k + ((b * dm.L + c * 64 + tok) * (long)dm.H + hk) * D + seg * 8);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int p = tid + 256 * i;
      const int tok = p / (D / 8), seg = p % (D / 8);
      *(lz_u32x4*)(&k_s[buf][tok * PITCH + seg * 16]) = kr[i];
    }
  };
  if (nc > 0) {
    fetch(0);
    stash(0);
  }
  __syncthreads();
  float keep[LZM_RT];
#pragma unroll
  for (int rt = 0; rt < LZM_RT; ++rt) keep[rt] = HILS_NEG_INF;
  for (int c = 0; c < nc; ++c) {
    fetch(c + 1 < nc ? c + 1 : c);
    const unsigned char* kb = k_s[c & 1];
    f32x4_t acc[LZM_RT][4];
#pragma unroll
    for (int rt = 0; rt < LZM_RT; ++rt)
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) acc[rt][tt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tt = 0; tt < 4; ++tt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8_t a = *(const bf16x8_t*)(kb + (tt * 16 + col) * PITCH + ks * 64 + j * 16);
#pragma unroll
        for (int rt = 0; rt < LZM_RT; ++rt)
          acc[rt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qa[rt][ks], acc[rt][tt], 0, 0, 0);
      }
#pragma unroll
    for (int rt = 0; rt < LZM_RT; ++rt) {
      // the maximum is taken over the raw products (the scale is positive) and the scale is applied
      // inside the exponent's fused multiply-add: no separate scaling pass
      float x[16];
#pragma unroll
      for (int tt = 0; tt < 4; ++tt)
#pragma unroll
        for (int i = 0; i < 4; ++i) x[tt * 4 + i] = acc[rt][tt][i];
      if (dm.mask_lmk && j == 3) x[15] = HILS_NEG_INF;  // token 63 = tile 3, lane row 3, register 3
      float m = fmaxf(x[0], x[1]);
#pragma unroll
      for (int i = 2; i < 16; i += 2) m = fmaxf(fmaxf(m, x[i]), x[i + 1]);
      m = rows_max(m) * sc2;  // in log2 units, as the sum below
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) s += __builtin_amdgcn_exp2f(fmaf(x[i], sc2, -m));
      s = rows_sum(s);
      const float val = (c < lim[rt]) ? (m + __builtin_amdgcn_logf(s)) * HILS_LN2 : HILS_NEG_INF;
      if (j == (c & 3)) keep[rt] = val;
    }
    if ((c & 3) == 3 || c == nc - 1) {
      const int cc = (c & ~3) + j;
#pragma unroll
      for (int rt = 0; rt < LZM_RT; ++rt)
        if (live[rt] && cc <= c) log_z[orow[rt] * dm.N + cc] = keep[rt];
    }
    stash((c + 1) & 1);
    __syncthreads();
  }
  // chunks past the workgroup's walk are not remote for any of its rows
  for (int r = 0; r < 16 * LZM_RT; ++r) {
    const int t = t0 + r / G, g = r % G;
    if (t >= dm.L) break;
    float* out = log_z + ((b * dm.L + t) * (long)dm.HQ + hk * G + g) * dm.N;
    for (int c = nc + lane; c < dm.N; c += 64) out[c] = HILS_NEG_INF;
  }
}

// ---- matrix-core backward -------------------------------------------------------------------
// Both gradients are a pair of products around the same element-wise step
//   dS[row, tok] = d_log_z[row, c(tok)] * exp(s[row, tok] - log_z[row, c(tok)]) * sm_scale
//   dQ = dS K,   dK = dS^T Q.
// One side of the product is OWNED by a wavefront (32 rows, held in registers as matrix operands,
// with the fp32 gradient accumulators), the other side STREAMS through LDS in 64-row tiles, stored
// twice: row-major (operand of the score product) and transposed (operand of the gradient
// product, whose contraction runs over the streamed rows).  The scores are computed with the
// owned side as matrix columns, so their accumulator registers are already the left operand of
// the gradient product.
// dQ: a wavefront owns 32 score rows (query x head), the chunks' keys stream.
template <int D, int G>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
logz_bwd_dq_mfma(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                 const float* __restrict__ log_z, const float* __restrict__ d_log_z,
                 bf16_t* __restrict__ dq, LzDims dm, int n_qt, int n_unit) {
  constexpr int KS = D / 32, DT = D / 16;
  constexpr int QW = 16 * LZM_RT / G, QB = 4 * QW;
  constexpr int PITCH = D * 2 + 16;
  constexpr int SEGS = D / 8;            // 16-byte pieces per row
  constexpr int PPP = 256 / SEGS;        // row pairs per pass of the workgroup
  constexpr int NPASS = 32 / PPP;
  __shared__ __align__(16) unsigned char k_s[64 * PITCH];
  __shared__ __align__(16) unsigned char kt_s[D * LZM_PT];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, j = lane >> 4;
  int unit, qt;
  if (!lz_xcd_unit(n_qt, n_unit, unit, qt)) return;
  qt = n_qt - 1 - qt;
  const int hk = unit % dm.H;
  const long b = unit / dm.H;
  const int t0 = qt * QB + wave * QW;

  bf16x8_t qa[LZM_RT][KS];
  int lim[LZM_RT];
  long orow[LZM_RT];
#pragma unroll
  for (int rt = 0; rt < LZM_RT; ++rt) {
    const int row = rt * 16 + col;
    const int t = t0 + row / G, g = row % G;
    const int tc = t < dm.L ? t : dm.L - 1;
    lim[rt] = t < dm.L ? lz_limit(dm, t) : 0;
    orow[rt] = ((b * dm.L + tc) * (long)dm.HQ + hk * G + g);
    const bf16_t* qp = q + orow[rt] * D + j * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qa[rt][ks] = *(const bf16x8_t*)(qp + ks * 32);
  }
  int t_last = qt * QB + QB - 1;
  if (t_last > dm.L - 1) t_last = dm.L - 1;
  const int nc = lz_limit(dm, t_last);
  const float sc2 = dm.sm_scale * HILS_LOG2E;

  const int seg = tid % SEGS, rp0 = tid / SEGS;
  uint4 kr[NPASS][2];
  auto fetch = [&](int c) {
#pragma unroll
    for (int i = 0; i < NPASS; ++i)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int tok = 2 * (rp0 + PPP * i) + h;
        kr[i][h] = *(const uint4*)(k + ((b * dm.L + c * 64 + tok) * (long)dm.H + hk) * D + seg * 8);
      }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < NPASS; ++i)
      lzm_stash_pair<PITCH>(k_s, kt_s, 2 * (rp0 + PPP * i), seg, kr[i][0], kr[i][1]);
  };
  f32x4_t acc[LZM_RT][DT];
#pragma unroll
  for (int rt = 0; rt < LZM_RT; ++rt)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[rt][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float lzn[LZM_RT], dln[LZM_RT];
  auto fetch_z = [&](int c) {
#pragma unroll
    for (int rt = 0; rt < LZM_RT; ++rt) {
      lzn[rt] = log_z[orow[rt] * dm.N + c];
      dln[rt] = d_log_z[orow[rt] * dm.N + c];
    }
  };
  if (nc > 0) {
    fetch(0);
    fetch_z(0);
    stash();
  }
  __syncthreads();
  for (int c = 0; c < nc; ++c) {
    float off[LZM_RT], coef[LZM_RT];
#pragma unroll
    for (int rt = 0; rt < LZM_RT; ++rt) {
      const bool ok = c < lim[rt] && lzn[rt] > -1e30f;
      off[rt] = ok ? lzn[rt] * HILS_LOG2E : 0.f;
      coef[rt] = ok ? dln[rt] * dm.sm_scale : 0.f;
    }
    const int cn = c + 1 < nc ? c + 1 : c;
    fetch(cn);
    fetch_z(cn);
    float p[LZM_RT][4][4];
    {
      f32x4_t st[LZM_RT][4];
#pragma unroll
      for (int rt = 0; rt < LZM_RT; ++rt)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) st[rt][tt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int tt = 0; tt < 4; ++tt)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8_t a = *(const bf16x8_t*)(k_s + (tt * 16 + col) * PITCH + ks * 64 + j * 16);
#pragma unroll
          for (int rt = 0; rt < LZM_RT; ++rt)
            st[rt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qa[rt][ks], st[rt][tt], 0, 0, 0);
        }
#pragma unroll
      for (int rt = 0; rt < LZM_RT; ++rt)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            p[rt][tt][i] = __builtin_amdgcn_exp2f(st[rt][tt][i] * sc2 - off[rt]) * coef[rt];
    }
    lzm_grad_product<D, LZM_RT>(kt_s, p, acc, col, j);
    __syncthreads();
    stash();
    __syncthreads();
  }
#pragma unroll
  for (int rt = 0; rt < LZM_RT; ++rt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = rt * 16 + 4 * j + i;
      const int t = t0 + row / G, g = row % G;
      if (t >= dm.L) continue;
      bf16_t* out = dq + ((b * dm.L + t) * (long)dm.HQ + hk * G + g) * D + col;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) out[dt * 16] = f2bf(acc[rt][dt][i]);
    }
}

// dK: a workgroup owns two chunks (wavefront: 32 tokens of one chunk), the score rows of the
// queries behind them stream in tiles of 64 rows (64/G queries x G heads).
template <int D, int G>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
logz_bwd_dk_mfma(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                 const float* __restrict__ log_z, const float* __restrict__ d_log_z,
                 bf16_t* __restrict__ dk, LzDims dm, int n_pair, int n_unit) {
  constexpr int KS = D / 32, DT = D / 16;
  constexpr int QT = 64 / G;  // queries per streamed tile
  constexpr int PITCH = D * 2 + 16;
  constexpr int SEGS = D / 8, PPP = 256 / SEGS, NPASS = 32 / PPP;
  __shared__ __align__(16) unsigned char q_s[64 * PITCH];
  __shared__ __align__(16) unsigned char qt_s[D * LZM_PT];
  __shared__ __align__(16) float off_s[2][64];
  __shared__ __align__(16) float coef_s[2][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, j = lane >> 4;
  // Workgroup order.  The workgroups of one (batch, KV head) stream the same query rows, each from the
  // first query behind its chunks to the last one: they walk the tiles from the END, so that all of
  // them are on the same tile at the same time, and the one-dimensional grid puts them on one XCD
  // (the hardware hands consecutive workgroup ids to the 8 XCDs in turn: id -> (xcd, slot)), whose L2
  // then serves all but the first reader of a tile.  Walking forward from different starting points
  // in the hardware's order, every read of a tile missed (L2 hit rate 2 %, the kernel waiting on
  // HBM latency at one wavefront per SIMD).  The chunk pairs of a unit come longest walk first.
  int unit, pair;
  if (!lz_xcd_unit(n_pair, n_unit, unit, pair)) return;
  const int c0 = 2 * pair, ch = wave >> 1;
  const int hk = unit % dm.H;
  const long b = unit / dm.H;
  const int tok0 = (c0 + ch) * 64 + (wave & 1) * 32;  // first owned token

  bf16x8_t ka[2][KS];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    int tok = tok0 + tt * 16 + col;
    if (tok > dm.L - 1) tok = dm.L - 1;  // such tokens get no gradient: every coefficient is 0
    const bf16_t* kp = k + ((b * dm.L + tok) * (long)dm.H + hk) * D + j * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ka[tt][ks] = *(const bf16x8_t*)(kp + ks * 32);
  }
  // first query with chunk c0 fully behind its window, rounded down to a tile
  int t_first = (c0 + 1) * 64 + dm.W - 1;
  if (t_first < 0) t_first = 0;
  const int tile0 = t_first / QT;
  const int n_tiles = (dm.L + QT - 1) / QT;
  const float sc2 = dm.sm_scale * HILS_LOG2E;

  const int seg = tid % SEGS, rp0 = tid / SEGS;
  uint4 qr[NPASS][2];
  float zo = 0.f, zc = 0.f;  // raw log_z and d_log_z of this thread's (row, chunk); zin: inside the limits
  bool zin = false;
  auto fetch = [&](int tile) {
#pragma unroll
    for (int i = 0; i < NPASS; ++i)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int row = 2 * (rp0 + PPP * i) + h;
        int t = tile * QT + row / G;
        if (t > dm.L - 1) t = dm.L - 1;
        qr[i][h] = *(const uint4*)(q + ((b * dm.L + t) * (long)dm.HQ + hk * G + row % G) * D + seg * 8);
      }
    if (tid < 128) {
      const int row = tid & 63, cc = c0 + (tid >> 6);
      const int t = tile * QT + row / G;
      const bool in = t < dm.L && cc < dm.N && cc < lz_limit(dm, t < dm.L ? t : 0);
      const long zi = ((b * dm.L + (t < dm.L ? t : dm.L - 1)) * (long)dm.HQ + hk * G + row % G) * dm.N +
                      (cc < dm.N ? cc : dm.N - 1);
      // raw values: what a row outside the limits gets is decided in stash(), so that nothing
      // here waits for a load (which would also wait for the query rows issued before it)
      zo = log_z[zi];
      zc = d_log_z[zi];
      zin = in;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < NPASS; ++i)
      lzm_stash_pair<PITCH>(q_s, qt_s, 2 * (rp0 + PPP * i), seg, qr[i][0], qr[i][1]);
    if (tid < 128) {
      const bool ok = zin && zo > -1e30f;
      off_s[tid >> 6][tid & 63] = ok ? zo * HILS_LOG2E : 0.f;
      coef_s[tid >> 6][tid & 63] = ok ? zc * dm.sm_scale : 0.f;
    }
  };
  f32x4_t acc[2][DT];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[tt][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  if (tile0 < n_tiles) {
    fetch(n_tiles - 1);
    stash();
  }
  __syncthreads();
  for (int tile = n_tiles - 1; tile >= tile0; --tile) {
    fetch(tile > tile0 ? tile - 1 : tile);
    float p[2][4][4];  // [owned token tile][streamed row tile][row 4j+i]
    {
      f32x4_t st[2][4];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) st[tt][rr] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int rr = 0; rr < 4; ++rr)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8_t a = *(const bf16x8_t*)(q_s + (rr * 16 + col) * PITCH + ks * 64 + j * 16);
#pragma unroll
          for (int tt = 0; tt < 2; ++tt)
            st[tt][rr] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, ka[tt][ks], st[tt][rr], 0, 0, 0);
        }
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        const float4 o4 = *(const float4*)&off_s[ch][rr * 16 + 4 * j];
        const float4 c4 = *(const float4*)&coef_s[ch][rr * 16 + 4 * j];
        const float o[4] = {o4.x, o4.y, o4.z, o4.w}, cf[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            p[tt][rr][i] = __builtin_amdgcn_exp2f(st[tt][rr][i] * sc2 - o[i]) * cf[i];
      }
    }
    lzm_grad_product<D, 2>(qt_s, p, acc, col, j);
    __syncthreads();
    stash();
    __syncthreads();
  }
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tok = tok0 + tt * 16 + 4 * j + i;
      if (tok >= dm.L) continue;
      bf16_t* out = dk + ((b * dm.L + tok) * (long)dm.H + hk) * D + col;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) out[dt * 16] = f2bf(acc[tt][dt][i]);
    }
}

// dq[b,t,hq,:] = sum_c sum_j dlz[c] * exp(s_j - lz[c]) * scale * k_j
__global__ void __launch_bounds__(LZ_THREADS)
logz_bwd_dq_simple(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                   const float* __restrict__ log_z, const float* __restrict__ d_log_z,
                   bf16_t* __restrict__ dq, LzDims dm) {
  extern __shared__ float smem[];
  float* q_s = smem;          // D
  float* ds = q_s + dm.D;     // S
  const int tid = threadIdx.x;
  const long row = blockIdx.x;
  const int hq = (int)(row % dm.HQ);
  const long bt = row / dm.HQ;
  const int t = (int)(bt % dm.L);
  const long b = bt / dm.L;
  const int hk = hq / dm.G;
  for (int d = tid; d < dm.D; d += LZ_THREADS) q_s[d] = bf2f(q[row * dm.D + d]);
  const int lim = lz_limit(dm, t);
  float acc = 0.f;  // thread d (< D) owns one output column
  for (int c = 0; c < lim; ++c) {
    const float lz = log_z[row * (long)dm.N + c];
    const float dlz = d_log_z[row * (long)dm.N + c];
    __syncthreads();
    for (int s = tid; s < dm.S; s += LZ_THREADS) {
      const int j = c * dm.S + s;
      float val = 0.f;
      if (j <= t && j < dm.L && lz > -1e30f) {
        const bf16_t* kr = k + ((b * dm.L + j) * (long)dm.H + hk) * dm.D;
        float a = 0.f;
        for (int d8 = 0; d8 < dm.D / 8; ++d8) {
          float f[8];
          unpack8(*(const uint4*)(kr + d8 * 8), f);
#pragma unroll
          for (int i = 0; i < 8; ++i) a = fmaf(q_s[d8 * 8 + i], f[i], a);
        }
        val = dlz * __expf(a * dm.sm_scale - lz) * dm.sm_scale;
      }
      ds[s] = val;
    }
    __syncthreads();
    for (int d = tid; d < dm.D; d += LZ_THREADS) {
      float a = 0.f;
      for (int s = 0; s < dm.S; ++s) {
        const int j = c * dm.S + s;
        if (j < dm.L) a = fmaf(ds[s], bf2f(k[((b * dm.L + j) * (long)dm.H + hk) * dm.D + d]), a);
      }
      acc += a;  // D <= LZ_THREADS: one column per thread
    }
  }
  if (tid < dm.D) dq[row * dm.D + tid] = f2bf(acc);
}

// dk[b, c*S+s, hk, :] = sum_{g} sum_{t} dlz[t,hq,c] * exp(s - lz) * scale * q[t,hq,:]
// One block per (b, c, hk); queries are streamed in tiles of LZ_TT.
#define LZ_TT 8
#define LZ_MAX_ACC 32
__global__ void __launch_bounds__(LZ_THREADS)
logz_bwd_dk_simple(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                   const float* __restrict__ log_z, const float* __restrict__ d_log_z,
                   bf16_t* __restrict__ dk, LzDims dm) {
  extern __shared__ float smem[];
  const int G = dm.G, S = dm.S, D = dm.D, DP = dm.D + 1;
  float* k_s = smem;                          // S*DP
  float* q_s = k_s + (size_t)S * DP;          // TT*G*D
  float* ds = q_s + (size_t)LZ_TT * G * D;    // TT*G*S
  const int tid = threadIdx.x;
  const int c = blockIdx.x, hk = blockIdx.y;
  const long b = blockIdx.z;
  for (int i = tid; i < S * D; i += LZ_THREADS) {
    const int s = i / D, d = i - s * D;
    const int j = c * S + s;
    k_s[s * DP + d] = (j < dm.L) ? bf2f(k[((b * dm.L + j) * (long)dm.H + hk) * D + d]) : 0.f;
  }
  float acc[LZ_MAX_ACC];
#pragma unroll
  for (int i = 0; i < LZ_MAX_ACC; ++i) acc[i] = 0.f;
  int t_first = (c + 1) * S + dm.W - 1;
  if (t_first < 0) t_first = 0;
  for (int t0 = t_first; t0 < dm.L; t0 += LZ_TT) {
    __syncthreads();
    for (int i = tid; i < LZ_TT * G * D; i += LZ_THREADS) {
      const int tt = i / (G * D), r = i - tt * (G * D);
      const int t = t0 + tt;
      q_s[i] = (t < dm.L) ? bf2f(q[((b * dm.L + t) * (long)dm.HQ + hk * G) * D + r]) : 0.f;
    }
    __syncthreads();
    for (int i = tid; i < LZ_TT * G * S; i += LZ_THREADS) {
      const int tt = i / (G * S), r = i - tt * (G * S);
      const int g = r / S, s = r - g * S;
      const int t = t0 + tt, j = c * S + s;
      float val = 0.f;
      if (t < dm.L && j <= t && j < dm.L) {
        const long zrow = ((b * dm.L + t) * (long)dm.HQ + hk * G + g) * dm.N + c;
        const float lz = log_z[zrow];
        if (lz > -1e30f) {
          const float* qr = q_s + (tt * G + g) * D;
          float a = 0.f;
          for (int d = 0; d < D; ++d) a = fmaf(qr[d], k_s[s * DP + d], a);
          val = d_log_z[zrow] * __expf(a * dm.sm_scale - lz) * dm.sm_scale;
        }
      }
      ds[i] = val;
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < LZ_MAX_ACC; ++e) {
      const int oi = tid + e * LZ_THREADS;
      if (oi < S * D) {
        const int s = oi / D, d = oi - s * D;
        float a = acc[e];
        for (int r = 0; r < LZ_TT * G; ++r) a = fmaf(ds[r * S + s], q_s[r * D + d], a);
        acc[e] = a;
      }
    }
  }
#pragma unroll
  for (int e = 0; e < LZ_MAX_ACC; ++e) {
    const int oi = tid + e * LZ_THREADS;
    if (oi < S * D) {
      const int s = oi / D, d = oi - s * D;
      const int j = c * S + s;
      if (j < dm.L) dk[((b * dm.L + j) * (long)dm.H + hk) * D + d] = f2bf(acc[e]);
    }
  }
}

// shapes of the matrix-core kernels: 64-token chunks, head dim 64/128, group size dividing 16
static bool lz_mfma_covers(int G, int D, int S, int H, int B) {
  return S == 64 && (D == 64 || D == 128) && (G == 1 || G == 2 || G == 4 || G == 8 || G == 16) &&
         H <= 65535 && B <= 65535;
}
// expands LZ_LAUNCH(D, G) for the covered (D, G)
#define LZ_DISPATCH_G(DD, G_)                                                                  \
  switch (G_) {                                                                                \
    case 1: LZ_LAUNCH(DD, 1); break;                                                           \
    case 2: LZ_LAUNCH(DD, 2); break;                                                           \
    case 4: LZ_LAUNCH(DD, 4); break;                                                           \
    case 8: LZ_LAUNCH(DD, 8); break;                                                           \
    default: LZ_LAUNCH(DD, 16); break;                                                         \
  }
#define LZ_DISPATCH(D_, G_)                                                                    \
  if ((D_) == 64) { LZ_DISPATCH_G(64, G_) } else { LZ_DISPATCH_G(128, G_) }

static int lz_check(const char* name, int B, int L, int HQ, int H, int D, int S) {
  HILS_REQUIRE(B > 0 && L > 0 && HQ > 0 && H > 0 && D > 0 && S > 0, "%s: sizes must be positive", name);
  HILS_REQUIRE(HQ % H == 0, "%s: HQ (%d) must be a multiple of H (%d)", name, HQ, H);
  HILS_REQUIRE(D % 8 == 0, "%s: D (%d) must be a multiple of 8", name, D);
  HILS_REQUIRE((long)B * L * HQ <= 2147483647L, "%s: grid too large", name);
  return HILS_OK;
}

extern "C" int hils_chunk_logz_fwd(const void* q, const void* k, float* log_z, int B, int L, int HQ,
                                   int H, int D, int S, int window, float sm_scale, int mask_lmk,
                                   void* stream) {
  HILS_REQUIRE(q && k && log_z, "hils_chunk_logz_fwd: null pointer");
  if (int rc = lz_check("hils_chunk_logz_fwd", B, L, HQ, H, D, S)) return rc;
  LzDims dm{L, HQ, H, HQ / H, D, S, window, (L + S - 1) / S, mask_lmk, sm_scale};
  const int G = HQ / H;
  if (lz_mfma_covers(G, D, S, H, B)) {
    const int QB = 4 * 16 * LZM_RT / G;
    const int n_qt = (L + QB - 1) / QB;
    HILS_REQUIRE(((long)B * H + 7) / 8 * 8 * n_qt < (1L << 31), "hils_chunk_logz_fwd: B * H * L too large for the grid");
    const dim3 grid = lz_xcd_grid(n_qt, B * H);
#define LZ_LAUNCH(DD, GG)                                                                      \
  hipLaunchKernelGGL((logz_fwd_mfma<DD, GG>), grid, dim3(256), 0, (hipStream_t)stream,         \
                     (const bf16_t*)q, (const bf16_t*)k, log_z, dm, n_qt, B * H)
    LZ_DISPATCH(D, G);
#undef LZ_LAUNCH
    HILS_CHECK_LAUNCH("hils_chunk_logz_fwd");
    return HILS_OK;
  }
  hipLaunchKernelGGL(logz_fwd_simple, dim3((unsigned)((long)B * L * HQ)), dim3(LZ_THREADS),
                     D * sizeof(float), (hipStream_t)stream, (const bf16_t*)q, (const bf16_t*)k,
                     log_z, dm);
  HILS_CHECK_LAUNCH("hils_chunk_logz_fwd");
  return HILS_OK;
}

extern "C" int hils_chunk_logz_bwd_dq(const void* q, const void* k, const float* log_z,
                                      const float* d_log_z, void* dq, int B, int L, int HQ, int H,
                                      int D, int S, int window, float sm_scale, void* stream) {
  HILS_REQUIRE(q && k && log_z && d_log_z && dq, "hils_chunk_logz_bwd_dq: null pointer");
  if (int rc = lz_check("hils_chunk_logz_bwd_dq", B, L, HQ, H, D, S)) return rc;
  HILS_REQUIRE(D <= LZ_THREADS, "hils_chunk_logz_bwd_dq: D (%d) must be <= %d", D, LZ_THREADS);
  LzDims dm{L, HQ, H, HQ / H, D, S, window, (L + S - 1) / S, 0, sm_scale};
  if (lz_mfma_covers(HQ / H, D, S, H, B)) {
    const int G = HQ / H;
    const int QB = 4 * 16 * LZM_RT / G;
    const int n_qt = (L + QB - 1) / QB;
    HILS_REQUIRE(((long)B * H + 7) / 8 * 8 * n_qt < (1L << 31), "hils_chunk_logz_bwd_dq: B * H * L too large for the grid");
    const dim3 grid = lz_xcd_grid(n_qt, B * H);
#define LZ_LAUNCH(DD, GG)                                                                      \
  hipLaunchKernelGGL((logz_bwd_dq_mfma<DD, GG>), grid, dim3(256), 0, (hipStream_t)stream,      \
                     (const bf16_t*)q, (const bf16_t*)k, log_z, d_log_z, (bf16_t*)dq, dm, n_qt, B * H)
    LZ_DISPATCH(D, G);
#undef LZ_LAUNCH
    HILS_CHECK_LAUNCH("hils_chunk_logz_bwd_dq");
    return HILS_OK;
  }
  hipLaunchKernelGGL(logz_bwd_dq_simple, dim3((unsigned)((long)B * L * HQ)), dim3(LZ_THREADS),
                     (D + S) * sizeof(float), (hipStream_t)stream, (const bf16_t*)q,
                     (const bf16_t*)k, log_z, d_log_z, (bf16_t*)dq, dm);
  HILS_CHECK_LAUNCH("hils_chunk_logz_bwd_dq");
  return HILS_OK;
}

extern "C" int hils_chunk_logz_bwd_dk(const void* q, const void* k, const float* log_z,
                                      const float* d_log_z, void* dk, int B, int L, int HQ, int H,
                                      int D, int S, int window, float sm_scale, void* stream) {
  HILS_REQUIRE(q && k && log_z && d_log_z && dk, "hils_chunk_logz_bwd_dk: null pointer");
  if (int rc = lz_check("hils_chunk_logz_bwd_dk", B, L, HQ, H, D, S)) return rc;
  const int G = HQ / H;
  HILS_REQUIRE(S * D <= LZ_MAX_ACC * LZ_THREADS, "hils_chunk_logz_bwd_dk: S*D (%d) too large", S * D);
  LzDims dm{L, HQ, H, G, D, S, window, (L + S - 1) / S, 0, sm_scale};
  if (lz_mfma_covers(G, D, S, H, B)) {
    const int n_pair = (dm.N + 1) / 2;
    HILS_REQUIRE(((long)B * H + 7) / 8 * 8 * n_pair < (1L << 31), "hils_chunk_logz_bwd_dk: B * H * N too large for the grid");
    const int n_unit = B * H;
    const dim3 grid = lz_xcd_grid(n_pair, n_unit);
#define LZ_LAUNCH(DD, GG)                                                                      \
  hipLaunchKernelGGL((logz_bwd_dk_mfma<DD, GG>), grid, dim3(256), 0, (hipStream_t)stream,      \
                     (const bf16_t*)q, (const bf16_t*)k, log_z, d_log_z, (bf16_t*)dk, dm, n_pair, n_unit)
    LZ_DISPATCH(D, G);
#undef LZ_LAUNCH
    HILS_CHECK_LAUNCH("hils_chunk_logz_bwd_dk");
    return HILS_OK;
  }
  size_t smem = ((size_t)S * (D + 1) + (size_t)LZ_TT * G * D + (size_t)LZ_TT * G * S) * sizeof(float);
  HILS_REQUIRE(smem <= 160 * 1024, "hils_chunk_logz_bwd_dk: tile does not fit in LDS");
  HILS_REQUIRE(H <= 65535 && B <= 65535, "hils_chunk_logz_bwd_dk: H/B too large for the grid");
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)logz_bwd_dk_simple,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  hipLaunchKernelGGL(logz_bwd_dk_simple, dim3(dm.N, H, B), dim3(LZ_THREADS), smem,
                     (hipStream_t)stream, (const bf16_t*)q, (const bf16_t*)k, log_z, d_log_z,
                     (bf16_t*)dk, dm);
  HILS_CHECK_LAUNCH("hils_chunk_logz_bwd_dk");
  return HILS_OK;
}
