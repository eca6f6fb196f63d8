/* C ABI of libhils_amd.so: hand-written gfx950 kernels for the HiLS-Attention
 * operator stack.  Plain pointers and sizes only; every pointer is a DEVICE
 * pointer unless stated; `stream` is a hipStream_t passed as void*.  All tensors
 * are contiguous, token-major (B, L, H, D), bf16 = raw bfloat16 bits.
 * Every function returns 0 on success, 1 on an invalid argument, 2 on a launch
 * failure; hils_last_error() then returns a message.  No function allocates or
 * frees device memory or synchronises the stream.
 *
 * Each entry point cites the reference interface it replaces (paths relative to
 * the reference repository root).
 */
#ifndef HILS_AMD_H
#define HILS_AMD_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

const char* hils_last_error(void);
int hils_version(void);

/* ---- chunk keys ------------------------------------------------------------ */

/* Mean pool: lmk_k[b,n,h,:] = mean_s k[b,n*S+s,h,:].
 * Replaces `k_chunked.mean(dim=2)` at models/FlashHiLS/hils_attention.py:398,436,446,460.
 * k (B,L,H,D) bf16 -> lmk_k (B,L/S,H,D) bf16.  L % S == 0, D % 8 == 0. */
int hils_mean_pool_fwd(const void* k, void* lmk_k, int B, int L, int H, int D, int S, void* stream);
/* Its backward: dk[b,t,h,:] = g_lmk[b,t/S,h,:] / S (bf16 in, bf16 out). */
int hils_mean_pool_bwd(const void* g_lmk, void* dk, int B, int L, int H, int D, int S, void* stream);

/* Attention pool forward.  Replaces chunk_attn_pool_fwd_kernel_fallback /
 * chunk_attn_pool_fwd_kernel behind ChunkAttnPoolFunction.forward
 * (ops/chunk_attn_pool_tilelang.py:329-410, :31-150, :540-570), and the K head repeat in front of it
 * (models/FlashHiLS/hils_attention.py:20-50, :339, :391: `_repeat_k_heads_for_gqa`).
 * mu_q (BN,H,D) bf16, k (BN,S,h_kv,D) bf16 -> lmk_k (BN,H,D) bf16, lmk_b (BN,H) fp32,
 * p (BN,S,H) fp32 (saved for backward).  H % h_kv == 0: query head h reads K head h / (H / h_kv)
 * (h_kv == H: a K tile per head, the reference kernels' layout).  compact != 0: lmk_k is written as
 * zeros.  shared_k != 0 (needs h_kv == H): K is read from head 0 for every head. */
int hils_attn_pool_fwd(const void* mu_q, const void* k, void* lmk_k, float* lmk_b, float* p,
                       int BN, int S, int H, int h_kv, int D, float sm_scale, int compact, int shared_k,
                       void* stream);
/* Attention pool backward.  Replaces chunk_attn_pool_bwd_kernel_fallback /
 * chunk_attn_pool_bwd_kernel (ops/chunk_attn_pool_tilelang.py:425-533, :165-314).
 * g_k (BN,H,D) bf16, g_b (BN,H) fp32 -> d_mu (BN,H,D) bf16, d_k (BN,S,h_kv,D) bf16 (h_kv < H: the sum
 * over the H / h_kv query heads of a K head, accumulated in fp32 and rounded once).
 * shared_k != 0: d_k is summed over heads into head 0 and heads 1.. are zero. */
int hils_attn_pool_bwd(const void* mu_q, const void* k, const float* p, const float* lmk_b,
                       const void* g_k, const float* g_b, void* d_mu, void* d_k,
                       int BN, int S, int H, int h_kv, int D, float sm_scale, int compact, int shared_k,
                       void* stream);

/* ---- top-k chunk selection -------------------------------------------------- */

/* Fused LSE + select + ascending sort + score gather.  Replaces hils_lse_kernel,
 * torch.logaddexp, weighted_select_kernel, sort_topk_indices_kernel and
 * recompute_topk_max_pooling_scores_kernel as sequenced by
 * SoftmaxTopKMaxPoolingFusedFn.forward (ops/topk_head_softmax.py:192-400, :438-631,
 * :870-971, :669-832, :1012-1038).
 * q (B,L,h_kv,G,D) bf16; lmks (B,N,h_kv,D) bf16 or, per_qhead != 0, (B,N,h_kv*G,D);
 * lse_swa (B,L,h_kv,G) fp32; bias (B,N,h_kv,G) fp32 or NULL; gumbel (h_kv*G,N) fp32 or
 * NULL; drop_mask (B,L,N) int32 or NULL.
 * Outputs: indices (B,L,h_kv,topk) int32 ascending, -1 padded; scores
 * (B,L,h_kv,G,topk) bf16 = sm_scale*<q,lmk[idx]>, -inf where idx < 0.
 * Optional outputs (NULL to skip): lse_total (B,L,h_kv,G) fp32 =
 * logaddexp(lse_swa, lse_hils); sel_logits (B,L,h_kv,G,N) fp32 = the selection
 * logits (scaled qk + bias + gumbel, -inf where the chunk is not visible).
 * Chunk c is visible to query t iff !causal or c < floor((t+q_offset-window+1)/block)
 * (window > 0) / floor((t+q_offset)/block) (window <= 0).  Ties: lower index wins.
 * workspace: device scratch of hils_topk_fwd_workspace(...) bytes or NULL.  With few queries
 * (decode) and a workspace, the logits are spread over many workgroups and parked there
 * before a separate selection kernel (or one workgroup per (query, KV head) keeps them in LDS
 * and needs no scratch); with many queries the chunk keys are first repacked there into MFMA
 * operand order, and behind them a bias head-major in blocks of 16 chunks.  Without a workspace one
 * fused kernel reads the chunk keys as they are (and, with a key per query head or more than four
 * query heads per KV head, a much slower general kernel runs).
 * workspace_bytes: size of the buffer behind `workspace` (here and in every entry point that takes
 * a workspace); a non-NULL workspace shorter than the matching *_workspace(...) query is rejected
 * with status 1 before anything is launched. */
size_t hils_topk_fwd_workspace(int B, int L, int N, int h_kv, int G);
int hils_topk_fwd(const void* q, const void* lmks, const float* lse_swa, const float* bias,
                  const float* gumbel, const int32_t* drop_mask, int32_t* indices, void* scores,
                  float* lse_total, float* sel_logits, void* workspace, size_t workspace_bytes, int B, int L,
                  int N, int h_kv, int G, int D, int topk, int block_size, int window_size, int causal,
                  int q_offset, int per_qhead, float sm_scale, void* stream);

/* hils_topk_fwd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments and results as hils_topk_fwd without the workspace: the scratch (repacked chunk keys
 * for prefill-sized calls, parked logits for the two-kernel decode path) lives in a device array
 * of hils_topk_fwd_noalloc_max_workspace() bytes (8 MiB) inside the library, one copy per GPU,
 * held until the process ends.  Shapes whose hils_topk_fwd_workspace(...) exceeds that are
 * rejected (status 1).  Calls no allocating routine; the first call on a device looks the array's
 * address up once (do that call outside a graph capture).  Every call on a GPU shares that GPU's
 * array: calls that overlap on one GPU (two streams, two host threads) race. */
size_t hils_topk_fwd_noalloc_max_workspace(void);
int hils_topk_fwd_noalloc(const void* q, const void* lmks, const float* lse_swa, const float* bias,
                          const float* gumbel, const int32_t* drop_mask, int32_t* indices,
                          void* scores, float* lse_total, float* sel_logits, int B, int L, int N,
                          int h_kv, int G, int D, int topk, int block_size, int window_size,
                          int causal, int q_offset, int per_qhead, float sm_scale, void* stream);

/* hils_topk_fwd plus the layer's inter-chunk softmax in the same call (inference): also writes
 * weights (B,L,h_kv*G,topk+1) bf16 = softmax over [scores (as bf16) (+ prior_b gathered at the
 * indices, cast to bf16), lse_swa], the K+1-way softmax of models/FlashHiLS/hils_attention.py:585-610
 * (what hils_chunk_weights computes from these scores).  prior_b (B,N,h_kv*G) fp32 or NULL; the
 * layer's default mode (enable_prior_query) passes one tensor as `bias` and as `prior_b`
 * (hils_attention.py:568-602).  With about one (query, KV head) row per compute unit the selection
 * kernel writes the weights itself (when prior_b == bias or both are NULL); otherwise
 * hils_chunk_weights runs on the same stream.  No lse_total / sel_logits outputs. */
int hils_topk_fwd_weights(const void* q, const void* lmks, const float* lse_swa, const float* bias,
                          const float* prior_b, const float* gumbel, const int32_t* drop_mask, int32_t* indices,
                          void* scores, void* weights, void* workspace, size_t workspace_bytes, int B, int L,
                          int N, int h_kv, int G, int D, int topk, int block_size, int window_size, int causal,
                          int q_offset, int per_qhead, float sm_scale, void* stream);

/* hils_topk_fwd_weights for lse_swa in bf16, the dtype the reference's layer hands it over in
 * (lse_sum.to(hidden_states.dtype), models/FlashHiLS/hils_attention.py:547; its kernels read it in
 * that dtype, ops/topk_head_softmax.py:1291-1367): saves the conversion pass.  Only the shapes
 * hils_topk_lse16_covers accepts (many queries, shared chunk keys, G <= 8, N <= 512, topk <= 32,
 * no noise / drop mask: the one-pass prefill kernel), with the workspace of
 * hils_topk_fwd_workspace; other shapes are rejected and take hils_topk_fwd_weights with fp32.
 * bias / prior_b as in hils_topk_fwd_weights (NULL for none). */
int hils_topk_lse16_covers(int B, int L, int N, int h_kv, int G, int D, int topk);
int hils_topk_fwd_weights_lse16(const void* q, const void* lmks, const void* lse_swa_bf16, const float* bias,
                                const float* prior_b, int32_t* indices,
                                void* scores, void* weights, void* workspace, size_t workspace_bytes, int B,
                                int L, int N, int h_kv, int G, int D, int topk, int block_size, int window_size,
                                int causal, int q_offset, float sm_scale, void* stream);

/* Sparse backward of the score gather.  Replaces the dense scatter + two torch.bmm of
 * SoftmaxTopKMaxPoolingFusedFn.backward (ops/topk_head_softmax.py:1040-1092).
 * g_scores (B,L,h_kv,G,topk) bf16 -> dq (B,L,h_kv,G,D) bf16 (written),
 * dlmk fp32 (B,N,h_kv or h_kv*G,D) (ACCUMULATED: caller zero-fills).
 * The chunk indices of one (query, KV head) row must be distinct (they are when they come from
 * the selection).  With D in {64, 128} and G (shared chunk keys) a divisor of 128 the two gradients
 * are two small dense MFMA products per block of 128 rows, over the rows' gradients scattered into
 * a dense tile in LDS; the chunk-key tiles of the query blocks are added with float atomics, so the
 * last bits of dlmk depend on the order the blocks finish in.  Other shapes:
 * workspace: device scratch of hils_topk_bwd_workspace(...) bytes (0 when none is needed); with it
 * the chunk-key gradient is summed chunk by chunk over an inverse index (no atomics); NULL selects
 * the atomic kernel. */
size_t hils_topk_bwd_workspace(int B, int L, int N, int h_kv, int G, int D, int topk);
int hils_topk_bwd(const void* g_scores, const void* q, const void* lmks, const int32_t* indices,
                  void* dq, float* dlmk, void* workspace, size_t workspace_bytes, int B, int L, int N,
                  int h_kv, int G, int D, int topk, int per_qhead, float sm_scale, void* stream);

/* ---- inter-chunk softmax (layer glue) ------------------------------------------ */

/* chunk_weights = softmax([scores_1..K (+ prior_b gathered at the indices), lse_swa (, 0)]).
 * Replaces the gather / cat / F.softmax glue of models/FlashHiLS/hils_attention.py:585-610.
 * scores (B,L,HQ,K) bf16; lse_swa (B,L,HQ) fp32, or bf16 when lse_bf16 != 0; prior_b (B,N,HQ)
 * fp32 or NULL; indices (B,L,H,K) int32 (needed with prior_b) -> weights (B,L,HQ,K+1(+1)) bf16, the
 * local-branch weight in column K, the softmax-1 sink (softmax1 != 0) in column K+1. */
int hils_chunk_weights(const void* scores, const void* lse_swa, int lse_bf16, const float* prior_b,
                       const int32_t* indices, void* weights, int B, int L, int HQ, int H, int N,
                       int K, int softmax1, void* stream);

/* Backward of hils_chunk_weights: the autograd of the same glue (F.softmax over the
 * concatenated columns, the gather of prior_b, models/FlashHiLS/hils_attention.py:585-610).
 * The forward's inputs again, d_weights (B,L,HQ,K+1(+1)) bf16 -> d_scores (B,L,HQ,K) bf16
 * (written), d_lse (B,L,HQ) fp32 (written) or NULL, d_prior_b (B,N,HQ) fp32 (ACCUMULATED with
 * atomics at the selected chunks: caller zero-fills) or NULL.  The probabilities are rebuilt in
 * fp32 from the inputs, not read back from the bf16 weights. */
int hils_chunk_weights_bwd(const void* scores, const void* lse_swa, int lse_bf16, const float* prior_b,
                           const int32_t* indices, const void* d_weights, void* d_scores, float* d_lse,
                           float* d_prior_b, int B, int L, int HQ, int H, int N, int K, int softmax1,
                           void* stream);

/* ---- sparse attention over the selected chunks ------------------------------ */

/* Forward.  Replaces hierarchical_sparse_attention_block_M_reuseIndices behind
 * _hils_block_M_attention_inverse.forward (ops/hils_fwd_bwd_head.py:198-496, :771-860)
 * and, with q_block > 1 / sm_n != 0 / mask_last == 0, _attn_fwd of ops/hsa_triton.py:77-197.
 * q (B,L,HQ,D), k (B,Lkv,H,D), v (B,Lkv,H,Dv) bf16; weights (B,L/q_block,WH,NW) bf16
 * with WH = HQ or H (first K of NW columns are read); indices (B,L/q_block,H,K) int32,
 * < 0 = empty slot; slope (HQ) fp32 or NULL.
 * Outputs: o (B,L,HQ,Dv) bf16; lse (B,L,HQ,K) fp32 per-chunk log2-domain LSE or NULL
 * (-inf for empty slots).
 * swa_o (B,L,HQ,Dv) bf16 or NULL: the local (sliding-window) branch's output; when given, the
 * layer's merge `torch.addcmul(hils_o, swa_o, chunk_weights[..., merge_col].unsqueeze(-1))`
 * (models/FlashHiLS/hils_attention.py:617-623) happens in the same call:
 * o = remote branch + swa_o * weights[..., merge_col], rounded once (merge_col = K for the plain
 * K+1-way softmax, NW-2 with the softmax-1 sink column).
 * workspace: device scratch of hils_sparse_attn_fwd_workspace(...) bytes; the MFMA path
 * keeps MFMA-operand-ordered copies of K and V there.  workspace_ready != 0 says the copies from
 * an earlier call (or from hils_pack_kv_chunks) on the same k and v are still valid and is not
 * rebuilt.  With workspace == NULL, or a size of 0 from the query, the shape-generic path
 * runs. */
size_t hils_sparse_attn_fwd_workspace(int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K,
                                      int WH, int q_block, int S, float sm_n);
int hils_sparse_attn_fwd(const void* q, const void* k, const void* v, const void* weights,
                         const int32_t* indices, const float* slope, const void* swa_o, void* o,
                         float* lse, void* workspace, size_t workspace_bytes, int workspace_ready, int B,
                         int L, int Lkv, int HQ, int H, int D, int Dv, int K, int NW, int WH, int q_block,
                         int S, float sm_scale, int mask_last, float sm_n, int merge_col, void* stream);
/* Fills a workspace of hils_sparse_attn_fwd_workspace(...) bytes on its own: per 64-token
 * chunk of a (batch, KV head), K and V rewritten in the register order of the MFMA operands
 * the prefill kernel loads (every operand load becomes one contiguous 1 KiB burst), followed
 * by max|V| of every chunk (fp32).  No counterpart in the reference (TileLang stages K/V
 * through shared memory on every use). */
int hils_pack_kv_chunks(const void* k, const void* v, void* workspace, size_t workspace_bytes, int B,
                        int Lkv, int H, int D, int Dv, void* stream);

/* Backward.  Replaces hierarchical_sparse_attention_bwd_dqkv_block_M_inverse
 * (ops/hils_fwd_bwd_head.py:506-766) and kernel_attn_bwd_dq / _attn_bwd_dkdv /
 * _fill_chunk_mask of ops/hsa_triton.py:201-597.
 * d_o (B,L,HQ,Dv) bf16, lse from the forward.
 * dq (B,L,HQ,D) bf16 (written); dk (B,Lkv,H,D) fp32, dv (B,Lkv,H,Dv) fp32 (ACCUMULATED
 * with atomics: caller zero-fills) - or, with kv_grad_bf16 != 0, bf16 tensors of those shapes that
 * the call OVERWRITES (every element; only with the workspace kernels, an error otherwise: they
 * sum a chunk's gradient in registers and write it once); dw fp32 (B,L/q_block,WH,NW) (accumulated with
 * atomics when q_block > 1 or WH != HQ, written otherwise: caller zero-fills).
 * workspace: device scratch of hils_sparse_attn_bwd_workspace(...) bytes (0 = shape not covered)
 * for the MFMA kernels: an inverse index (pairs of (query, slot) grouped by chunk) is built there
 * and dK, dV are then computed chunk-major without atomics.  NULL selects the shape-generic
 * kernel for everything.
 * swa_o / d_swa_o / merge_col: when the forward merged the local branch (swa_o given there), pass
 * the same swa_o and merge_col: d_swa_o (B,L,HQ,Dv) bf16 = d_o * weights[..., merge_col] is written
 * and dw[..., merge_col] = <d_o, swa_o> (q_block = 1, WH = HQ only).  NULL otherwise. */
size_t hils_sparse_attn_bwd_workspace(int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K,
                                      int WH, int q_block, int S, float sm_n);
int hils_sparse_attn_bwd(const void* q, const void* k, const void* v, const void* weights,
                         const int32_t* indices, const float* slope, const float* lse,
                         const void* d_o, void* dq, void* dk, void* dv, float* dw, void* workspace,
                         size_t workspace_bytes, int B, int L, int Lkv, int HQ, int H, int D, int Dv, int K, int NW,
                         int WH, int q_block, int S, float sm_scale, int mask_last, float sm_n,
                         const void* swa_o, void* d_swa_o, int merge_col, int kv_grad_bf16, void* stream);

/* fp32 tensors: the reference's dtype="float32" / accum_dtype="float" mode of HiLS_block_M_head
 * (ops/hils_fwd_bwd_head.py:928-964; its test_correctness_fp32, :1045-1126, runs in it).  Same
 * arguments as above with q, k, v, weights, d_o, o, dq as fp32 tensors; everything is computed in
 * fp32 (P is not rounded to bf16) on the shape-generic kernels (any D, Dv multiple of 8, any chunk
 * size, slope, HSA arguments); no workspace, no merged local branch.  dk, dv, dw as in
 * hils_sparse_attn_bwd without a workspace (fp32, ACCUMULATED: caller zero-fills). */
int hils_sparse_attn_fwd_f32(const float* q, const float* k, const float* v, const float* weights,
                             const int32_t* indices, const float* slope, float* o, float* lse, int B,
                             int L, int Lkv, int HQ, int H, int D, int Dv, int K, int NW, int WH,
                             int q_block, int S, float sm_scale, int mask_last, float sm_n, void* stream);
int hils_sparse_attn_bwd_f32(const float* q, const float* k, const float* v, const float* weights,
                             const int32_t* indices, const float* slope, const float* lse,
                             const float* d_o, float* dq, float* dk, float* dv, float* dw, int B, int L,
                             int Lkv, int HQ, int H, int D, int Dv, int K, int NW, int WH, int q_block,
                             int S, float sm_scale, int mask_last, float sm_n, void* stream);

/* ---- decode over a paged cache (page = chunk = 64 tokens) ------------------------------ */

/* The serving backend of the reference keeps the KV cache in pages of one chunk (README.md:262-264)
 * and the layer's per-chunk keys beside it (models/FlashHiLS/hils_attention.py:361-416,
 * utils/hils_cache_utils.py:8-76).  Layout here: k_pages, v_pages (num_pages, H, 64, D) bf16 (the 64
 * tokens of a (page, head) contiguous: one 16 KiB read per selected chunk and tensor at D = 128);
 * lmk_pages (num_pages, h_kv, D) bf16 = the pooled key of every page; page_table (B, max_pages)
 * int32 maps chunk c of batch element b to its page (negative or >= num_pages = unmapped: the chunk
 * is invisible to the selection and contributes nothing to the attention).
 *
 * hils_topk_fwd_weights_paged: selection + inter-chunk softmax as hils_topk_fwd_weights (no noise /
 * drop mask, causal), N = chunks of the sequence, L <= a few queries; per_qhead != 0: one pooled key per
 * query head, lmk_pages (num_pages, h_kv*G, D);
 * bias_pages (num_pages, h_kv*G) fp32 or NULL: the prior bias of every page (selection bias and the
 * bias of the inter-chunk softmax, as the layer uses it); lse_total / sel_logits optional as in
 * hils_topk_fwd.
 * hils_sparse_attn_decode_paged: hils_sparse_attn_fwd's decode path; indices are chunk numbers of the
 * sequence (what the selection returns).  workspace: hils_sparse_attn_decode_paged_workspace bytes
 * or NULL. */
int hils_topk_fwd_weights_paged(const void* q, const void* lmk_pages, const int32_t* page_table,
                                const float* lse_swa, const float* bias_pages, int32_t* indices, void* scores, void* weights,
                                float* lse_total, float* sel_logits, int B, int L, int N, int h_kv, int G,
                                int D, int topk, int block_size, int window_size, int q_offset,
                                int max_pages, int num_pages, float sm_scale, int per_qhead, void* stream);
size_t hils_sparse_attn_decode_paged_workspace(int B, int L, int HQ, int H, int D, int K);
int hils_sparse_attn_decode_paged(const void* q, const void* k_pages, const void* v_pages,
                                  const int32_t* page_table, const void* weights, const int32_t* indices,
                                  void* o, void* workspace, size_t workspace_bytes, int B, int L, int HQ, int H,
                                  int D, int K, int NW, int max_pages, int num_pages, float sm_scale,
                                  int mask_last, void* stream);

/* ---- the remote branch of a decode step in one launch ---------------------------------- */

/* hils_topk_fwd_weights followed by the decode path of hils_sparse_attn_fwd (contiguous cache) or
 * hils_topk_fwd_weights_paged followed by hils_sparse_attn_decode_paged (paged cache), fused: what
 * the layer runs per generated token between the local branch and the merge
 * (models/FlashHiLS/hils_attention.py:568-623 on the cached keys of utils/hils_cache_utils.py:34-62).
 * One workgroup per (query, KV head) row selects the row's chunks, writes indices / scores / weights
 * and then attends over the chunks it has selected: one launch instead of two, and the rows'
 * selection tails overlap other rows' memory streams.  Outputs as the two calls give them; o
 * (B,L,HQ,D) bf16 is the remote branch's output (the caller adds swa_o * weights[..., topk]).
 * lse_total / sel_logits optional as in hils_topk_fwd.  q (B,L,HQ,D); k, v (B,Lkv,H,D) with
 * Lkv >= N * 64 or k_pages, v_pages (num_pages,H,64,D).
 * Chunk keys: lmks (B,N,H,D), the layout of the reference's _hils_prior_cache; or, lmk_head_major != 0,
 * (B,H,lmk_cap,D) with lmk_cap >= N chunks allocated per (batch, head): the N keys a row streams are
 * then one contiguous block instead of 2*D-byte rows at a stride of H*2*D bytes (what this build's cache
 * layers keep).  The paged entry point takes lmk_pages (num_pages,H,D) addressed through the page
 * table, or, lmk_dense != 0, dense chunk keys in one of the two layouts above beside paged K and V.
 * lmk_per_qhead != 0: one chunk key per QUERY head (the layer's attention-pooled keys,
 * models/FlashHiLS/hils_attention.py:391-396): HQ heads in place of H in all three key layouts; a row
 * then streams HQ/H times the key bytes.
 * bias: the layer's prior bias (models/FlashHiLS/hils_attention.py:568-602: the selection's `bias`
 * and the bias gathered into the inter-chunk softmax), fp32, NULL for none; laid out like the chunk
 * keys with the G heads of a KV head in place of D: (B,N,H*G), (B,H,lmk_cap,G) or (num_pages,H*G).
 * Covered shapes (hils_decode_step_covers returns 1): causal, block_size 64,
 * D = Dv in {64, 128}, HQ/H <= 8, 256 <= N <= 4096 (with more than four query heads per KV head, whose
 * logits take eight rows of LDS: 2752 chunks at D = 128 and 3200 at D = 64, 2496 / 2880 with chunk keys
 * per page; the covers function knows), topk <= 64, at least 96 rows B*L*H.  A bias is staged in LDS
 * beside the logits; where the two do not fit side by side (from about 2900 chunks at D = 128, half of
 * that with eight head rows) it shares the logits' array and a winner's raw score is its biased logit
 * minus the bias (one fp32 rounding away from the product, far inside the bf16 it is returned in). */
int hils_decode_step_covers(int B, int L, int N, int HQ, int H, int D, int topk, int block_size, int with_bias);
int hils_decode_step(const void* q, const void* lmks, const void* k, const void* v, const float* lse_swa,
                     const float* bias, int32_t* indices, void* scores, void* weights, void* o,
                     float* lse_total, float* sel_logits, int B, int L, int Lkv, int N, int HQ, int H, int D,
                     int topk, int block_size, int window_size, int q_offset, float sm_scale_sel,
                     float sm_scale_attn, int mask_last, int lmk_head_major, int lmk_cap, int lmk_per_qhead,
                     void* stream);
int hils_decode_step_paged(const void* q, const void* lmk_pages, const void* k_pages, const void* v_pages,
                           const int32_t* page_table, const float* lse_swa, const float* bias, int32_t* indices,
                           void* scores, void* weights, void* o, float* lse_total, float* sel_logits, int B,
                           int L, int N, int HQ, int H, int D, int topk, int block_size, int window_size,
                           int q_offset, int max_pages, int num_pages, float sm_scale_sel, float sm_scale_attn,
                           int mask_last, int lmk_dense, int lmk_head_major, int lmk_cap, int lmk_per_qhead,
                           void* stream);

/* ---- exact per-chunk log Z ---------------------------------------------------- */

/* Forward.  Replaces exact_chunk_log_z_fwd (ops/exact_chunk_log_z_tilelang.py:25-137).
 * q (B,L,HQ,D), k (B,L,H,D) bf16 -> log_z (B,L,HQ,ceil(L/S)) fp32, every element
 * written (-inf where the chunk is not fully remote). */
int hils_chunk_logz_fwd(const void* q, const void* k, float* log_z, int B, int L, int HQ, int H,
                        int D, int S, int window, float sm_scale, int mask_lmk, void* stream);
/* Backward w.r.t. q.  Replaces exact_chunk_log_z_bwd_dq (:148-262).  dq bf16 (written). */
int hils_chunk_logz_bwd_dq(const void* q, const void* k, const float* log_z, const float* d_log_z,
                           void* dq, int B, int L, int HQ, int H, int D, int S, int window,
                           float sm_scale, void* stream);
/* Backward w.r.t. k.  Replaces exact_chunk_log_z_bwd_dk (:273-391) and the GQA sum of
 * :472-476.  dk bf16 (B,L,H,D) (written, already summed over the G heads). */
int hils_chunk_logz_bwd_dk(const void* q, const void* k, const float* log_z, const float* d_log_z,
                           void* dk, int B, int L, int HQ, int H, int D, int S, int window,
                           float sm_scale, void* stream);

/* ---- sliding-window attention of the local branch ------------------------------- */

/* Forward.  Replaces flex_attn_fwd (ops/flex_attn_tilelang.py:26-267) behind flex_attn_tl
 * (:1261-1310).  q (B,Lq,HQ,D), k (B,Lk,H,D), v (B,Lk,H,Dv) bf16, Lq <= Lk; query t sits at the
 * absolute position kv_start + Lk - Lq + t, key j at kv_start + j.  A query sees the keys from
 * chunk_start to itself, chunk_start = floor((pos - window + 1) / chunk) * chunk when
 * expand_to_chunk, else pos - window + 1; with mask_lmk the keys with (pos + 1) % chunk == 0 are
 * excluded.  Writes o (B,Lq,HQ,Dv) bf16 and lse (B,Lq,HQ) fp32 in natural-log units (the
 * reference's kernel writes log2 units and converts at :1307-1309); rows that see no key get
 * o = 0, lse = -inf.  D, Dv in {64,128}; HQ/H in {1,2,4,8,16}. */
int hils_swa_fwd(const void* q, const void* k, const void* v, void* o, float* lse, int B, int Lq,
                 int Lk, int HQ, int H, int D, int Dv, int window, int chunk, int mask_lmk,
                 int expand_to_chunk, int kv_start, float sm_scale, void* stream);

/* Backward (training: Lq == Lk = L, kv_start = 0).  Replaces flex_attn_bwd_preprocess,
 * flex_attn_bwd_dq and flex_attn_bwd_dkdv (ops/flex_attn_tilelang.py:270-1153) as driven by
 * _FlexAttnTL.backward.  o, lse: the forward's outputs (lse in natural-log units); d_o bf16;
 * d_lse (B,L,HQ) fp32 gradient of lse, may be NULL (= 0).  Writes dq (B,L,HQ,D), dk (B,L,H,D),
 * dv (B,L,H,Dv) bf16 (every element, dk/dv already summed over the heads of a group) and uses
 * delta (B,L,HQ) fp32 as scratch (sum_d o*d_o - d_lse). */
int hils_swa_bwd(const void* q, const void* k, const void* v, const void* o, const float* lse,
                 const void* d_o, const float* d_lse, void* dq, void* dk, void* dv, float* delta,
                 int B, int L, int HQ, int H, int D, int Dv, int window, int chunk, int mask_lmk,
                 int expand_to_chunk, float sm_scale, void* stream);

/* ---- rotary position embedding ---------------------------------------------------- */

/* Replaces rope_fwd_kernel and single_tensor_rope_kernel (ops/rope_tilelang_fp32.py:19-81,
 * :96-137).  x, out (B,L,H,D) bf16, D a multiple of 16; with x = (x1, x2) the two halves of a
 * head vector: out1 = x1*cos[d] - x2*sin[d]*sin_sign, out2 = x2*cos[d'] + x1*sin[d']*sin_sign,
 * d' = d (lo_only != 0, the two-tensor kernel) or d + D/2 (the single-tensor kernel).  Tables
 * cos_t, sin_t: (L,D), or (B,L,D) when table_per_batch != 0; fp32 when table_f32 != 0, else bf16.
 * sin_sign = -1 gives the backward (rotation by the opposite angle). */
int hils_rope(const void* x, const void* cos_t, const void* sin_t, void* out, int B, int L, int H,
              int D, int table_per_batch, int table_f32, int lo_only, float sin_sign, void* stream);

/* Key (or query) preparation in one pass: per-head RMS norm, rotary embedding and the mean over
 * every chunk.  Replaces the layer's sequence k_norm (models/FlashHiLS/hils_attention.py:314-321 with
 * rms_norm of models/FlashHiLS/modeling_qwen_hils.py:80-86), apply_rotary_pos_emb
 * (hils_attention.py:144-171, called at :479-483) and k_chunked.mean(dim=2) (:398,:460), which
 * otherwise read and write the tensor once per step.
 * x, out (B,L,H,D) bf16, D in {64,128,256}; norm_weight (D) bf16 or NULL (no norm); cos_t, sin_t
 * (L,D) bf16 - (B,L,D) when table_per_batch != 0 - or both NULL (no rotation):
 *   y = bf16(x * rsqrt(mean_d x^2 + eps)); z = bf16(norm_weight * y);
 *   out = bf16(bf16(z*cos) + bf16(rotate_half(z)*sin)), rotate_half(z) = (-z_hi, z_lo);
 *   lmk[b,n,h,:] = bf16(mean_s out[b,nS+s,h,:]) for the L/S whole chunks; lmk (B,L/S,H,D) bf16 or NULL.
 * Backward: d_out (B,L,H,D) bf16 and/or d_lmk (B,L/S,H,D) bf16 -> dx bf16 (written), d_weight (D) fp32
 * (ADDED to with float atomics: caller zero-fills; required when norm_weight is given). */
int hils_norm_rope_pool_fwd(const void* x, const void* norm_weight, const void* cos_t, const void* sin_t,
                            void* out, void* lmk, int B, int L, int H, int D, int S, int table_per_batch,
                            float eps, void* stream);
int hils_norm_rope_pool_bwd(const void* x, const void* norm_weight, const void* cos_t, const void* sin_t,
                            const void* d_out, const void* d_lmk, void* dx, float* d_weight, int B, int L,
                            int H, int D, int S, int table_per_batch, float eps, void* stream);

#ifdef __cplusplus
}
#endif
#endif
