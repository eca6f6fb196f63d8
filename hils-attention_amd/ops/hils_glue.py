"""Fused inter-chunk softmax of the HiLS layer (forward and backward).

The reference computes it with torch ops inside the layer
(models/FlashHiLS/hils_attention.py:585-610): gather the prior bias at the selected chunks,
add it to the scores, concatenate the local-branch LSE (and a zero logit when
``enable_softmax1``), softmax, cast to the hidden dtype.  ``chunk_weights`` does that in one
kernel; column K is the weight of the local (sliding-window) branch.
"""
import torch

from . import _cabi


class _ChunkWeightsFn(torch.autograd.Function):
    """softmax([scores (+ prior_b at the indices), lse_swa (, 0)]) with its backward, one kernel each."""

    @staticmethod
    def forward(ctx, scores, lse_swa, prior_b, indices, softmax1):
        B, L, HQ, K = scores.shape
        sc = scores.contiguous()
        lse = lse_swa.reshape(B, L, HQ).contiguous()
        if lse.dtype not in (torch.bfloat16, torch.float32):
            lse = lse.float()
        H, N = HQ, 1
        pb = idx = None
        if prior_b is not None:
            assert indices is not None, "prior_b needs the selected indices"
            H = indices.shape[2]
            N = prior_b.shape[1]
            assert prior_b.shape == (B, N, HQ), f"prior_b shape {tuple(prior_b.shape)} != {(B, N, HQ)}"
            assert indices.shape == (B, L, H, K)
            pb = prior_b.float().contiguous()
            idx = indices.to(torch.int32).contiguous()
        out = torch.empty((B, L, HQ, K + 1 + int(softmax1)), dtype=scores.dtype, device=scores.device)
        _cabi.call("hils_chunk_weights", _cabi.ptr(sc), _cabi.ptr(lse), int(lse.dtype == torch.bfloat16),
                   _cabi.ptr(pb), _cabi.ptr(idx), _cabi.ptr(out), B, L, HQ, H, N, K, int(softmax1))
        ctx.save_for_backward(sc, lse, pb, idx)
        ctx.cfg = (B, L, HQ, H, N, K, int(softmax1))
        ctx.lse_meta = (lse_swa.shape, lse_swa.dtype)
        ctx.prior_dtype = None if prior_b is None else prior_b.dtype
        return out

    @staticmethod
    def backward(ctx, d_w):
        sc, lse, pb, idx = ctx.saved_tensors
        B, L, HQ, H, N, K, softmax1 = ctx.cfg
        d_w = d_w.to(sc.dtype).contiguous()
        d_sc = torch.empty_like(sc)
        d_lse = torch.empty((B, L, HQ), dtype=torch.float32, device=sc.device) if ctx.needs_input_grad[1] else None
        d_pb = None
        if pb is not None and ctx.needs_input_grad[2]:
            d_pb = torch.zeros_like(pb)
        _cabi.call("hils_chunk_weights_bwd", _cabi.ptr(sc), _cabi.ptr(lse), int(lse.dtype == torch.bfloat16),
                   _cabi.ptr(pb), _cabi.ptr(idx), _cabi.ptr(d_w), _cabi.ptr(d_sc), _cabi.ptr(d_lse),
                   _cabi.ptr(d_pb), B, L, HQ, H, N, K, softmax1)
        if d_lse is not None:
            shape, dtype = ctx.lse_meta
            d_lse = d_lse.reshape(shape).to(dtype)
        if d_pb is not None:
            d_pb = d_pb.to(ctx.prior_dtype)
        return d_sc, d_lse, d_pb, None, None


def chunk_weights(scores, lse_swa, prior_b=None, indices=None, enable_softmax1=False):
    """scores (B,L,HQ,K) bf16, lse_swa (B,L,HQ) -> weights (B,L,HQ,K+1(+1)) bf16.
    ``prior_b`` (B,N,HQ) with ``indices`` (B,L,H,K) adds the gathered prior bias first.
    Differentiable in scores, lse_swa and prior_b."""
    _cabi.require_gpu_bf16("chunk_weights", scores)
    return _ChunkWeightsFn.apply(scores, lse_swa, prior_b, indices, bool(enable_softmax1))


def _prior_bias(prior_b, B, N, h_q):
    """The layer's prior bias as a contiguous fp32 (B, N, h_q) tensor (None stays None)."""
    if prior_b is None:
        return None
    assert prior_b.numel() == B * N * h_q and prior_b.shape[0] == B and prior_b.shape[1] == N, (
        f"prior_b shape {tuple(prior_b.shape)} must be ({B}, {N}, {h_q})")
    return prior_b.reshape(B, N, h_q).float().contiguous()


def topk_chunk_weights(q, lmks, lse_swa, topk, block_size, window_size, is_causal=True, q_offset=0,
                       sm_scale=None, prior_b=None, num_kv_heads=None):
    """Inference: ``online_softmax_topk_head`` (no Gumbel / drop mask) followed by ``chunk_weights``
    in one call, for the serving loop.  q (B,L,h_q,D) bf16, lmks (B,N,h_kv,D) bf16 (one chunk key per
    KV head) or, with ``num_kv_heads`` given, (B,N,h_q,D) (one per query head, the layer's
    attention-pooled keys), lse_swa (B,L,h_q) -> indices (B,L,h_kv,topk) int32, scores (B,L,h_q,topk)
    bf16, weights (B,L,h_q,topk+1) bf16.  ``prior_b`` (B,N,h_q): the layer's prior bias (its
    ``enable_prior_query`` mode, models/FlashHiLS/hils_attention.py:568-602), used as the selection's
    ``bias`` and gathered into the softmax.  With about one (query, KV head) row per compute unit the
    selection kernel writes the weights itself; otherwise two kernels run."""
    import math
    _cabi.require_gpu_bf16("topk_chunk_weights", q, lmks)
    if torch.is_grad_enabled() and (q.requires_grad or lmks.requires_grad or lse_swa.requires_grad):
        raise RuntimeError("topk_chunk_weights is forward-only")
    B, L, h_q, D = q.shape
    N, h_lmk = lmks.shape[1], lmks.shape[2]
    h_kv = h_lmk if num_kv_heads is None else int(num_kv_heads)
    assert lmks.shape[0] == B and lmks.shape[3] == D
    assert h_q % h_kv == 0, f"h_q ({h_q}) must be divisible by h_kv ({h_kv})"
    assert h_lmk in (h_kv, h_q), f"lmks carries {h_lmk} heads: neither the {h_kv} KV heads nor the {h_q} query heads"
    per_qhead = int(h_lmk != h_kv)
    G = h_q // h_kv
    scale = float(sm_scale) if sm_scale is not None else 1.0 / math.sqrt(D)
    dev = q.device
    pb = _prior_bias(prior_b, B, N, h_q)
    indices = torch.empty((B, L, h_kv, topk), dtype=torch.int32, device=dev)
    scores = torch.empty((B, L, h_q, topk), dtype=q.dtype, device=dev)
    weights = torch.empty((B, L, h_q, topk + 1), dtype=q.dtype, device=dev)
    ws = _cabi.topk_fwd_workspace(dev, B, L, N, h_kv, G)
    if (lse_swa.dtype == torch.bfloat16 and ws is not None and not per_qhead
            and _cabi.load().hils_topk_lse16_covers(B, L, N, h_kv, G, D, int(topk))):
        # lse_swa as the layer hands it over (bf16): read in place, no conversion pass
        _cabi.call("hils_topk_fwd_weights_lse16", _cabi.ptr(q.contiguous()), _cabi.ptr(lmks.contiguous()),
                   _cabi.ptr(lse_swa.reshape(B, L, h_q).contiguous()), _cabi.ptr(pb), _cabi.ptr(pb),
                   _cabi.ptr(indices), _cabi.ptr(scores), _cabi.ptr(weights), _cabi.ptr(ws), _cabi.nbytes(ws),
                   B, L, N, h_kv, G, D, int(topk), int(block_size), int(window_size), int(bool(is_causal)),
                   int(q_offset), scale)
        return indices, scores, weights
    lse = lse_swa.reshape(B, L, h_q).float().contiguous()
    _cabi.call("hils_topk_fwd_weights", _cabi.ptr(q.contiguous()), _cabi.ptr(lmks.contiguous()),
               _cabi.ptr(lse), _cabi.ptr(pb), _cabi.ptr(pb), None, None, _cabi.ptr(indices), _cabi.ptr(scores),
               _cabi.ptr(weights), _cabi.ptr(ws), _cabi.nbytes(ws), B, L, N, h_kv, G, D, int(topk),
               int(block_size), int(window_size), int(bool(is_causal)), int(q_offset), per_qhead, scale)
    return indices, scores, weights


def head_major_chunk_keys(lmks, prior_b=None, capacity=None, num_kv_heads=None):
    """Chunk keys (B,N,h,D) (and the prior bias (B,N,h_q)) re-laid head-major, (B,h,cap,D) and
    (B,h_kv,cap,G): the N keys a decode row streams become one contiguous block.  What this
    package's cache layers keep; ``decode_step(..., lmk_head_major=True)`` takes them.  ``num_kv_heads``:
    needed for the bias when lmks carries one key per query head (h = h_q)."""
    B, N, h, D = lmks.shape
    cap = N if capacity is None else int(capacity)
    assert cap >= N
    out = torch.zeros((B, h, cap, D), dtype=lmks.dtype, device=lmks.device)
    out[:, :, :N] = lmks.permute(0, 2, 1, 3)
    if prior_b is None:
        return out
    h_kv = h if num_kv_heads is None else int(num_kv_heads)
    G = prior_b.shape[2] // h_kv
    pb = torch.zeros((B, h_kv, cap, G), dtype=torch.float32, device=lmks.device)
    pb[:, :, :N] = prior_b.reshape(B, N, h_kv, G).permute(0, 2, 1, 3).float()
    return out, pb


def decode_step(q, lmks, k, v, lse_swa, topk, block_size, window_size, q_offset=0, sm_scale=None,
                mask_last_token=True, _debug=None, prior_b=None, lmk_head_major=False, num_chunks=None):
    """Inference: the remote branch of a decode step, ``topk_chunk_weights`` followed by
    ``HiLS_block_M_head(..., is_training=False)`` on the selected chunks, in one kernel launch (one
    workgroup per (query, KV head) selects and then attends).  q (B,L,h_q,D), lmks (B,N,h_kv,D), k, v
    (B,Lkv,h_kv,D) bf16 (k, v may live in pinned host memory), lse_swa (B,L,h_q) -> o (B,L,h_q,D),
    weights (B,L,h_q,topk+1), indices (B,L,h_kv,topk), scores (B,L,h_q,topk).  ``prior_b`` (B,N,h_q):
    the layer's prior bias (selection bias and the bias of the inter-chunk softmax).
    ``lmk_head_major``: lmks is (B,h_kv,cap,D) and prior_b (B,h_kv,cap,G) (``head_major_chunk_keys``),
    of which the first ``num_chunks`` (default cap) chunks are looked at.  lmks may carry h_q heads
    instead of h_kv (one chunk key per query head, the layer's attention-pooled keys): (B,N,h_q,D) or,
    head-major, (B,h_q,cap,D).  Shapes the fused kernel does not take (few rows, short caches, more
    than eight query heads per KV head, ...) run as the two calls."""
    import math
    from .hils_fwd_bwd_head import HiLS_block_M_head
    _cabi.require_gpu_bf16("decode_step", q, lmks)
    _cabi.require_gpu_bf16("decode_step", k, v, pinned_ok=True)
    if torch.is_grad_enabled() and any(t.requires_grad for t in (q, lmks, k, v, lse_swa)):
        raise RuntimeError("decode_step is forward-only")
    B, L, h_q, D = q.shape
    h_kv = k.shape[2]
    if lmk_head_major:
        h_lmk, cap = lmks.shape[1], lmks.shape[2]
        N = cap if num_chunks is None else int(num_chunks)
        assert 0 < N <= cap
    else:
        N, h_lmk = lmks.shape[1], lmks.shape[2]
        cap = N
        assert num_chunks is None or int(num_chunks) == N
    Lkv = k.shape[1]
    assert lmks.shape[0] == B and lmks.shape[3] == D and k.shape == v.shape and k.shape[0] == B
    assert k.shape[3] == D and h_q % h_kv == 0
    assert h_lmk in (h_kv, h_q), f"lmks carries {h_lmk} heads: neither the {h_kv} KV heads nor the {h_q} query heads"
    per_qhead = int(h_lmk != h_kv)
    G = h_q // h_kv
    scale = float(sm_scale) if sm_scale is not None else 1.0 / math.sqrt(D)
    lib = _cabi.load()
    pb = None
    if prior_b is not None:
        if lmk_head_major:
            assert prior_b.shape == (B, h_kv, cap, G), f"prior_b shape {tuple(prior_b.shape)} != {(B, h_kv, cap, G)}"
            pb = prior_b.float().contiguous()
        else:
            pb = _prior_bias(prior_b, B, N, h_q)
    if not (lib.hils_decode_step_covers(B, L, N, h_q, h_kv, D, int(topk), int(block_size), int(pb is not None))
            and Lkv >= N * block_size):
        if lmk_head_major:  # the two-call kernels read the reference's layout
            lmks = lmks[:, :, :N].permute(0, 2, 1, 3).contiguous()
            if pb is not None:
                pb = pb[:, :, :N].permute(0, 2, 1, 3).reshape(B, N, h_q).contiguous()
        idx, sc, w = topk_chunk_weights(q, lmks, lse_swa, topk, block_size, window_size, q_offset=q_offset,
                                        sm_scale=scale, prior_b=pb, num_kv_heads=h_kv)
        o = HiLS_block_M_head(q, k, v, w, idx, block_size=block_size, sm_scale=scale,
                              mask_last_token=mask_last_token, is_training=False)
        return o, w, idx, sc
    dev = q.device
    lse = lse_swa.reshape(B, L, h_q).float().contiguous()
    indices = torch.empty((B, L, h_kv, topk), dtype=torch.int32, device=dev)
    scores = torch.empty((B, L, h_q, topk), dtype=q.dtype, device=dev)
    weights = torch.empty((B, L, h_q, topk + 1), dtype=q.dtype, device=dev)
    o = torch.empty((B, L, h_q, D), dtype=q.dtype, device=dev)
    lse_total = sel_logits = None
    if _debug is not None:
        lse_total = torch.empty((B, L, h_kv, G), dtype=torch.float32, device=dev)
        sel_logits = torch.full((B, L, h_kv, G, N), float("-inf"), dtype=torch.float32, device=dev)
    kk, vv = _cabi.gpu_readable(k, dev), _cabi.gpu_readable(v, dev)
    _cabi.call("hils_decode_step", _cabi.ptr(q.contiguous()), _cabi.ptr(lmks.contiguous()), _cabi.ptr(kk),
               _cabi.ptr(vv), _cabi.ptr(lse), _cabi.ptr(pb), _cabi.ptr(indices), _cabi.ptr(scores),
               _cabi.ptr(weights), _cabi.ptr(o), _cabi.ptr(lse_total), _cabi.ptr(sel_logits), B, L, Lkv, N, h_q,
               h_kv, D, int(topk), int(block_size), int(window_size), int(q_offset), scale, scale,
               int(bool(mask_last_token)), int(bool(lmk_head_major)), cap, per_qhead)
    if _debug is not None:
        _debug.update(lse_total=lse_total, sel_logits=sel_logits)
    return o, weights, indices, scores
