"""Top-k chunk selection (drop-in for the reference's ops/topk_head_softmax.py).

``online_softmax_topk_head`` keeps the call signature of ops/topk_head_softmax.py:1212-1228.
One fused HIP kernel replaces the reference's LSE / select / sort / score-recompute kernel
sequence; the backward of the returned scores is sparse (no dense (L x N) scatter).
Selection order: score descending, lower chunk index wins a tie; indices come back sorted
ascending with -1 padding.
"""
import math

import torch

from . import _cabi


class SoftmaxTopKMaxPoolingFusedFn(torch.autograd.Function):
    """Mirrors SoftmaxTopKMaxPoolingFusedFn (ops/topk_head_softmax.py:975-1092)."""

    @staticmethod
    def forward(ctx, q, lmks, lse_swa, topk, block_size, window_size, is_causal, q_offset,
                drop_mask, sm_scale, bias, gumbel_noise, per_qhead_lmks, debug):
        B, L, h_kv, G, D = q.shape
        B2, N, lmks_h, D2 = lmks.shape
        assert B == B2 and D == D2
        if per_qhead_lmks:
            assert lmks_h == h_kv * G, (
                f"per_qhead_lmks expects lmks h dim = h_kv*G ({h_kv * G}), got {lmks_h}")
        else:
            assert lmks_h == h_kv, f"default mode expects lmks h dim = h_kv ({h_kv}), got {lmks_h}"
        _cabi.require_gpu_bf16("online_softmax_topk_head", q, lmks)
        q_in = q.contiguous()
        k_in = lmks.contiguous()
        lse_in = lse_swa.reshape(B, L, h_kv, G).float().contiguous()
        dev = q.device
        scale = float(sm_scale) if sm_scale is not None else 1.0 / math.sqrt(D)
        indices = torch.empty((B, L, h_kv, topk), dtype=torch.int32, device=dev)
        scores = torch.empty((B, L, h_kv, G, topk), dtype=q.dtype, device=dev)
        lse_total = sel_logits = None
        if debug is not None:
            lse_total = torch.empty((B, L, h_kv, G), dtype=torch.float32, device=dev)
            sel_logits = torch.full((B, L, h_kv, G, N), float("-inf"), dtype=torch.float32, device=dev)
        if drop_mask is not None:
            assert drop_mask.shape == (B, L, N), f"drop_mask shape {tuple(drop_mask.shape)} != {(B, L, N)}"
            drop_mask = drop_mask.to(torch.int32).contiguous()
        ws = None
        if debug is None or not debug.get("no_workspace"):  # test hook: keep the one-kernel path
            ws = _cabi.topk_fwd_workspace(dev, B, L, N, h_kv, G)
        _cabi.call("hils_topk_fwd", _cabi.ptr(q_in), _cabi.ptr(k_in), _cabi.ptr(lse_in),
                   _cabi.ptr(bias), _cabi.ptr(gumbel_noise), _cabi.ptr(drop_mask),
                   _cabi.ptr(indices), _cabi.ptr(scores), _cabi.ptr(lse_total),
                   _cabi.ptr(sel_logits), _cabi.ptr(ws), _cabi.nbytes(ws), B, L, N, h_kv, G, D, int(topk), int(block_size),
                   int(window_size), int(bool(is_causal)), int(q_offset), int(bool(per_qhead_lmks)),
                   scale)
        if debug is not None:
            debug["lse_total"] = lse_total
            debug["sel_logits"] = sel_logits
        ctx.save_for_backward(q_in, k_in, indices)
        ctx.cfg = (B, L, N, h_kv, G, D, int(topk), bool(per_qhead_lmks), scale)
        ctx.mark_non_differentiable(indices)
        return indices, scores

    @staticmethod
    def backward(ctx, grad_indices_unused, grad_scores):
        q_in, k_in, indices = ctx.saved_tensors
        B, L, N, h_kv, G, D, topk, per_qhead, scale = ctx.cfg
        gs = grad_scores.to(q_in.dtype).contiguous()
        dq = torch.empty_like(q_in)
        dlmk = torch.zeros(k_in.shape, dtype=torch.float32, device=k_in.device)
        ws = _cabi.topk_bwd_workspace(q_in.device, B, L, N, h_kv, G, D, topk)
        _cabi.call("hils_topk_bwd", _cabi.ptr(gs), _cabi.ptr(q_in), _cabi.ptr(k_in),
                   _cabi.ptr(indices), _cabi.ptr(dq), _cabi.ptr(dlmk), _cabi.ptr(ws), _cabi.nbytes(ws), B, L, N, h_kv, G, D, topk,
                   int(per_qhead), scale)
        return (dq, dlmk.to(k_in.dtype)) + (None,) * 12


def _bias_per_group(bias, B, N, h_kv, G, device):
    """Additive selection bias as a contiguous fp32 (B, N, h_kv, G) tensor, or None.
    Accepts the flat per-query-head form (B, N, h_q) and the grouped form (B, N, h_kv, G)."""
    if bias is None:
        return None
    want = {3: (B, N, h_kv * G), 4: (B, N, h_kv, G)}.get(bias.dim())
    if want is None:
        raise AssertionError(f"bias must be [B, S, h_q] or [B, S, h_kv, G], got {tuple(bias.shape)}")
    assert tuple(bias.shape) == want, f"bias shape {tuple(bias.shape)} != {want}"
    return bias.to(device=device, dtype=torch.float32).reshape(B, N, h_kv, G).contiguous()


def _gumbel_rows(use_gumbel, noise, is_training, h_q, N, device):
    """Gumbel noise per (query head, chunk) as fp32 (1, 1, h_q, N), or None when sampling is off.
    Given noise is used as it is (no gradient); otherwise -log(-log(u)) is drawn here."""
    if not use_gumbel and noise is None:
        return None
    assert is_training, "gumbel_noise is only supported in training mode"
    want = (1, 1, h_q, N)
    if noise is not None:
        assert tuple(noise.shape) == want, f"gumbel_noise shape {tuple(noise.shape)} != {want}"
        return noise.detach().to(device=device, dtype=torch.float32).contiguous()
    u = torch.rand(want, device=device, dtype=torch.float32).clamp_(min=1e-20, max=1 - 1e-7)
    return u.log_().neg_().log_().neg_()


class SoftmaxTopKMaxPooling_Fused(torch.nn.Module):
    """Mirrors SoftmaxTopKMaxPooling_Fused (ops/topk_head_softmax.py:1095-1207): the selection
    settings are fixed at construction, forward takes q (B,L,h_kv,G,D), chunk keys, lse_swa."""

    def __init__(self, topk, block_size, window_size, is_causal, is_training=True,
                 use_drop_mask=False, per_qhead_lmks=False):
        super().__init__()
        self.topk, self.block_size, self.window_size = topk, block_size, window_size
        self.is_causal, self.is_training = is_causal, is_training
        self.use_drop_mask, self.per_qhead_lmks = use_drop_mask, per_qhead_lmks

    def forward(self, q, lmks, lse_swa, q_offset, drop_mask=None, sm_scale=None, bias=None,
                use_gumbel=False, gumbel_noise=None, _debug=None):
        B, L, h_kv, G, D = q.shape
        N = lmks.shape[1]
        bias_arg = _bias_per_group(bias, B, N, h_kv, G, q.device)
        gumbel_arg = _gumbel_rows(use_gumbel, gumbel_noise, self.is_training, h_kv * G, N, q.device)
        # the reference's training-mode kernels take the query offset as 0 whatever is passed
        # (ops/topk_head_softmax.py:246,492)
        q_off = 0 if self.is_training else int(q_offset)
        indices, scores = SoftmaxTopKMaxPoolingFusedFn.apply(
            q, lmks, lse_swa, self.topk, self.block_size, self.window_size, self.is_causal, q_off,
            drop_mask, sm_scale, bias_arg, gumbel_arg, self.per_qhead_lmks, _debug)
        return indices, scores.view(B, L, h_kv * G, -1)


_SOFTMAX_MODULE_CACHE = {}


def _group_heads(q, lmks, lse_swa, G):
    """Bring the accepted input forms to one: q (B,L,h_kv,g,D), lmks (B,N,h_lmk,D), lse_swa
    (B,L,h_kv,g), plus whether every query head has chunk keys of its own.

    q may come flat (B,L,h_q,D) or grouped (B,L,h_kv,g,D).  Chunk keys whose last dimension is a
    multiple of q's are split into that many heads.  ``G == 1``: the chunk keys are shared by the
    heads of a group (h_lmk == h_kv; a flat q is grouped by h_q // h_lmk) or, for a grouped q
    only, h_lmk == h_q selects per-head keys.  ``G > 1``: per-head keys, h_lmk == h_q, and q is
    regrouped into h_q // G groups of G heads."""
    B, L, D = q.shape[0], q.shape[1], q.shape[-1]
    flat = q.dim() == 4
    h_q = q.shape[2] if flat else q.shape[2] * q.shape[3]
    if lmks.shape[3] != D:
        assert lmks.shape[3] % D == 0, f"lmks D dim ({lmks.shape[3]}) must be divisible by q D dim ({D})"
        lmks = lmks.reshape(lmks.shape[0], lmks.shape[1], -1, D)
    h_lmk = lmks.shape[2]
    if G > 1:
        assert h_lmk == h_q, f"when G>1, lmks must have h_q ({h_q}) heads, got {h_lmk}"
        assert h_q % G == 0, f"h_q ({h_q}) must be divisible by G ({G})"
        h_kv, g, per_qhead = h_q // G, G, True
    elif flat:
        assert h_q % h_lmk == 0, f"h_q ({h_q}) must be divisible by lmks_h ({h_lmk})"
        h_kv, g, per_qhead = h_lmk, h_q // h_lmk, False
    else:
        h_kv, g = q.shape[2], q.shape[3]
        if h_lmk not in (h_kv, h_q):
            raise AssertionError(f"lmks_h ({h_lmk}) must be h_kv ({h_kv}) or h_q ({h_q})")
        per_qhead = h_lmk != h_kv
    return q.reshape(B, L, h_kv, g, D), lmks, lse_swa.reshape(B, L, h_kv, g), per_qhead


def online_softmax_topk_head(q, lmks, lse_swa, topk, block_size, window_size, is_causal=True,
                             q_offset=0, is_training=True, drop_mask=None, sm_scale=None, bias=None,
                             use_gumbel=False, gumbel_noise=None, G=1, _debug=None):
    """Per-(query, KV head) top-k chunk selection.

    q (B,L,h_q,D) or (B,L,h_kv,G,D) bf16; lmks (B,N,h_lmk,D) bf16 with h_lmk = h_kv (shared,
    ``G == 1``) or h_q (per-q-head lmks, pass ``G``); lse_swa (B,L,h_q) or (B,L,h_kv,G).
    Returns indices (B,L,h_kv,topk) int32 ascending with -1 padding and scores
    (B,L,h_q,topk) in q's dtype: raw sm_scale*<q,lmk> (no bias / Gumbel), -inf at -1.
    Argument meaning and shape checks follow ops/topk_head_softmax.py:1291-1367.
    ``_debug`` (a dict) additionally receives the fp32 ``sel_logits`` and ``lse_total`` the
    selection was made from.
    """
    q, lmks, lse_swa, per_qhead = _group_heads(q, lmks, lse_swa, G)
    key = (topk, block_size, window_size, is_causal, is_training, drop_mask is not None, per_qhead)
    mod = _SOFTMAX_MODULE_CACHE.get(key)
    if mod is None:
        mod = _SOFTMAX_MODULE_CACHE[key] = SoftmaxTopKMaxPooling_Fused(*key)
    return mod(q, lmks, lse_swa, q_offset=q_offset, drop_mask=drop_mask, sm_scale=sm_scale,
               bias=bias, use_gumbel=use_gumbel, gumbel_noise=gumbel_noise, _debug=_debug)
