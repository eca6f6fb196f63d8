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
                   _cabi.ptr(sel_logits), _cabi.ptr(ws), B, L, N, h_kv, G, D, int(topk), int(block_size),
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
                   _cabi.ptr(indices), _cabi.ptr(dq), _cabi.ptr(dlmk), _cabi.ptr(ws), B, L, N, h_kv, G, D, topk,
                   int(per_qhead), scale)
        return (dq, dlmk.to(k_in.dtype)) + (None,) * 12


class SoftmaxTopKMaxPooling_Fused(torch.nn.Module):
    """Mirrors SoftmaxTopKMaxPooling_Fused (ops/topk_head_softmax.py:1095-1207)."""

    def __init__(self, topk, block_size, window_size, is_causal, is_training=True,
                 use_drop_mask=False, per_qhead_lmks=False):
        super().__init__()
        self.topk = topk
        self.block_size = block_size
        self.window_size = window_size
        self.is_causal = is_causal
        self.is_training = is_training
        self.use_drop_mask = use_drop_mask
        self.per_qhead_lmks = per_qhead_lmks

    def forward(self, q, lmks, lse_swa, q_offset, drop_mask=None, sm_scale=None, bias=None,
                use_gumbel=False, gumbel_noise=None, _debug=None):
        B, L, h_kv, G, D = q.shape
        N = lmks.shape[1]
        bias_arg = None
        if bias is not None:
            bias_arg = bias.to(device=q.device, dtype=torch.float32)
            if bias_arg.dim() == 3:
                assert bias_arg.shape == (B, N, h_kv * G), (
                    f"bias shape {tuple(bias_arg.shape)} != ({B}, {N}, {h_kv * G})")
                bias_arg = bias_arg.reshape(B, N, h_kv, G).contiguous()
            elif bias_arg.dim() == 4:
                assert bias_arg.shape == (B, N, h_kv, G), (
                    f"bias shape {tuple(bias_arg.shape)} != ({B}, {N}, {h_kv}, {G})")
                bias_arg = bias_arg.contiguous()
            else:
                raise AssertionError(
                    f"bias must be [B, S, h_q] or [B, S, h_kv, G], got {tuple(bias_arg.shape)}")
        use_gumbel = bool(use_gumbel) or (gumbel_noise is not None)
        gumbel_arg = None
        if use_gumbel:
            assert self.is_training, "gumbel_noise is only supported in training mode"
            if gumbel_noise is None:
                u = torch.rand(1, 1, h_kv * G, N, device=q.device, dtype=torch.float32)
                u.clamp_(min=1e-20, max=1 - 1e-7)
                gumbel_arg = -torch.log(-torch.log(u))
            else:
                assert gumbel_noise.shape == (1, 1, h_kv * G, N), (
                    f"gumbel_noise shape {tuple(gumbel_noise.shape)} != ({1}, {1}, {h_kv * G}, {N})")
                gumbel_arg = gumbel_noise.detach().to(device=q.device, dtype=torch.float32).contiguous()
        # the reference's training-mode kernels take the query offset as 0 whatever is passed
        # (ops/topk_head_softmax.py:246,492)
        q_off = 0 if self.is_training else int(q_offset)
        indices, scores = SoftmaxTopKMaxPoolingFusedFn.apply(
            q, lmks, lse_swa, self.topk, self.block_size, self.window_size, self.is_causal, q_off,
            drop_mask, sm_scale, bias_arg, gumbel_arg, self.per_qhead_lmks, _debug)
        return indices, scores.view(B, L, h_kv * G, -1)


_SOFTMAX_MODULE_CACHE = {}


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
    if q.dim() == 4:
        B, L, h_q, D = q.shape
        lmks_h = lmks.shape[2]
        D_lmk = lmks.shape[3]
        if D != D_lmk:
            assert D_lmk % D == 0, f"lmks D dim ({D_lmk}) must be divisible by q D dim ({D})"
            d_ratio = D_lmk // D
            lmks = lmks.reshape(lmks.shape[0], lmks.shape[1], lmks_h * d_ratio, D)
            lmks_h = lmks_h * d_ratio
        if G == 1:
            assert h_q % lmks_h == 0, f"h_q ({h_q}) must be divisible by lmks_h ({lmks_h})"
            h_kv = lmks_h
            G_eff = h_q // h_kv
            per_qhead_lmks = False
        else:
            assert lmks_h == h_q, f"when G>1, lmks must have h_q ({h_q}) heads, got {lmks_h}"
            assert h_q % G == 0, f"h_q ({h_q}) must be divisible by G ({G})"
            h_kv = h_q // G
            G_eff = G
            per_qhead_lmks = True
        q = q.view(B, L, h_kv, G_eff, D)
    else:
        B, L, h_kv, G_in, D = q.shape
        h_q = h_kv * G_in
        D_lmk = lmks.shape[3]
        if D != D_lmk:
            assert D_lmk % D == 0, f"lmks D dim ({D_lmk}) must be divisible by q D dim ({D})"
            d_ratio = D_lmk // D
            lmks = lmks.reshape(lmks.shape[0], lmks.shape[1], lmks.shape[2] * d_ratio, D)
        lmks_h = lmks.shape[2]
        if G == 1:
            if lmks_h == h_kv:
                per_qhead_lmks = False
            elif lmks_h == h_q:
                per_qhead_lmks = True
            else:
                raise AssertionError(f"lmks_h ({lmks_h}) must be h_kv ({h_kv}) or h_q ({h_q})")
            G_eff = G_in
        else:
            assert lmks_h == h_q, f"when G>1, lmks must have h_q ({h_q}) heads, got {lmks_h}"
            assert h_q % G == 0, f"h_q ({h_q}) must be divisible by G ({G})"
            new_h_kv = h_q // G
            if (new_h_kv != h_kv) or (G != G_in):
                q = q.reshape(B, L, new_h_kv, G, D)
                h_kv = new_h_kv
            G_eff = G
            per_qhead_lmks = True
    lse_swa = lse_swa.reshape(B, L, h_kv, G_eff)
    use_drop_mask = drop_mask is not None
    cache_key = (topk, block_size, window_size, is_causal, is_training, use_drop_mask, per_qhead_lmks)
    mod = _SOFTMAX_MODULE_CACHE.get(cache_key)
    if mod is None:
        mod = _SOFTMAX_MODULE_CACHE[cache_key] = SoftmaxTopKMaxPooling_Fused(
            topk, block_size, window_size, is_causal, is_training, use_drop_mask,
            per_qhead_lmks=per_qhead_lmks)
    return mod(q, lmks, lse_swa, q_offset=q_offset, drop_mask=drop_mask, sm_scale=sm_scale,
               bias=bias, use_gumbel=use_gumbel, gumbel_noise=gumbel_noise, _debug=_debug)
