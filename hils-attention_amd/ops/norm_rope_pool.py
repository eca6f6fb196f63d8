"""Key / query preparation in one pass: per-head RMS norm, rotary embedding, chunk mean.

The reference has no single function for this; its attention layer runs the three steps one
after the other (models/FlashHiLS/hils_attention.py:314-321 k_norm, :479-483 apply_rotary_pos_emb,
:398 / :460 ``k_chunked.mean(dim=2)``), each a full pass over the (B, L, H, D) tensor.
"""
import torch

from . import _cabi


def _tables(cos, sin, B, L, D):
    """cos/sin as contiguous bf16 (L,D) or (B,L,D) tensors and the per-batch flag."""
    if cos is None:
        assert sin is None, "cos and sin come together"
        return None, None, 0
    assert cos.shape == sin.shape, f"cos {tuple(cos.shape)} and sin {tuple(sin.shape)} differ"
    if cos.ndim == 3 and cos.shape[0] == 1:
        cos, sin = cos[0], sin[0]
    per_batch = int(cos.ndim == 3)
    want = (B, L, D) if per_batch else (L, D)
    assert tuple(cos.shape) == want, f"cos/sin must be ({L},{D}), (1,{L},{D}) or ({B},{L},{D}); got {tuple(cos.shape)}"
    return cos.to(torch.bfloat16).contiguous(), sin.to(torch.bfloat16).contiguous(), per_batch


class _NormRopePoolFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, norm_weight, cos, sin, chunk_size, eps, want_lmk):
        _cabi.require_gpu_bf16("norm_rope_pool", x)
        B, L, H, D = x.shape
        x_in = x.contiguous()
        w_in = None
        if norm_weight is not None:
            assert norm_weight.shape == (D,), f"norm_weight must have shape ({D},), got {tuple(norm_weight.shape)}"
            w_in = norm_weight.to(device=x.device, dtype=torch.bfloat16).contiguous()
        cos_in, sin_in, per_batch = _tables(cos, sin, B, L, D)
        S = int(chunk_size)
        out = torch.empty_like(x_in)
        lmk = torch.empty((B, L // S, H, D), dtype=x.dtype, device=x.device) if want_lmk else None
        _cabi.call("hils_norm_rope_pool_fwd", _cabi.ptr(x_in), _cabi.ptr(w_in), _cabi.ptr(cos_in), _cabi.ptr(sin_in),
                   _cabi.ptr(out), _cabi.ptr(lmk), B, L, H, D, S, per_batch, float(eps))
        ctx.save_for_backward(x_in, w_in, cos_in, sin_in)
        ctx.cfg = (B, L, H, D, S, per_batch, float(eps))
        ctx.w_dtype = None if norm_weight is None else norm_weight.dtype
        return out, lmk

    @staticmethod
    def backward(ctx, d_out, d_lmk):
        x_in, w_in, cos_in, sin_in = ctx.saved_tensors
        B, L, H, D, S, per_batch, eps = ctx.cfg
        g_out = None if d_out is None else d_out.to(torch.bfloat16).contiguous()
        g_lmk = None if d_lmk is None else d_lmk.to(torch.bfloat16).contiguous()
        if g_out is None and g_lmk is None:
            return None, None, None, None, None, None, None
        dx = torch.empty_like(x_in)
        dw = torch.zeros(D, dtype=torch.float32, device=x_in.device) if w_in is not None else None
        _cabi.call("hils_norm_rope_pool_bwd", _cabi.ptr(x_in), _cabi.ptr(w_in), _cabi.ptr(cos_in), _cabi.ptr(sin_in),
                   _cabi.ptr(g_out), _cabi.ptr(g_lmk), _cabi.ptr(dx), _cabi.ptr(dw), B, L, H, D, S, per_batch, eps)
        return dx, (None if dw is None else dw.to(ctx.w_dtype)), None, None, None, None, None


def norm_rope_pool(x, norm_weight=None, cos=None, sin=None, chunk_size=64, eps=1e-6, pool=True):
    """x (B,L,H,D) bf16 -> (out (B,L,H,D), lmk (B,L//chunk_size,H,D) or None).

    ``out = rope(rms_norm(x) * norm_weight)`` with the roundings of the layer's bf16 sequence;
    ``lmk`` is the mean of ``out`` over every whole chunk (``pool=False`` skips it: the query
    side).  ``norm_weight`` (D,) or None (no norm); ``cos`` / ``sin`` (L,D), (1,L,D) or (B,L,D),
    HF rotate-half convention, or None (no rotation).  Differentiable in ``x`` and ``norm_weight``.
    """
    return _NormRopePoolFn.apply(x, norm_weight, cos, sin, chunk_size, eps, bool(pool))
