"""Rotary position embedding (drop-in for the reference's ops/rope_tilelang_fp32.py)."""
import torch

from . import _cabi


def _rope(x, cos, sin, per_batch, lo_only, sin_sign=1.0):
    B, L, H, D = x.shape
    out = torch.empty_like(x)
    _cabi.call("hils_rope", _cabi.ptr(x), _cabi.ptr(cos), _cabi.ptr(sin), _cabi.ptr(out), B, L, H, D,
               int(per_batch), int(cos.dtype == torch.float32), int(lo_only), float(sin_sign))
    return out


def rope_rotary_pos_emb(q, k, cos, sin):
    """q (B,L,H_q,D), k (B,L,H_k,D) bf16; cos, sin (B,L,D) bf16 -> (q_out, k_out) bf16.  Both halves
    of a head vector are rotated by the first D/2 table entries, as rope_fwd_kernel does
    (ops/rope_tilelang_fp32.py:19-89)."""
    _cabi.require_gpu_bf16("rope_rotary_pos_emb", q, k, cos, sin)
    B, L, _, D = q.shape
    assert k.shape[0] == B and k.shape[1] == L and k.shape[3] == D
    assert cos.shape == (B, L, D) and sin.shape == (B, L, D)
    cos, sin = cos.contiguous(), sin.contiguous()
    return (_rope(q.contiguous(), cos, sin, True, True), _rope(k.contiguous(), cos, sin, True, True))


def _single_tensor_rope(x, x_cos, x_sin, sin_sign=1.0):
    """Mirrors _single_tensor_rope (ops/rope_tilelang_fp32.py:140-154): tables (L,D) or (1,L,D),
    bf16 or fp32, the low half rotated by the low half of the tables and the high half by their
    high half."""
    B, L, H, D = x.shape
    if x_cos.ndim == 3:
        assert x_cos.shape[0] == 1 and x_sin.shape[0] == 1, (
            "Expected batch dim of x_cos/x_sin to be 1 when ndim==3 (shared across batch), but got "
            f"x_cos.shape={tuple(x_cos.shape)}, x_sin.shape={tuple(x_sin.shape)}")
        x_cos, x_sin = x_cos[0], x_sin[0]
    assert x_cos.shape == (L, D) and x_sin.shape == (L, D)
    if x_cos.dtype != torch.float32:
        x_cos, x_sin = x_cos.to(torch.bfloat16), x_sin.to(torch.bfloat16)
    else:
        x_sin = x_sin.float()
    _cabi.require_gpu_bf16("single_tensor_rope", x)
    return _rope(x.contiguous(), x_cos.contiguous(), x_sin.contiguous(), False, False, sin_sign)


class SingleTensorRoPEFunction(torch.autograd.Function):
    """Mirrors SingleTensorRoPEFunction (ops/rope_tilelang_fp32.py:157-170): the backward is the
    same rotation with -sin."""

    @staticmethod
    def forward(ctx, x, x_cos, x_sin):
        ctx.save_for_backward(x_cos, x_sin)
        return _single_tensor_rope(x, x_cos, x_sin)

    @staticmethod
    def backward(ctx, dx):
        x_cos, x_sin = ctx.saved_tensors
        return _single_tensor_rope(dx.to(torch.bfloat16).contiguous(), x_cos, x_sin, sin_sign=-1.0), None, None


def single_tensor_rope_autograd(x, x_cos, x_sin):
    """x (B,L,H,D) bf16; x_cos, x_sin (L,D) or (1,L,D), bf16 or fp32 -> (B,L,H,D) bf16."""
    return SingleTensorRoPEFunction.apply(x, x_cos, x_sin)
