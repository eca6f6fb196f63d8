"""Sliding-window attention of the local branch (drop-in for flex_attn_tl of the reference's
ops/flex_attn_tilelang.py)."""
import math

import torch

from . import _cabi


class _FlexAttnTL(torch.autograd.Function):
    """Mirrors _FlexAttnTL (ops/flex_attn_tilelang.py:1156-1255; kernels :26-267 forward,
    :270-1153 backward).  lse is kept in natural-log units throughout."""

    @staticmethod
    def forward(ctx, q, k, v, window_size, chunk_size, mask_lmk, expand_to_chunk, use_cache, sm_scale,
                kv_start):
        assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4
        _cabi.require_gpu_bf16("flex_attn_tl", q)
        _cabi.require_gpu_bf16("flex_attn_tl", k, v, pinned_ok=bool(use_cache))  # an offloaded cache is read in place
        B, Lq, HQ, D = q.shape
        Lk, H = k.shape[1], k.shape[2]
        Dv = v.shape[-1]
        assert k.shape[0] == B and v.shape[0] == B and v.shape[1] == Lk and v.shape[2] == H
        assert k.shape[-1] == D, f"q/k head dims differ: {D} vs {k.shape[-1]}"
        assert HQ % H == 0, f"H_q ({HQ}) must be a multiple of H_kv ({H})"
        if not use_cache:
            assert Lq == Lk, f"training mode needs Lq == Lk (got {Lq}, {Lk})"
        assert Lq <= Lk, f"Lq ({Lq}) must not exceed Lk ({Lk})"
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(D)
        q_c, k_c, v_c = q.contiguous(), _cabi.gpu_readable(k, q.device), _cabi.gpu_readable(v, q.device)
        o = torch.empty((B, Lq, HQ, Dv), dtype=q.dtype, device=q.device)
        lse = torch.empty((B, Lq, HQ), dtype=torch.float32, device=q.device)
        _cabi.call("hils_swa_fwd", _cabi.ptr(q_c), _cabi.ptr(k_c), _cabi.ptr(v_c), _cabi.ptr(o),
                   _cabi.ptr(lse), B, Lq, Lk, HQ, H, D, Dv, int(window_size), int(chunk_size),
                   int(bool(mask_lmk)), int(bool(expand_to_chunk)), int(kv_start), float(sm_scale))
        ctx.save_for_backward(q_c, k_c, v_c, o, lse)
        ctx.cfg = (int(window_size), int(chunk_size), bool(mask_lmk), bool(expand_to_chunk),
                   bool(use_cache), float(sm_scale))
        return o, lse

    @staticmethod
    def backward(ctx, do, dlse):
        q, k, v, o, lse = ctx.saved_tensors
        window_size, chunk_size, mask_lmk, expand_to_chunk, use_cache, sm_scale = ctx.cfg
        if use_cache:
            raise RuntimeError("flex_attn_tl backward is not supported in inference (training=False) mode")
        B, L, HQ, D = q.shape
        H, Dv = k.shape[2], v.shape[-1]
        do = do.to(torch.bfloat16).contiguous()
        d_lse = None if dlse is None else dlse.float().contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        delta = torch.empty((B, L, HQ), dtype=torch.float32, device=q.device)
        _cabi.call("hils_swa_bwd", _cabi.ptr(q), _cabi.ptr(k), _cabi.ptr(v), _cabi.ptr(o), _cabi.ptr(lse),
                   _cabi.ptr(do), _cabi.ptr(d_lse), _cabi.ptr(dq), _cabi.ptr(dk), _cabi.ptr(dv),
                   _cabi.ptr(delta), B, L, HQ, H, D, Dv, window_size, chunk_size, int(mask_lmk),
                   int(expand_to_chunk), sm_scale)
        return dq, dk, dv, None, None, None, None, None, None, None


def flex_attn_tl(q, k, v, window_size: int, chunk_size: int, training: bool = True,
                 mask_lmk: bool = True, expand_to_chunk: bool = True, sm_scale: float = None,
                 kv_start: int = 0):
    """q (B,Lq,H_q,D), k (B,Lk,H_kv,D), v (B,Lk,H_kv,Dv) bf16 -> o (B,Lq,H_q,Dv) bf16 and
    lse (B,Lq,H_q) fp32 in natural-log units.  Causal window of ``window_size`` tokens whose left
    edge moves to the start of its chunk when ``expand_to_chunk``; ``mask_lmk`` hides the last
    token of every chunk.  ``training=False`` allows Lq <= Lk (queries are the last Lq positions)
    and a cache truncated at ``kv_start``."""
    if training and int(kv_start) != 0:
        raise ValueError("flex_attn_tl only supports non-zero kv_start in inference (training=False)")
    return _FlexAttnTL.apply(q, k, v, int(window_size), int(chunk_size), bool(mask_lmk),
                             bool(expand_to_chunk), not training, sm_scale, int(kv_start))


def flex_attn_tl_two_phase(q, k, v, window_size: int, chunk_size: int, training: bool = True,
                           mask_lmk: bool = True, expand_to_chunk: bool = True, sm_scale: float = None,
                           kv_start: int = 0):
    """Same as ``flex_attn_tl`` (ops/flex_attn_tilelang.py:1313-1349 of the reference): the
    reference's variant with an atomic-free backward of two kernels (dQ over query blocks, dK/dV
    over key blocks, bf16 outputs written directly), which is how the backward here always works."""
    if training and int(kv_start) != 0:
        raise ValueError(
            "flex_attn_tl_two_phase only supports non-zero kv_start in inference (training=False)")
    return flex_attn_tl(q, k, v, window_size, chunk_size, training=training, mask_lmk=mask_lmk,
                        expand_to_chunk=expand_to_chunk, sm_scale=sm_scale, kv_start=kv_start)
