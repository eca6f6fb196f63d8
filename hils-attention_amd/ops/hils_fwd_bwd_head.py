"""HiLS sparse attention over the selected chunks (drop-in for ops/hils_fwd_bwd_head.py)."""
import math

import torch

from . import _cabi


def _check_kv_workspace(ws, need_bytes, device, what):
    """The kernels index a caller-held workspace by the shape of the call it is passed to: one
    packed for another (shorter) shape would be read and written past its end, so reject it."""
    if (ws.device != device or ws.dtype != torch.uint8 or not ws.is_contiguous()
            or ws.numel() < need_bytes):
        raise ValueError(
            f"kv_workspace must be a contiguous uint8 tensor on {device} of at least {need_bytes} "
            f"bytes for this call ({what}); got {ws.dtype} x {ws.numel()} on {ws.device}.  Build it "
            "with prepare_kv_workspace for this shape.")


class _hils_block_M_attention_inverse(torch.autograd.Function):
    """Mirrors _hils_block_M_attention_inverse (ops/hils_fwd_bwd_head.py:771-913)."""

    @staticmethod
    def forward(ctx, q, k, v, weights, indices, block_size, sm_scale, mask_last_token,
                is_training, slope=None, kv_workspace=None, swa_o=None, swa_weight_index=None):
        assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
        assert weights.is_contiguous() and indices.is_contiguous()
        _cabi.require_gpu_bf16("HiLS_block_M_head", q)
        # inference may read K and V of an offloaded cache in place (pinned host memory)
        _cabi.require_gpu_bf16("HiLS_block_M_head", k, v, pinned_ok=not is_training)
        B, L, HQ, D = q.shape
        L_kv, H, Dk = k.shape[1], k.shape[2], k.shape[-1]
        Dv = v.shape[-1]
        K = indices.shape[-1]
        num_weights = weights.shape[-1]
        assert HQ % H == 0, f"HQ={HQ} must be divisible by H={H}"
        assert Dk == D, f"Q head_dim ({D}) must equal K head_dim ({Dk})"
        assert indices.shape == (B, L, H, K), f"indices shape {tuple(indices.shape)} != {(B, L, H, K)}"
        assert weights.shape[:3] == (B, L, HQ) and num_weights >= K, (
            f"weights shape {tuple(weights.shape)} must be ({B}, {L}, {HQ}, >= {K})")
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(D)
        slope_dev = None
        if slope is not None:
            assert slope.shape == (HQ,), f"slope must be 1-D with shape ({HQ},), got {tuple(slope.shape)}"
            slope_dev = slope.to(dtype=torch.float32, device=q.device).contiguous()
        w_in = weights.to(q.dtype).contiguous()
        idx_in = indices.to(torch.int32).contiguous()
        swa_in, merge_col = None, 0
        if swa_o is not None:
            assert swa_o.shape == (B, L, HQ, Dv), f"swa_o shape {tuple(swa_o.shape)} != {(B, L, HQ, Dv)}"
            merge_col = int(K if swa_weight_index is None else swa_weight_index) % num_weights
            assert merge_col >= K, f"the local branch's weight column ({merge_col}) lies among the {K} chunk slots"
            _cabi.require_gpu_bf16("HiLS_block_M_head", swa_o)
            swa_in = swa_o.contiguous()
        o = torch.empty((B, L, HQ, Dv), dtype=q.dtype, device=q.device)
        lse = None
        if is_training:
            lse = torch.empty((B, L, HQ, K), dtype=torch.float32, device=q.device)
        ws_ready = 0
        if kv_workspace is not None:
            need = _cabi.sparse_attn_fwd_workspace_bytes(B, L, L_kv, HQ, H, D, Dv, K, HQ, 1,
                                                         int(block_size), 0.0)
            _check_kv_workspace(kv_workspace, need, q.device,
                                f"q_len {L}, kv_len {L_kv}, {HQ}/{H} heads, D {D}, Dv {Dv}, top-{K}")
            ws, ws_ready = kv_workspace, 1
        else:
            ws = _cabi.sparse_attn_fwd_workspace(q.device, B, L, L_kv, HQ, H, D, Dv, K, HQ, 1,
                                                 int(block_size), 0.0)
        _cabi.call("hils_sparse_attn_fwd", _cabi.ptr(q), _cabi.ptr(k), _cabi.ptr(v), _cabi.ptr(w_in),
                   _cabi.ptr(idx_in), _cabi.ptr(slope_dev), _cabi.ptr(swa_in), _cabi.ptr(o), _cabi.ptr(lse),
                   _cabi.ptr(ws), _cabi.nbytes(ws), ws_ready, B, L, L_kv, HQ, H, D, Dv, K, num_weights, HQ, 1, int(block_size),
                   float(sm_scale), int(bool(mask_last_token)), 0.0, merge_col)
        ctx.is_training = bool(is_training)
        if is_training:
            ctx.save_for_backward(q, k, v, w_in, idx_in, lse, slope_dev, swa_in)
            ctx.cfg = (B, L, L_kv, HQ, H, D, Dv, K, num_weights, int(block_size), float(sm_scale),
                       int(bool(mask_last_token)), merge_col)
            ctx.w_dtype = weights.dtype
        return o

    @staticmethod
    def backward(ctx, do):
        if not getattr(ctx, "is_training", True):
            raise RuntimeError(
                "[_hils_block_M_attention_inverse] forward ran with is_training=False: the "
                "per-chunk LSE needed by the backward was not saved.")
        q, k, v, w_in, idx_in, lse, slope_dev, swa_in = ctx.saved_tensors
        B, L, L_kv, HQ, H, D, Dv, K, NW, S, sm_scale, mask_last, merge_col = ctx.cfg
        d_swa = torch.empty_like(swa_in) if swa_in is not None else None
        do = do.to(q.dtype).contiguous()
        dq = torch.empty_like(q)
        dw = torch.zeros((B, L, HQ, NW), dtype=torch.float32, device=q.device)
        ws = _cabi.sparse_attn_bwd_workspace(q.device, B, L, L_kv, HQ, H, D, Dv, K, HQ, 1, S, 0.0)
        # the workspace kernels write dk / dv once, as bf16; the shape-generic one adds into fp32
        kv16 = ws is not None and k.dtype == torch.bfloat16 and v.dtype == torch.bfloat16
        if kv16:
            dk, dv = torch.empty_like(k), torch.empty_like(v)
        else:
            dk = torch.zeros(k.shape, dtype=torch.float32, device=k.device)
            dv = torch.zeros(v.shape, dtype=torch.float32, device=v.device)
        _cabi.call("hils_sparse_attn_bwd", _cabi.ptr(q), _cabi.ptr(k), _cabi.ptr(v), _cabi.ptr(w_in),
                   _cabi.ptr(idx_in), _cabi.ptr(slope_dev), _cabi.ptr(lse), _cabi.ptr(do),
                   _cabi.ptr(dq), _cabi.ptr(dk), _cabi.ptr(dv), _cabi.ptr(dw), _cabi.ptr(ws), _cabi.nbytes(ws),
                   B, L, L_kv, HQ, H, D, Dv, K, NW, HQ, 1, S, sm_scale, mask_last, 0.0,
                   _cabi.ptr(swa_in), _cabi.ptr(d_swa), merge_col, int(kv16))
        return (dq, dk.to(k.dtype), dv.to(v.dtype), dw.to(ctx.w_dtype), None,
                None, None, None, None, None, None, d_swa, None)


class _hils_block_M_attention_f32(torch.autograd.Function):
    """The dtype="float32" mode (ops/hils_fwd_bwd_head.py:928-964 with dtype="float32"): fp32 q, k, v,
    weights; every product and the softmax in fp32 on the shape-generic kernels."""

    @staticmethod
    def forward(ctx, q, k, v, weights, indices, block_size, sm_scale, mask_last_token, is_training, slope):
        for name, t in (("q", q), ("k", k), ("v", v)):
            if not t.is_cuda:
                raise RuntimeError(f"HiLS_block_M_head: {name} must live on the GPU (got {t.device}); "
                                   "this package has no CPU path")
            if t.dtype != torch.float32:
                raise TypeError(f"HiLS_block_M_head(dtype='float32'): {name} must be float32, got {t.dtype}")
        assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
        B, L, HQ, D = q.shape
        L_kv, H, Dv = k.shape[1], k.shape[2], v.shape[-1]
        K, NW = indices.shape[-1], weights.shape[-1]
        assert indices.shape == (B, L, H, K), f"indices shape {tuple(indices.shape)} != {(B, L, H, K)}"
        assert weights.shape[:3] == (B, L, HQ) and NW >= K, (
            f"weights shape {tuple(weights.shape)} must be ({B}, {L}, {HQ}, >= {K})")
        if sm_scale is None:
            sm_scale = 1.0 / math.sqrt(D)
        slope_dev = None
        if slope is not None:
            assert slope.shape == (HQ,), f"slope must be 1-D with shape ({HQ},), got {tuple(slope.shape)}"
            slope_dev = slope.to(dtype=torch.float32, device=q.device).contiguous()
        w_in = weights.to(torch.float32).contiguous()
        idx_in = indices.to(torch.int32).contiguous()
        o = torch.empty((B, L, HQ, Dv), dtype=torch.float32, device=q.device)
        lse = torch.empty((B, L, HQ, K), dtype=torch.float32, device=q.device) if is_training else None
        _cabi.call("hils_sparse_attn_fwd_f32", _cabi.ptr(q), _cabi.ptr(k), _cabi.ptr(v), _cabi.ptr(w_in),
                   _cabi.ptr(idx_in), _cabi.ptr(slope_dev), _cabi.ptr(o), _cabi.ptr(lse), B, L, L_kv, HQ, H, D, Dv,
                   K, NW, HQ, 1, int(block_size), float(sm_scale), int(bool(mask_last_token)), 0.0)
        ctx.is_training = bool(is_training)
        if is_training:
            ctx.save_for_backward(q, k, v, w_in, idx_in, lse, slope_dev)
            ctx.cfg = (B, L, L_kv, HQ, H, D, Dv, K, NW, int(block_size), float(sm_scale), int(bool(mask_last_token)))
            ctx.w_dtype = weights.dtype
        return o

    @staticmethod
    def backward(ctx, do):
        if not getattr(ctx, "is_training", True):
            raise RuntimeError(
                "[_hils_block_M_attention_inverse] forward ran with is_training=False: the "
                "per-chunk LSE needed by the backward was not saved.")
        q, k, v, w_in, idx_in, lse, slope_dev = ctx.saved_tensors
        B, L, L_kv, HQ, H, D, Dv, K, NW, S, sm_scale, mask_last = ctx.cfg
        do = do.to(torch.float32).contiguous()
        dq = torch.empty_like(q)
        dk, dv = torch.zeros_like(k), torch.zeros_like(v)
        dw = torch.zeros((B, L, HQ, NW), dtype=torch.float32, device=q.device)
        _cabi.call("hils_sparse_attn_bwd_f32", _cabi.ptr(q), _cabi.ptr(k), _cabi.ptr(v), _cabi.ptr(w_in),
                   _cabi.ptr(idx_in), _cabi.ptr(slope_dev), _cabi.ptr(lse), _cabi.ptr(do), _cabi.ptr(dq),
                   _cabi.ptr(dk), _cabi.ptr(dv), _cabi.ptr(dw), B, L, L_kv, HQ, H, D, Dv, K, NW, HQ, 1, S,
                   sm_scale, mask_last, 0.0)
        return dq, dk, dv, dw.to(ctx.w_dtype), None, None, None, None, None, None


def HiLS_block_M_head(q, k, v, weights, indices, block_size=64, sm_scale=None, block_M=None,
                      mask_last_token=True, dtype="bfloat16", accum_dtype="float",
                      num_threads=None, num_threads_fwd=None, num_threads_bwd=None,
                      is_training=True, slope=None, kv_workspace=None, swa_o=None, swa_weight_index=None):
    """o[t,h] = sum_k weights[t,h,k] * softmax_{j in chunk indices[t,k]}(sm_scale*q.K_j) V_j.

    q (B,L,HQ,D), k (B,Lkv,H,D), v (B,Lkv,H,Dv) bf16 contiguous; weights (B,L,HQ,>=K) (the
    first K columns are read); indices (B,L,H,K) int32, negative = empty slot.  Call
    signature of ops/hils_fwd_bwd_head.py:928-934; ``block_M`` and the ``num_threads*``
    tuning knobs are accepted and ignored (tile shapes are chosen by the HIP launcher),
    ``dtype`` "bfloat16" (the MFMA kernels) or "float32" (fp32 tensors, everything computed in fp32 on
    the shape-generic kernels: the mode the reference's fp32 correctness test runs in) and
    ``accum_dtype`` "float".  ``kv_workspace`` (not in the
    reference) is an optional tensor from ``prepare_kv_workspace`` for the same ``v``: the
    MFMA-operand-ordered copies of K and V the prefill kernel reads, reusable across calls.
    ``swa_o`` (B,L,HQ,Dv), not in the reference either: the local branch's output; with it the
    call returns the layer's merged output ``hils_o + swa_o * weights[..., swa_weight_index]``
    (``torch.addcmul`` at models/FlashHiLS/hils_attention.py:617-623; ``swa_weight_index``
    defaults to K, pass -2 with the softmax-1 sink column), with gradients to ``swa_o`` and to
    that weight column.
    """
    B, L, HQ, D = q.shape
    _, L_kv, H, Dk = k.shape
    assert D == Dk, f"Q head_dim ({D}) must equal K head_dim ({Dk})"
    assert HQ % H == 0, f"HQ={HQ} must be divisible by H={H}"
    if accum_dtype not in ("float", "float32", torch.float32):
        raise ValueError("HiLS_block_M_head: only accum_dtype='float' is built")
    if dtype in ("float32", "float", torch.float32):
        if kv_workspace is not None or swa_o is not None:
            raise ValueError("HiLS_block_M_head(dtype='float32'): kv_workspace and swa_o belong to the bf16 kernels")
        return _hils_block_M_attention_f32.apply(q, k, v, weights, indices, block_size, sm_scale,
                                                 mask_last_token, is_training, slope)
    if dtype not in ("bfloat16", torch.bfloat16):
        raise ValueError("HiLS_block_M_head: dtype must be 'bfloat16' or 'float32'")
    return _hils_block_M_attention_inverse.apply(
        q, k, v, weights, indices, block_size, sm_scale, mask_last_token, is_training, slope,
        kv_workspace, swa_o, swa_weight_index)


def prepare_kv_workspace(q_len, k, v, num_q_heads, topk, block_size=64):
    """Build the packed K/V workspace ``HiLS_block_M_head(..., kv_workspace=...)`` accepts
    (None when the shape runs on kernels that need none)."""
    _cabi.require_gpu_bf16("prepare_kv_workspace", k, v)
    B, L_kv, H, Dv = v.shape
    D = k.shape[-1]
    ws = _cabi.sparse_attn_fwd_workspace(v.device, B, q_len, L_kv, num_q_heads, H, D, Dv,
                                         topk, num_q_heads, 1, int(block_size), 0.0)
    if ws is not None and q_len >= 64:
        _cabi.call("hils_pack_kv_chunks", _cabi.ptr(k.contiguous()), _cabi.ptr(v.contiguous()),
                   _cabi.ptr(ws), _cabi.nbytes(ws), B, L_kv, H, D, Dv)
    return ws
