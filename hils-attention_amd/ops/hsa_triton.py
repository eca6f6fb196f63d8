"""Older hierarchical sparse attention operator (drop-in for ops/hsa_triton.py:HSA)."""
import math

import torch

from . import _cabi


class _attention(torch.autograd.Function):
    """Mirrors _attention (ops/hsa_triton.py:603-795): indices and weights are shared by a
    block of Q_X consecutive queries and by the G heads of a KV head; every per-chunk softmax
    has ``sm_n * exp(-max)`` added to its denominator; landmark tokens are not masked."""

    @staticmethod
    def forward(ctx, q, k, v, weights, indices, sm_n, chunk_size, sm_scale, l2_lamda, l2_C):
        assert not torch.any(torch.isnan(q))
        assert not torch.any(torch.isnan(k))
        assert not torch.any(torch.isnan(v))
        assert not torch.any(torch.isnan(weights))
        assert torch.all(indices >= 0)
        _cabi.require_gpu_bf16("HSA", q, k, v)
        N, L, HQ, D = q.shape
        L_kv = k.shape[1]
        assert L_kv % chunk_size == 0
        assert indices.is_contiguous()
        assert weights.is_contiguous()
        assert q.is_contiguous()
        assert k.is_contiguous()
        assert v.is_contiguous()
        if sm_scale is None:
            sm_scale = 1 / math.sqrt(D)
        H = k.shape[2]
        K = indices.shape[-1]
        block_num = indices.shape[1]
        assert q.shape[1] % block_num == 0
        q_x = q.shape[1] // block_num
        assert HQ % H == 0
        assert weights.shape == indices.shape
        w_in = weights.to(q.dtype).contiguous()
        idx_in = indices.to(torch.int32).contiguous()
        o = torch.empty_like(q)
        lse = torch.empty((N, L, HQ, K), dtype=torch.float32, device=q.device)
        ws = _cabi.sparse_attn_fwd_workspace(q.device, N, L, L_kv, HQ, H, D, v.shape[-1], K, H, q_x,
                                             int(chunk_size), float(sm_n))
        _cabi.call("hils_sparse_attn_fwd", _cabi.ptr(q), _cabi.ptr(k), _cabi.ptr(v), _cabi.ptr(w_in),
                   _cabi.ptr(idx_in), None, None, _cabi.ptr(o), _cabi.ptr(lse), _cabi.ptr(ws), _cabi.nbytes(ws), 0,
                   N, L, L_kv, HQ, H, D, v.shape[-1], K, K, H, q_x, int(chunk_size),
                   float(sm_scale), 0, float(sm_n), 0)
        ctx.save_for_backward(q, k, v, w_in, idx_in, lse)
        ctx.cfg = (N, L, L_kv, HQ, H, D, v.shape[-1], K, q_x, int(chunk_size), float(sm_scale), float(sm_n))
        ctx.w_dtype = weights.dtype
        assert not torch.any(torch.isnan(o))
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, w_in, idx_in, lse = ctx.saved_tensors
        N, L, L_kv, HQ, H, D, Dv, K, q_x, S, sm_scale, sm_n = ctx.cfg
        do = do.to(q.dtype).contiguous()
        dq = torch.empty_like(q)
        # The MFMA backward works on per-query indices and per-query-head weights: hand it the
        # block-shared rows expanded (small tensors) and fold the weight gradient back afterwards.
        ws = _cabi.sparse_attn_bwd_workspace(q.device, N, L, L_kv, HQ, H, D, Dv, K, HQ, 1, S, sm_n)
        if ws is not None:
            G = HQ // H
            idx_full = idx_in.repeat_interleave(q_x, dim=1).contiguous()
            w_full = w_in.repeat_interleave(q_x, dim=1).repeat_interleave(G, dim=2).contiguous()
            dw_full = torch.zeros((N, L, HQ, K), dtype=torch.float32, device=q.device)
            dk, dv = torch.empty_like(k), torch.empty_like(v)  # written once, as bf16
            _cabi.call("hils_sparse_attn_bwd", _cabi.ptr(q), _cabi.ptr(k), _cabi.ptr(v), _cabi.ptr(w_full),
                       _cabi.ptr(idx_full), None, _cabi.ptr(lse), _cabi.ptr(do),
                       _cabi.ptr(dq), _cabi.ptr(dk), _cabi.ptr(dv), _cabi.ptr(dw_full), _cabi.ptr(ws), _cabi.nbytes(ws),
                       N, L, L_kv, HQ, H, D, Dv, K, K, HQ, 1, S, sm_scale, 0, sm_n, None, None, 0, 1)
            dw = dw_full.view(N, L // q_x, q_x, H, G, K).sum(dim=(2, 4))
            return (dq, dk.to(k.dtype), dv.to(v.dtype), dw.to(ctx.w_dtype),
                    None, None, None, None, None, None)
        dw = torch.zeros(w_in.shape, dtype=torch.float32, device=q.device)
        dk = torch.zeros(k.shape, dtype=torch.float32, device=k.device)
        dv = torch.zeros(v.shape, dtype=torch.float32, device=v.device)
        _cabi.call("hils_sparse_attn_bwd", _cabi.ptr(q), _cabi.ptr(k), _cabi.ptr(v), _cabi.ptr(w_in),
                   _cabi.ptr(idx_in), None, _cabi.ptr(lse), _cabi.ptr(do),
                   _cabi.ptr(dq), _cabi.ptr(dk), _cabi.ptr(dv), _cabi.ptr(dw), None, 0,
                   N, L, L_kv, HQ, H, D, Dv, K, K, H, q_x, S, sm_scale, 0, sm_n, None, None, 0, 0)
        return (dq, dk.to(k.dtype), dv.to(v.dtype), dw.to(ctx.w_dtype),
                None, None, None, None, None, None)


def HSA(q, k, v, weights, indices, sm_n, chunk_size, sm_scale, reg_lamda=0.01, reg_C=50.0):
    """q (N,L,h_q,d), k/v (N,L_kv,h_kv,d) bf16; weights/indices (N, L//Q_X, h_kv, K), all
    indices >= 0.  ``reg_lamda`` / ``reg_C`` are accepted and unused, as in the reference
    (its regulariser code is commented out, ops/hsa_triton.py:358-369)."""
    return _attention.apply(q, k, v, weights, indices, sm_n, chunk_size, sm_scale, reg_lamda, reg_C)
