"""Exact per-chunk log Z (drop-in for the reference's ops/exact_chunk_log_z_tilelang.py)."""
from typing import Optional

import torch

from . import _cabi


class _ExactChunkLogZ(torch.autograd.Function):
    """Mirrors _ExactChunkLogZ (ops/exact_chunk_log_z_tilelang.py:394-478)."""

    @staticmethod
    def forward(ctx, q, k, chunk_size, window_size, sm_scale, mask_lmk=False):
        assert q.dim() == 4 and k.dim() == 4
        _cabi.require_gpu_bf16("exact_chunk_log_z_tl", q, k)
        B, L, H_q, D = q.shape
        Bk, Lk, H_kv, Dk = k.shape
        assert (Bk, Lk, Dk) == (B, L, D), (
            f"q/k batch/seq/dim mismatch: q={tuple(q.shape)}, k={tuple(k.shape)}")
        assert H_q % H_kv == 0, f"H_q ({H_q}) must be a multiple of H_kv ({H_kv}) for GQA"
        q_c = q.contiguous()
        k_c = k.contiguous()
        n_chunk = (L + chunk_size - 1) // chunk_size
        log_z = torch.empty((B, L, H_q, n_chunk), dtype=torch.float32, device=q.device)
        _cabi.call("hils_chunk_logz_fwd", _cabi.ptr(q_c), _cabi.ptr(k_c), _cabi.ptr(log_z),
                   B, L, H_q, H_kv, D, int(chunk_size), int(window_size), float(sm_scale),
                   int(bool(mask_lmk)))
        ctx.save_for_backward(q_c, k_c, log_z)
        ctx.cfg = (int(chunk_size), int(window_size), float(sm_scale), H_kv, bool(mask_lmk))
        return log_z

    @staticmethod
    def backward(ctx, d_log_z):
        q, k, log_z = ctx.saved_tensors
        chunk_size, window_size, sm_scale, H_kv, mask_lmk = ctx.cfg
        if mask_lmk:
            raise NotImplementedError(
                "exact_chunk_log_z_tl(mask_lmk=True) is forward/eval-only; "
                "backward is not implemented for the landmark-masked path.")
        B, L, H_q, D = q.shape
        d_log_z = d_log_z.float().contiguous()
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        args = (B, L, H_q, H_kv, D, chunk_size, window_size, sm_scale)
        _cabi.call("hils_chunk_logz_bwd_dq", _cabi.ptr(q), _cabi.ptr(k), _cabi.ptr(log_z),
                   _cabi.ptr(d_log_z), _cabi.ptr(dq), *args)
        _cabi.call("hils_chunk_logz_bwd_dk", _cabi.ptr(q), _cabi.ptr(k), _cabi.ptr(log_z),
                   _cabi.ptr(d_log_z), _cabi.ptr(dk), *args)
        return dq, dk, None, None, None, None


def exact_chunk_log_z_tl(q: torch.Tensor, k: torch.Tensor, *, chunk_size: int, window_size: int,
                         sm_scale: Optional[float] = None, mask_lmk: bool = False) -> torch.Tensor:
    """log_Z[b,t,h,c] = log sum_{j in chunk c} exp(sm_scale*<q_t,k_j>) for chunks fully
    before the local window; (B, L, H_q, ceil(L/chunk_size)) fp32, -inf elsewhere.
    ``mask_lmk=True`` also masks landmark keys and is forward-only (backward raises)."""
    if sm_scale is None:
        sm_scale = (1.0 / q.shape[-1]) ** 0.5
    return _ExactChunkLogZ.apply(q, k, int(chunk_size), int(window_size), float(sm_scale),
                                 bool(mask_lmk))
