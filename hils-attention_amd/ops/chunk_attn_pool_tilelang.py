"""Chunk-key pooling (drop-in for the reference's ops/chunk_attn_pool_tilelang.py).

``chunk_attn_pool_tilelang`` / ``chunk_attn_pool_tilelang_shared_k`` keep the call
signatures of ops/chunk_attn_pool_tilelang.py:605-626 and :629-648; ``chunk_mean_pool``
is the mean-pool variant the attention layer computes with ``k_chunked.mean(dim=2)``
(models/FlashHiLS/hils_attention.py:398,436,446,460).
"""
import math

import torch

from . import _cabi


class ChunkAttnPoolFunction(torch.autograd.Function):
    """Mirrors ChunkAttnPoolFunction (ops/chunk_attn_pool_tilelang.py:540-602); k_chunked may carry
    fewer heads than mu_q (grouped query heads: head h reads K head h // (H // h_kv)), which the
    reference reaches by repeating K's heads in memory first
    (models/FlashHiLS/hils_attention.py:20-50, :391)."""

    @staticmethod
    def forward(ctx, mu_q, k_chunked, sm_scale, compact_lmk_k=False, shared_k=False):
        _cabi.require_gpu_bf16("chunk_attn_pool", mu_q, k_chunked)
        B, N, H, D = mu_q.shape
        S, HK = k_chunked.shape[2], k_chunked.shape[3]
        assert k_chunked.shape == (B, N, S, HK, D) and H % HK == 0, (
            f"k_chunked shape {tuple(k_chunked.shape)} does not go with mu_q {tuple(mu_q.shape)}")
        assert not shared_k or HK == H
        BN = B * N
        mu_flat = mu_q.reshape(BN, H, D).contiguous()
        k_flat = k_chunked.reshape(BN, S, HK, D).contiguous()
        compact = bool(compact_lmk_k)
        lmk_k = torch.empty((BN, H, D), dtype=mu_q.dtype, device=mu_q.device)
        lmk_b = torch.empty((BN, H), dtype=torch.float32, device=mu_q.device)
        p_saved = torch.empty((BN, S, H), dtype=torch.float32, device=mu_q.device)
        _cabi.call("hils_attn_pool_fwd", _cabi.ptr(mu_flat), _cabi.ptr(k_flat), _cabi.ptr(lmk_k),
                   _cabi.ptr(lmk_b), _cabi.ptr(p_saved), BN, S, H, HK, D, float(sm_scale),
                   int(compact), int(bool(shared_k)))
        ctx.save_for_backward(mu_flat, k_flat, p_saved, lmk_b)
        ctx.sm_scale = float(sm_scale)
        ctx.orig_shape = (B, N, H, HK, D, S)
        ctx.compact = compact
        ctx.shared_k = bool(shared_k)
        return lmk_k.reshape(B, N, H, D), lmk_b.reshape(B, N, H)

    @staticmethod
    def backward(ctx, grad_lmk_k, grad_lmk_b):
        mu_flat, k_flat, p_saved, lmk_b = ctx.saved_tensors
        B, N, H, HK, D, S = ctx.orig_shape
        BN = B * N
        if grad_lmk_k is None or ctx.compact:
            grad_lmk_k = torch.zeros((BN, H, D), dtype=mu_flat.dtype, device=mu_flat.device)
        else:
            grad_lmk_k = grad_lmk_k.reshape(BN, H, D).to(mu_flat.dtype).contiguous()
        if grad_lmk_b is None:
            grad_lmk_b = torch.zeros((BN, H), dtype=torch.float32, device=mu_flat.device)
        else:
            grad_lmk_b = grad_lmk_b.reshape(BN, H).float().contiguous()
        d_mu = torch.empty_like(mu_flat)
        d_k = torch.empty_like(k_flat)
        _cabi.call("hils_attn_pool_bwd", _cabi.ptr(mu_flat), _cabi.ptr(k_flat), _cabi.ptr(p_saved),
                   _cabi.ptr(lmk_b), _cabi.ptr(grad_lmk_k), _cabi.ptr(grad_lmk_b), _cabi.ptr(d_mu),
                   _cabi.ptr(d_k), BN, S, H, HK, D, ctx.sm_scale, int(ctx.compact), int(ctx.shared_k))
        return d_mu.reshape(B, N, H, D), d_k.reshape(B, N, S, HK, D), None, None, None


def chunk_attn_pool(mu_q, k_chunked, sm_scale=None):
    """The layer's pooling call (models/FlashHiLS/hils_attention.py:66-135), same signature and
    argument errors: mu_q (B,N,h_q,D), k_chunked (B,N,S,h_kv,D) at the model's own KV head count
    (h_q % h_kv == 0; nothing is repeated in memory) -> lmk_k (B,N,h_q,D) in K's dtype, lmk_b
    (B,N,h_q) fp32."""
    if mu_q.dim() != 4 or k_chunked.dim() != 5:
        raise ValueError(f"chunk_attn_pool: expected mu_q (B, N, h_q, d) and k_chunked (B, N, S, h_kv, d); got "
                         f"{tuple(mu_q.shape)} and {tuple(k_chunked.shape)}")
    B, N, h_q, D = mu_q.shape
    Bk, Nk, _, h_kv, Dk = k_chunked.shape
    if (B, N, D) != (Bk, Nk, Dk):
        raise ValueError(f"chunk_attn_pool: mu_q vs k_chunked shape mismatch on (B, N, d) -- got "
                         f"mu_q={tuple(mu_q.shape)}, k_chunked={tuple(k_chunked.shape)}")
    if h_q % h_kv != 0:
        raise ValueError(f"chunk_attn_pool: mu_q h_q ({h_q}) must be a multiple of k_chunked h_kv ({h_kv}) "
                         f"for GQA grouping")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    return ChunkAttnPoolFunction.apply(mu_q, k_chunked, sm_scale, False, False)


def chunk_attn_pool_tilelang(mu_q, k_chunked, sm_scale=None, compact_lmk_k=False):
    """mu_q (B,N,H,D) bf16, k_chunked (B,N,S,H,D) bf16 (or (B,N,S,h_kv,D) with H % h_kv == 0, which
    the reference's kernel does not take) -> lmk_k (B,N,H,D) bf16, lmk_b (B,N,H) fp32.

    One prior query per (chunk, head) attends to the chunk's first S-1 keys (the last
    token, the landmark slot, is masked); lmk_k = P @ K, lmk_b = entropy(P).
    ``compact_lmk_k`` skips P @ K and returns zeros for lmk_k.
    """
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(mu_q.shape[-1])
    return ChunkAttnPoolFunction.apply(mu_q, k_chunked, sm_scale, compact_lmk_k, False)


def chunk_attn_pool_tilelang_shared_k(mu_q, k_chunked, sm_scale=None):
    """Shared-K variant: K is identical across the H heads and is read from head 0 only;
    the backward sums dK over heads into head 0 and zeroes heads 1..H-1.
    Requires H >= 16 and H % 16 == 0, as the reference does."""
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(mu_q.shape[-1])
    H = mu_q.shape[2]
    assert H >= 16 and H % 16 == 0, f"shared_k variant requires H>=16 and H%16==0, got H={H}"
    return ChunkAttnPoolFunction.apply(mu_q, k_chunked, sm_scale, False, True)


class ChunkMeanPoolFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, k, chunk_size):
        _cabi.require_gpu_bf16("chunk_mean_pool", k)
        B, L, H, D = k.shape
        assert L % chunk_size == 0, f"L ({L}) must be a multiple of chunk_size ({chunk_size})"
        k = k.contiguous()
        out = torch.empty((B, L // chunk_size, H, D), dtype=k.dtype, device=k.device)
        _cabi.call("hils_mean_pool_fwd", _cabi.ptr(k), _cabi.ptr(out), B, L, H, D, int(chunk_size))
        ctx.dims = (B, L, H, D, int(chunk_size))
        return out

    @staticmethod
    def backward(ctx, g):
        B, L, H, D, S = ctx.dims
        g = g.to(torch.bfloat16).contiguous()
        dk = torch.empty((B, L, H, D), dtype=g.dtype, device=g.device)
        _cabi.call("hils_mean_pool_bwd", _cabi.ptr(g), _cabi.ptr(dk), B, L, H, D, S)
        return dk, None


def chunk_mean_pool(k, chunk_size):
    """k (B,L,H,D) bf16 -> (B, L//chunk_size, H, D) bf16: mean over each chunk's tokens."""
    return ChunkMeanPoolFunction.apply(k, chunk_size)
