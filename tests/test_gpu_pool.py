"""HIP chunk-key pooling vs the CPU oracle, through the C ABI.

Shapes follow unittests/test_chunk_attn_pool_tilelang.py:62-71 of the reference (seed 42).
"""
import math

import pytest
import torch

from util import assert_close_bf16, assert_close_f32, note

pytestmark = pytest.mark.gpu

POOL_SHAPES = [(1, 64, 2, 128, 64), (2, 32, 4, 128, 64), (1, 16, 16, 64, 64), (1, 16, 1, 128, 32),
               (2, 8, 32, 128, 64), (1, 4, 3, 64, 16)]


@pytest.mark.parametrize("B,N,H,D,S", POOL_SHAPES)
def test_attn_pool_fwd(pkg, orc, dev, B, N, H, D, S):
    note(f"attn_pool_fwd B{B} N{N} H{H} D{D} S{S}")
    torch.manual_seed(42)
    mu = torch.randn(B, N, H, D).bfloat16()
    k = torch.randn(B, N, S, H, D).bfloat16()
    lk, lb = pkg.chunk_attn_pool_tilelang(mu.to(dev), k.to(dev))
    rk, rb, _ = orc.chunk_attn_pool(mu, k)
    assert lk.dtype == torch.bfloat16 and lb.dtype == torch.float32
    assert_close_bf16(lk, rk, "lmk_k")
    assert_close_f32(lb, rb, 1e-4, "lmk_b")


def test_attn_pool_default_scale_and_explicit(pkg, orc, dev):
    torch.manual_seed(1)
    mu = torch.randn(1, 8, 2, 64).bfloat16()
    k = torch.randn(1, 8, 64, 2, 64).bfloat16()
    a = pkg.chunk_attn_pool_tilelang(mu.to(dev), k.to(dev))
    b = pkg.chunk_attn_pool_tilelang(mu.to(dev), k.to(dev), sm_scale=1 / math.sqrt(64))
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    c = pkg.chunk_attn_pool_tilelang(mu.to(dev), k.to(dev), sm_scale=0.3)
    rk, rb, _ = orc.chunk_attn_pool(mu, k, 0.3)
    assert_close_bf16(c[0], rk, "lmk_k scale 0.3")
    assert_close_f32(c[1], rb, 1e-4, "lmk_b scale 0.3")


def test_attn_pool_last_token_masked(pkg, dev):
    """Changing the landmark (last) token of every chunk must not change any output."""
    torch.manual_seed(2)
    mu = torch.randn(1, 8, 2, 64).bfloat16()
    k = torch.randn(1, 8, 64, 2, 64).bfloat16()
    k2 = k.clone()
    k2[:, :, -1] = torch.randn(1, 8, 2, 64).bfloat16() * 10
    a = pkg.chunk_attn_pool_tilelang(mu.to(dev), k.to(dev))
    b = pkg.chunk_attn_pool_tilelang(mu.to(dev), k2.to(dev))
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_attn_pool_compact(pkg, orc, dev):
    torch.manual_seed(3)
    mu = torch.randn(1, 8, 2, 64).bfloat16()
    k = torch.randn(1, 8, 64, 2, 64).bfloat16()
    lk, lb = pkg.chunk_attn_pool_tilelang(mu.to(dev), k.to(dev), compact_lmk_k=True)
    assert torch.count_nonzero(lk).item() == 0
    assert_close_f32(lb, orc.chunk_attn_pool(mu, k)[1], 1e-4, "lmk_b compact")


def _pool_grads(orc, mu, k, gk, gb, scale=None):
    mu_f = mu.float().requires_grad_()
    k_f = k.float().requires_grad_()
    rk, rb, _ = orc.chunk_attn_pool(mu_f, k_f, scale)
    ((rk * gk.float()).sum() + (rb * gb).sum()).backward()
    return mu_f.grad, k_f.grad


@pytest.mark.parametrize("B,N,H,D,S", [(1, 16, 2, 128, 64), (2, 8, 4, 64, 64), (1, 8, 1, 128, 32)])
def test_attn_pool_bwd(pkg, orc, dev, B, N, H, D, S):
    note(f"attn_pool_bwd B{B} N{N} H{H} D{D} S{S}")
    torch.manual_seed(42)
    mu = torch.randn(B, N, H, D).bfloat16()
    k = torch.randn(B, N, S, H, D).bfloat16()
    gk = torch.randn(B, N, H, D).bfloat16()
    gb = torch.randn(B, N, H)
    mu_d = mu.to(dev).requires_grad_()
    k_d = k.to(dev).requires_grad_()
    lk, lb = pkg.chunk_attn_pool_tilelang(mu_d, k_d)
    torch.autograd.backward([lk, lb], [gk.to(dev), gb.to(dev)])
    rmu, rk = _pool_grads(orc, mu, k, gk, gb)
    assert_close_bf16(mu_d.grad, rmu, "d_mu")
    assert_close_bf16(k_d.grad, rk, "d_k")


def test_attn_pool_bwd_compact_ignores_grad_k(pkg, orc, dev):
    """With compact_lmk_k the gradient w.r.t. lmk_k is ignored bit-exactly
    (reference: unittests/test_chunk_attn_pool_tilelang.py:292-420)."""
    torch.manual_seed(5)
    mu = torch.randn(1, 8, 2, 64).bfloat16()
    k = torch.randn(1, 8, 64, 2, 64).bfloat16()
    gb = torch.randn(1, 8, 2)
    outs = []
    for gk_scale in (0.0, 7.0):
        mu_d = mu.to(dev).requires_grad_()
        k_d = k.to(dev).requires_grad_()
        lk, lb = pkg.chunk_attn_pool_tilelang(mu_d, k_d, compact_lmk_k=True)
        gk = torch.randn(1, 8, 2, 64).bfloat16() * gk_scale
        torch.autograd.backward([lk, lb], [gk.to(dev), gb.to(dev)])
        outs.append((mu_d.grad.clone(), k_d.grad.clone()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    rmu, rk = _pool_grads(orc, mu, k, torch.zeros(1, 8, 2, 64), gb)
    assert_close_bf16(outs[0][0], rmu, "d_mu compact")
    assert_close_bf16(outs[0][1], rk, "d_k compact")


def test_attn_pool_shared_k(pkg, orc, dev):
    """Shared-K variant: forward equals the plain op on K broadcast over heads; backward sums
    dK over heads into head 0 and zeroes the others
    (reference: unittests/test_chunk_attn_pool_tilelang.py:135-154, :435-497)."""
    torch.manual_seed(6)
    B, N, H, D, S = 1, 8, 16, 64, 64
    mu = torch.randn(B, N, H, D).bfloat16()
    k1 = torch.randn(B, N, S, 1, D).bfloat16()
    k = k1.expand(B, N, S, H, D).contiguous()
    gk = torch.randn(B, N, H, D).bfloat16()
    gb = torch.randn(B, N, H)
    mu_d = mu.to(dev).requires_grad_()
    k_d = k.to(dev).requires_grad_()
    lk, lb = pkg.chunk_attn_pool_tilelang_shared_k(mu_d, k_d)
    rk_, rb_, _ = orc.chunk_attn_pool(mu, k)
    assert_close_bf16(lk, rk_, "shared lmk_k")
    assert_close_f32(lb, rb_, 1e-4, "shared lmk_b")
    torch.autograd.backward([lk, lb], [gk.to(dev), gb.to(dev)])
    rmu, rk = _pool_grads(orc, mu, k, gk, gb)
    assert_close_bf16(mu_d.grad, rmu, "shared d_mu")
    assert_close_bf16(k_d.grad[:, :, :, 0], rk.sum(dim=3), "shared d_k head 0")
    assert torch.count_nonzero(k_d.grad[:, :, :, 1:]).item() == 0
    with pytest.raises(AssertionError):
        pkg.chunk_attn_pool_tilelang_shared_k(mu_d[:, :, :8], k_d[:, :, :, :8])


@pytest.mark.parametrize("B,N,H,HK,D,S", [(1, 40, 32, 8, 128, 64), (2, 9, 8, 2, 64, 64), (1, 5, 6, 3, 128, 64),
                                           (1, 7, 16, 1, 64, 64), (1, 3, 32, 1, 128, 64),
                                           # other chunk sizes / head dims: the kernels that stage K in LDS
                                           (1, 6, 8, 2, 128, 32), (2, 3, 4, 2, 32, 16)])
def test_attn_pool_grouped_query_heads(pkg, orc, dev, B, N, H, HK, D, S):
    """K at the model's own KV head count (models/FlashHiLS/hils_attention.py:66-135): forward and
    backward equal the oracle on K repeated to the query heads, dK being the sum over a group."""
    note(f"attn_pool grouped B{B} N{N} H{H}/{HK} D{D} S{S}")
    torch.manual_seed(43)
    G = H // HK
    mu = torch.randn(B, N, H, D).bfloat16()
    k = torch.randn(B, N, S, HK, D).bfloat16()
    gk = torch.randn(B, N, H, D).bfloat16()
    gb = torch.randn(B, N, H)
    mu_d = mu.to(dev).requires_grad_()
    k_d = k.to(dev).requires_grad_()
    lk, lb = pkg.chunk_attn_pool(mu_d, k_d)
    k_rep = k.repeat_interleave(G, dim=3)
    rk_, rb_, _ = orc.chunk_attn_pool(mu, k_rep)
    assert lk.shape == (B, N, H, D) and lb.shape == (B, N, H) and lb.dtype == torch.float32
    assert_close_bf16(lk, rk_, "grouped lmk_k")
    assert_close_f32(lb, rb_, 1e-4, "grouped lmk_b")
    # and the per-head kernels on the repeated K (the logits are summed in another order)
    lk2, lb2 = pkg.chunk_attn_pool_tilelang(mu.to(dev), k_rep.to(dev))
    assert_close_bf16(lk, lk2.float(), "grouped vs per-head lmk_k")
    assert_close_f32(lb, lb2, 2e-5, "grouped vs per-head lmk_b")
    torch.autograd.backward([lk, lb], [gk.to(dev), gb.to(dev)])
    rmu, rk = _pool_grads(orc, mu, k_rep, gk, gb)
    assert_close_bf16(mu_d.grad, rmu, "grouped d_mu")
    assert k_d.grad.shape == k.shape
    assert_close_bf16(k_d.grad, rk.view(B, N, S, HK, G, D).sum(4), "grouped d_k")


def test_attn_pool_argument_errors(pkg, dev):
    """The wrapper's own argument checks (models/FlashHiLS/hils_attention.py:113-131)."""
    mu = torch.randn(1, 4, 6, 64, device=dev).bfloat16()
    k = torch.randn(1, 4, 64, 4, 64, device=dev).bfloat16()
    with pytest.raises(ValueError, match="multiple"):
        pkg.chunk_attn_pool(mu, k)
    with pytest.raises(ValueError, match="expected mu_q"):
        pkg.chunk_attn_pool(mu[0], k)
    with pytest.raises(ValueError, match="mismatch"):
        pkg.chunk_attn_pool(mu[:, :3], k[:, :, :, :3])


@pytest.mark.parametrize("B,L,H,D,S", [(1, 2048, 4, 64, 64), (2, 1024, 8, 128, 64), (1, 256, 2, 64, 32),
                                        (1, 128, 1, 8, 16)])
def test_mean_pool(pkg, orc, dev, B, L, H, D, S):
    note(f"mean_pool B{B} L{L} H{H} D{D} S{S}")
    torch.manual_seed(7)
    k = torch.randn(B, L, H, D).bfloat16()
    k_d = k.to(dev).requires_grad_()
    out = pkg.chunk_mean_pool(k_d, S)
    assert_close_bf16(out, orc.mean_pool(k, S), "mean pool", max_abs=4e-3)
    g = torch.randn(out.shape).bfloat16()
    out.backward(g.to(dev))
    ref = (g.float() / S).repeat_interleave(S, dim=1)
    assert_close_bf16(k_d.grad, ref, "mean pool bwd", max_abs=4e-3)
