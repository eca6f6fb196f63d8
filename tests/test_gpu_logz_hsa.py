"""HIP exact chunk log-Z and the older HSA operator vs the CPU oracle, through the C ABI."""
import math

import pytest
import torch

from util import LSE_TOL, assert_close_bf16, assert_close_f32, note

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,L,HQ,H,D,S,W,mask_lmk", [
    (1, 512, 4, 2, 64, 64, 64, False), (2, 300, 4, 4, 64, 32, 16, False),
    (1, 512, 8, 2, 128, 64, 1, True), (1, 256, 2, 1, 64, 64, 0, False), (1, 100, 2, 2, 64, 64, 8, False),
    (1, 1100, 8, 2, 128, 64, 33, True), (2, 700, 16, 1, 64, 64, 1, False), (1, 650, 2, 2, 128, 64, 64, False),
    (1, 330, 16, 2, 64, 64, 64, True), (1, 200, 3, 1, 64, 64, 16, False)])
def test_logz_fwd(pkg, orc, dev, B, L, HQ, H, D, S, W, mask_lmk):
    note(f"logz_fwd B{B} L{L} HQ{HQ} H{H} D{D} S{S} W{W} lmk{mask_lmk}")
    torch.manual_seed(42)
    q = torch.randn(B, L, HQ, D).bfloat16()
    k = torch.randn(B, L, H, D).bfloat16()
    out = pkg.exact_chunk_log_z_tl(q.to(dev), k.to(dev), chunk_size=S, window_size=W, mask_lmk=mask_lmk)
    ref = orc.exact_chunk_log_z(q, k, chunk_size=S, window_size=W, mask_lmk=mask_lmk)
    assert out.dtype == torch.float32 and out.shape == ref.shape
    assert_close_f32(out, ref, LSE_TOL, "log_z")  # also checks the -inf pattern exactly


def test_logz_bwd(pkg, orc, dev):
    note("logz_bwd")
    torch.manual_seed(43)
    for (B, L, HQ, H, D, S, W) in [(1, 384, 4, 2, 64, 64, 32), (1, 200, 2, 2, 128, 32, 1),
                                   (1, 700, 8, 2, 128, 64, 64), (2, 330, 16, 1, 64, 64, 1),
                                   (1, 450, 2, 2, 128, 64, 17), (1, 300, 3, 1, 64, 64, 8)]:
        q = torch.randn(B, L, HQ, D).bfloat16()
        k = torch.randn(B, L, H, D).bfloat16()
        qd, kd = q.to(dev).requires_grad_(), k.to(dev).requires_grad_()
        out = pkg.exact_chunk_log_z_tl(qd, kd, chunk_size=S, window_size=W)
        g = torch.randn(out.shape)
        finite = torch.isfinite(out).cpu()
        g = torch.where(finite, g, torch.zeros(()))
        out.backward(g.to(dev))
        qf, kf = q.float().requires_grad_(), k.float().requires_grad_()
        ref = orc.exact_chunk_log_z(qf, kf, chunk_size=S, window_size=W)
        torch.where(finite, ref, torch.zeros(())).mul(g).sum().backward()
        assert_close_bf16(qd.grad, qf.grad, "logz dq")
        assert_close_bf16(kd.grad, kf.grad, "logz dk")


def test_logz_mask_lmk_backward_raises(pkg, dev):
    q = torch.randn(1, 128, 2, 64, device=dev).bfloat16().requires_grad_()
    k = torch.randn(1, 128, 2, 64, device=dev).bfloat16()
    out = pkg.exact_chunk_log_z_tl(q, k, chunk_size=64, window_size=1, mask_lmk=True)
    with pytest.raises(NotImplementedError):
        torch.where(torch.isfinite(out), out, torch.zeros((), device=dev)).sum().backward()


def test_logz_total_mass_invariant(pkg, orc, dev):
    """logaddexp(logsumexp_c log_Z, lse_swa) == LSE of full causal attention."""
    torch.manual_seed(44)
    B, L, HQ, H, D, S, W = 1, 512, 4, 2, 64, 64, 64
    q = (torch.randn(B, L, HQ, D) * 0.5).bfloat16()
    k = (torch.randn(B, L, H, D) * 0.5).bfloat16()
    lz = pkg.exact_chunk_log_z_tl(q.to(dev), k.to(dev), chunk_size=S, window_size=W).cpu()
    _, lse_swa = orc.swa(q, k, k, window_size=W, chunk_size=S, mask_lmk=False)
    total = torch.logaddexp(torch.logsumexp(lz, -1), lse_swa)
    s = torch.einsum("bihd,bjhd->bhij", q.float(), k.float().repeat_interleave(HQ // H, 2)) / math.sqrt(D)
    s = s.masked_fill(torch.ones(L, L, dtype=torch.bool).triu(1), float("-inf"))
    full = torch.logsumexp(s, -1).permute(0, 2, 1)
    assert_close_f32(total, full, 1e-4, "total mass")


@pytest.mark.parametrize("Z,HQ,H,N_CTX,D,K,S,Q_X,sm_n", [
    (1, 16, 1, 32, 16, 2, 16, 1, 1.0),    # the reference's own test shape (hsa_triton.py:818)
    (2, 16, 4, 256, 64, 4, 64, 16, 1.0), (2, 16, 1, 256, 64, 4, 64, 1, 0.0), (1, 8, 2, 128, 32, 4, 32, 4, 0.5),
    (1, 8, 2, 512, 128, 8, 64, 32, 2.0), (1, 4, 4, 320, 64, 3, 64, 8, 0.25)])
def test_hsa(pkg, orc, dev, Z, HQ, H, N_CTX, D, K, S, Q_X, sm_n):
    note(f"HSA Z{Z} HQ{HQ} H{H} L{N_CTX} D{D} K{K} S{S} QX{Q_X} sm_n{sm_n}")
    torch.manual_seed(22)
    q = (torch.randn(Z, N_CTX, HQ, D) * 0.5).bfloat16()
    k = (torch.randn(Z, N_CTX, H, D) * 0.5).bfloat16()
    v = (torch.randn(Z, N_CTX, H, D) * 0.5).bfloat16()
    nb = N_CTX // Q_X
    idx = torch.randint(0, N_CTX // S, (Z, nb, H, K), dtype=torch.int32)
    w = torch.softmax(torch.rand(Z, nb, H, K), -1).bfloat16()
    do = torch.randn(Z, N_CTX, HQ, D).bfloat16()
    qd, kd, vd, wd = (t.to(dev).requires_grad_() for t in (q, k, v, w))
    o = pkg.HSA(qd, kd, vd, wd, idx.to(dev), sm_n, S, 1 / math.sqrt(D))
    o.backward(do.to(dev))
    qf, kf, vf, wf = (t.float().requires_grad_() for t in (q, k, v, w))
    ref = orc.hsa(qf, kf, vf, wf, idx, sm_n, S, 1 / math.sqrt(D))
    ref.backward(do.float())
    assert_close_bf16(o, ref, "hsa o")
    assert_close_bf16(qd.grad, qf.grad, "hsa dq")
    assert_close_bf16(kd.grad, kf.grad, "hsa dk")
    assert_close_bf16(vd.grad, vf.grad, "hsa dv")
    assert_close_bf16(wd.grad, wf.grad, "hsa dw")


def test_hsa_sm_n_zero_equals_hils_without_mask(pkg, dev):
    torch.manual_seed(23)
    Z, L, HQ, H, D, K, S = 1, 128, 8, 2, 64, 2, 64
    q, k, v = (torch.randn(Z, L, h, D, device=dev).bfloat16() for h in (HQ, H, H))
    idx = torch.randint(0, L // S, (Z, L, H, K), dtype=torch.int32, device=dev)
    w = torch.softmax(torch.rand(Z, L, H, K, device=dev), -1).bfloat16()
    a = pkg.HSA(q, k, v, w, idx, 0.0, S, None)
    b = pkg.HiLS_block_M_head(q, k, v, w.repeat_interleave(HQ // H, 2).contiguous(), idx, block_size=S,
                              mask_last_token=False, is_training=False)
    # the two entry points may run on different kernels (shape-generic vs MFMA): same math
    assert_close_bf16(a, b.float(), "hsa(sm_n=0) vs hils(no mask)", max_abs=1e-2, rel_l2=5e-3)
