"""HIP rotary position embedding vs the CPU oracle, through the C ABI.  Shapes follow the
reference's in-file tests (ops/rope_tilelang_fp32.py:192-215, :394-420)."""
import pytest
import torch

from util import assert_close_bf16, note

pytestmark = pytest.mark.gpu


def tables(L, D, batch=None, dtype=torch.bfloat16, seed=3):
    gen = torch.Generator().manual_seed(seed)
    shape = (L, D // 2) if batch is None else (batch, L, D // 2)
    ang = torch.rand(*shape, generator=gen) * 6.283
    return torch.cat([ang.cos(), ang.cos()], -1).to(dtype), torch.cat([ang.sin(), ang.sin()], -1).to(dtype)


@pytest.mark.parametrize("B,L,HQ,H,D", [(2, 1024, 8, 2, 128), (1, 333, 4, 4, 64), (3, 17, 2, 1, 96)])
def test_rope_two_tensors(pkg, orc, dev, B, L, HQ, H, D):
    note(f"rope q,k B{B} L{L} HQ{HQ} H{H} D{D}")
    torch.manual_seed(42)
    q, k = torch.randn(B, L, HQ, D).bfloat16(), torch.randn(B, L, H, D).bfloat16()
    cos, sin = tables(L, D, batch=B)
    qo, ko = pkg.rope_rotary_pos_emb(q.to(dev), k.to(dev), cos.to(dev), sin.to(dev))
    assert qo.dtype == torch.bfloat16 and qo.shape == q.shape and ko.shape == k.shape
    assert_close_bf16(qo, orc.rope(q, cos, sin, lo_only=True), "rope q")
    assert_close_bf16(ko, orc.rope(k, cos, sin, lo_only=True), "rope k")


@pytest.mark.parametrize("tab_dtype,with_batch_dim", [(torch.bfloat16, False), (torch.float32, True)])
def test_rope_single_tensor_forward_backward(pkg, orc, dev, tab_dtype, with_batch_dim):
    note(f"rope single tensor tables {tab_dtype}")
    torch.manual_seed(42)
    B, L, H, D = 2, 500, 6, 128
    x = torch.randn(B, L, H, D).bfloat16()
    gen = torch.Generator().manual_seed(9)
    cos = torch.randn(L, D, generator=gen).to(tab_dtype)  # halves differ on purpose
    sin = torch.randn(L, D, generator=gen).to(tab_dtype)
    g = torch.randn(B, L, H, D).bfloat16()
    cd, sd = (cos.unsqueeze(0), sin.unsqueeze(0)) if with_batch_dim else (cos, sin)
    xd = x.to(dev).requires_grad_()
    out = pkg.single_tensor_rope_autograd(xd, cd.to(dev), sd.to(dev))
    out.backward(g.to(dev))
    xf = x.float().requires_grad_()
    ref = orc.rope(xf, cos, sin)
    ref.backward(g.float())
    assert out.dtype == torch.bfloat16
    assert_close_bf16(out, ref.detach(), "rope out")
    # the reference's backward is the rotation by the opposite angle; for tables with equal halves
    # that is the exact gradient, for these arbitrary tables it is what the reference computes
    want = orc.rope(g, cos, -sin.float())
    assert_close_bf16(xd.grad, want, "rope backward (rotation with -sin)")
    c2, s2 = tables(L, D, dtype=tab_dtype)
    xd2 = x.to(dev).requires_grad_()
    pkg.single_tensor_rope_autograd(xd2, c2.to(dev), s2.to(dev)).backward(g.to(dev))
    xf2 = x.float().requires_grad_()
    orc.rope(xf2, c2, s2).backward(g.float())
    assert_close_bf16(xd2.grad, xf2.grad, "rope backward == autograd for rotation tables")


def test_rope_argument_errors(pkg, dev):
    x = torch.randn(1, 8, 2, 64, device=dev).bfloat16()
    bad = torch.randn(2, 8, 64, device=dev).bfloat16()
    with pytest.raises(AssertionError):
        pkg.single_tensor_rope_autograd(x, bad, bad)
    with pytest.raises(RuntimeError):
        y = torch.randn(1, 8, 2, 40, device=dev).bfloat16()
        t = torch.randn(8, 40, device=dev).bfloat16()
        pkg.single_tensor_rope_autograd(y, t, t)
