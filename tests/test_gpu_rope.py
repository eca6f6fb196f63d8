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


@pytest.mark.parametrize("B,L,H,D,S,norm,rot,per_batch", [(1, 512, 4, 128, 64, True, True, False),
                                                          (2, 200, 3, 64, 64, True, True, True),    # ragged tail chunk
                                                          (1, 256, 2, 256, 32, True, False, False),  # norm only, 32-token chunks
                                                          (2, 192, 8, 128, 64, False, True, False),  # rotation only
                                                          (1, 128, 2, 64, 64, False, False, False)])  # plain chunk mean
def test_norm_rope_pool(pkg, orc, dev, B, L, H, D, S, norm, rot, per_batch):
    """One pass for the layer's key preparation: against the oracle run in bf16 (the layer's own
    roundings: nearly every element identical, none further than two bf16 steps) and in fp64 (the
    exact function), forward and backward."""
    note(f"norm_rope_pool B{B} L{L} H{H} D{D} S{S} norm={norm} rot={rot}")
    torch.manual_seed(41)
    x = (torch.randn(B, L, H, D) * 1.5).bfloat16()
    w = (torch.rand(D) + 0.5).bfloat16() if norm else None
    cos = sin = None
    if rot:
        ang = torch.rand(B if per_batch else 1, L, D // 2) * 6.0
        cos = torch.cat([ang.cos(), ang.cos()], -1).bfloat16()
        sin = torch.cat([ang.sin(), ang.sin()], -1).bfloat16()
        if not per_batch:
            cos, sin = cos[0], sin[0]
    xd = x.to(dev).requires_grad_()
    wd = w.to(dev).requires_grad_() if norm else None
    out, lmk = pkg.norm_rope_pool(xd, wd, None if cos is None else cos.to(dev), None if sin is None else sin.to(dev), S)
    ref_o, ref_l = orc.norm_rope_pool(x, w, cos, sin, S)  # bf16 arithmetic, op by op
    got_o, got_l = out.detach().cpu(), lmk.detach().cpu()
    same = (got_o == ref_o).float().mean().item()
    step = (got_o.float() - ref_o.float()).abs() / ref_o.float().abs().clamp_min(1e-3)
    note(f"    out: {same * 100:.3f} % of the elements bit-identical, worst relative difference {step.max().item():.2e}")
    # (a last-bit difference of the fp32 reciprocal square root can move the first rounding by one
    # bf16 step, and a later rounding by one more)
    assert same >= 0.995 and step.max().item() <= 2 ** -6
    assert_close_bf16(got_l, ref_l.float(), "pooled keys vs bf16 oracle")
    x64 = x.double().requires_grad_()
    w64 = w.double().requires_grad_() if norm else None
    o64, l64 = orc.norm_rope_pool(x64, w64, None if cos is None else cos.double(), None if sin is None else sin.double(), S)
    assert_close_bf16(got_o, o64.detach().float(), "out vs fp64 oracle")
    assert_close_bf16(got_l, l64.detach().float(), "pooled keys vs fp64 oracle")
    g_o = torch.randn(B, L, H, D).bfloat16()
    g_l = torch.randn(B, L // S, H, D).bfloat16()
    (out.float() * g_o.to(dev).float()).sum().backward(retain_graph=True)
    dx_o = xd.grad.clone(); xd.grad = None
    (o64 * g_o.double()).sum().backward(retain_graph=True)
    assert_close_bf16(dx_o.cpu(), x64.grad.float(), "dx from d_out alone"); x64.grad = None
    if norm:
        wd.grad = None; w64.grad = None
    ((out.float() * g_o.to(dev).float()).sum() + (lmk.float() * g_l.to(dev).float()).sum()).backward()
    ((o64 * g_o.double()).sum() + (l64 * g_l.double()).sum()).backward()
    assert_close_bf16(xd.grad.cpu(), x64.grad.float(), "dx")
    if norm:
        assert_close_bf16(wd.grad.cpu(), w64.grad.float(), "d_weight")
    # the query side: no pooled output
    o_q, none = pkg.norm_rope_pool(x.to(dev), w.to(dev) if norm else None, None if cos is None else cos.to(dev),
                                   None if sin is None else sin.to(dev), S, pool=False)
    assert none is None and torch.equal(o_q.cpu(), got_o)
