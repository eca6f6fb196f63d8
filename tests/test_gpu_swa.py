"""HIP sliding-window attention (forward of flex_attn_tl) vs the CPU oracle, through the C ABI.

The reference checks this operator against torch's flex_attention with the mask of
ops/flex_attn_tilelang.py:1355-1386; the oracle restates that mask."""
import pytest
import torch

from util import LSE_TOL, assert_close_bf16, assert_close_f32, note

pytestmark = pytest.mark.gpu


def run(pkg, orc, dev, B, Lq, Lk, HQ, H, D, Dv, W, S, mask_lmk=True, expand=True, kv_start=0, seed=42,
        sm_scale=None):
    note(f"swa B{B} Lq{Lq} Lk{Lk} HQ{HQ} H{H} D{D} Dv{Dv} W{W} S{S} lmk{mask_lmk} exp{expand} kv0 {kv_start}")
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Lq, HQ, D, generator=gen).bfloat16()
    k = torch.randn(B, Lk, H, D, generator=gen).bfloat16()
    v = torch.randn(B, Lk, H, Dv, generator=gen).bfloat16()
    o, lse = pkg.flex_attn_tl(q.to(dev), k.to(dev), v.to(dev), W, S, training=(Lq == Lk and kv_start == 0),
                              mask_lmk=mask_lmk, expand_to_chunk=expand, sm_scale=sm_scale, kv_start=kv_start)
    torch.cuda.synchronize()
    ro, rlse = orc.swa(q, k, v, window_size=W, chunk_size=S, mask_lmk=mask_lmk, expand_to_chunk=expand,
                       kv_start=kv_start, sm_scale=sm_scale)
    assert o.dtype == torch.bfloat16 and o.shape == (B, Lq, HQ, Dv)
    assert lse.dtype == torch.float32 and lse.shape == (B, Lq, HQ)
    assert_close_bf16(o, ro, "swa o")
    assert_close_f32(lse, rlse, LSE_TOL, "swa lse")  # also the -inf pattern (rows that see no key)


@pytest.mark.parametrize("B,L,HQ,H,D,W,S", [
    (1, 512, 8, 2, 128, 64, 64), (2, 300, 4, 4, 64, 64, 64), (1, 1000, 16, 1, 64, 128, 64),
    (1, 257, 2, 1, 128, 1, 64), (1, 700, 8, 4, 64, 200, 32), (1, 130, 2, 2, 64, 512, 64)])
def test_swa_training_shapes(pkg, orc, dev, B, L, HQ, H, D, W, S):
    run(pkg, orc, dev, B, L, L, HQ, H, D, D, W, S)


def test_swa_mask_variants(pkg, orc, dev):
    for mask_lmk in (False, True):
        for expand in (False, True):
            run(pkg, orc, dev, 1, 400, 400, 4, 2, 64, 64, 48, 64, mask_lmk=mask_lmk, expand=expand)
    # chunk size that is not a power of two; explicit scale; different value head dim
    run(pkg, orc, dev, 1, 333, 333, 4, 1, 128, 64, 100, 48, sm_scale=0.05)
    run(pkg, orc, dev, 1, 200, 200, 2, 2, 64, 128, 30, 20, expand=False)
    # sharp softmax over several key tiles: a row's running maximum both jumps far (the accumulated
    # output is rescaled) and creeps (it is not), for 8- and 4-wavefront workgroups
    run(pkg, orc, dev, 1, 500, 500, 4, 2, 64, 64, 200, 64, sm_scale=0.7)
    run(pkg, orc, dev, 1, 500, 500, 8, 2, 128, 128, 64, 64, sm_scale=0.5)
    run(pkg, orc, dev, 1, 500, 500, 4, 4, 64, 64, 100, 64, sm_scale=0.6, expand=False)


def test_swa_inference_cache_and_truncated_cache(pkg, orc, dev):
    # decode: one query against a cache; chunked prefill: 100 queries at the end of 612 keys;
    # a cache truncated by sliding-window generation (kv_start > 0)
    run(pkg, orc, dev, 3, 1, 777, 8, 2, 128, 128, 64, 64)
    run(pkg, orc, dev, 1, 100, 612, 8, 2, 64, 64, 64, 64)
    run(pkg, orc, dev, 2, 5, 150, 4, 4, 64, 64, 64, 64, kv_start=4000)
    run(pkg, orc, dev, 1, 64, 64, 16, 2, 128, 128, 32, 64, kv_start=0)


def test_swa_landmark_query_row_sees_no_key(pkg, dev):
    """window 1 on a landmark position: the only candidate key is masked -> o = 0, lse = -inf."""
    q = torch.randn(1, 128, 2, 64, device=dev).bfloat16()
    o, lse = pkg.flex_attn_tl(q, q, q, 1, 64, expand_to_chunk=False)
    assert lse[0, 63, 0].item() == float("-inf") and lse[0, 127, 1].item() == float("-inf")
    assert torch.count_nonzero(o[0, 63]).item() == 0
    assert torch.isfinite(lse[0, 62]).all()


@pytest.mark.parametrize("B,L,HQ,H,D,Dv,W,S,mask_lmk,expand", [
    (1, 384, 4, 2, 64, 64, 64, 64, True, True), (2, 200, 8, 2, 128, 128, 48, 64, True, True),
    (1, 300, 2, 2, 64, 128, 100, 32, False, True), (1, 260, 16, 1, 64, 64, 33, 48, True, False),
    (1, 513, 4, 4, 128, 64, 1, 64, False, False)])
def test_swa_backward(pkg, orc, dev, B, L, HQ, H, D, Dv, W, S, mask_lmk, expand):
    """dq, dk, dv with gradients arriving through both outputs (o and lse)."""
    _forward_backward(pkg, orc, dev, B, L, HQ, H, D, Dv, W, S, mask_lmk, expand)


@pytest.mark.parametrize("HQ,H,D", [(16, 2, 64), (8, 8, 128)])
@pytest.mark.parametrize("W", [256, 512])
def test_swa_long_windows_forward_backward(pkg, orc, dev, HQ, H, D, W):
    """Windows of several key tiles on a sequence of many query blocks: the windows and head shapes the
    reference times this operator at (scripts/bench/bench_flex_attn_bwd_clamp.py:66-72), forward and
    backward against the oracle."""
    _forward_backward(pkg, orc, dev, 1, 2048, HQ, H, D, D, W, 64, True, True)


def _forward_backward(pkg, orc, dev, B, L, HQ, H, D, Dv, W, S, mask_lmk, expand):
    note(f"swa_bwd B{B} L{L} HQ{HQ} H{H} D{D} Dv{Dv} W{W} S{S} lmk{mask_lmk} exp{expand}")
    gen = torch.Generator().manual_seed(7)
    q = torch.randn(B, L, HQ, D, generator=gen).bfloat16()
    k = torch.randn(B, L, H, D, generator=gen).bfloat16()
    v = torch.randn(B, L, H, Dv, generator=gen).bfloat16()
    do = torch.randn(B, L, HQ, Dv, generator=gen).bfloat16()
    dl = torch.randn(B, L, HQ, generator=gen)
    qd, kd, vd = (t.to(dev).requires_grad_() for t in (q, k, v))
    o, lse = pkg.flex_attn_tl(qd, kd, vd, W, S, mask_lmk=mask_lmk, expand_to_chunk=expand)
    fin = torch.isfinite(lse)
    ((o.float() * do.to(dev).float()).sum() + torch.where(fin, lse, torch.zeros_like(lse)).mul(dl.to(dev)).sum()).backward()
    qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
    ro, rlse = orc.swa(qf, kf, vf, window_size=W, chunk_size=S, mask_lmk=mask_lmk, expand_to_chunk=expand)
    rfin = torch.isfinite(rlse)
    assert torch.equal(fin.cpu(), rfin)
    assert_close_bf16(o, ro.detach(), "swa o")
    assert_close_f32(lse.detach(), rlse.detach(), LSE_TOL, "swa lse")
    ((ro * do.float()).sum() + torch.where(rfin, rlse, torch.zeros_like(rlse)).mul(dl).sum()).backward()
    assert_close_bf16(qd.grad, qf.grad, "swa dq")
    assert_close_bf16(kd.grad, kf.grad, "swa dk")
    assert_close_bf16(vd.grad, vf.grad, "swa dv")


def test_swa_backward_only_through_o(pkg, orc, dev):
    torch.manual_seed(8)
    q, k, v = (torch.randn(1, 192, h, 64).bfloat16() for h in (4, 2, 2))
    qd, kd, vd = (t.to(dev).requires_grad_() for t in (q, k, v))
    o, _ = pkg.flex_attn_tl(qd, kd, vd, 64, 64)
    o.float().pow(2).sum().backward()
    qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
    ro, _ = orc.swa(qf, kf, vf, window_size=64, chunk_size=64)
    ro.pow(2).sum().backward()
    assert_close_bf16(qd.grad, qf.grad, "swa dq (o only)")
    assert_close_bf16(kd.grad, kf.grad, "swa dk (o only)")
    assert_close_bf16(vd.grad, vf.grad, "swa dv (o only)")


def test_swa_two_phase_name_is_the_same_operator(pkg, dev):
    q = torch.randn(1, 130, 4, 64, device=dev).bfloat16()
    k = torch.randn(1, 130, 2, 64, device=dev).bfloat16()
    a = pkg.flex_attn_tl(q, k, k, 40, 64)
    b = pkg.flex_attn_tl_two_phase(q, k, k, 40, 64)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    with pytest.raises(ValueError):
        pkg.flex_attn_tl_two_phase(q, k, k, 40, 64, training=True, kv_start=3)


def test_swa_inference_backward_raises_and_argument_errors(pkg, dev):
    q = torch.randn(1, 64, 2, 64, device=dev).bfloat16().requires_grad_()
    o, lse = pkg.flex_attn_tl(q, q.detach(), q.detach(), 16, 64, training=False)
    with pytest.raises(RuntimeError):
        o.sum().backward()
    with pytest.raises(ValueError):
        pkg.flex_attn_tl(q, q, q, 16, 64, training=True, kv_start=5)
    with pytest.raises(RuntimeError):  # head dim the kernels do not cover
        x = torch.randn(1, 64, 2, 32, device=dev).bfloat16()
        pkg.flex_attn_tl(x, x, x, 16, 64)


@pytest.mark.parametrize("L,HQ,H,D,W", [(512, 4, 2, 64, 64), (448, 8, 2, 128, 1)])
def test_local_and_remote_branch_sum_to_dense_attention(pkg, dev, L, HQ, H, D, W):
    """Every piece on the GPU: local branch (o, lse) + every remote chunk selected with the weights
    softmax([log Z_c, lse_swa]) must equal ordinary causal attention over the non-landmark tokens
    (torch scaled_dot_product_attention); the log-sum-exps must add up to the dense one."""
    import torch.nn.functional as F
    torch.manual_seed(17)
    B, S = 1, 64
    N = L // S
    q = (torch.randn(B, L, HQ, D, device=dev) * 0.5).bfloat16()
    k = (torch.randn(B, L, H, D, device=dev) * 0.5).bfloat16()
    v = torch.randn(B, L, H, D, device=dev).bfloat16()
    swa_o, lse_swa = pkg.flex_attn_tl(q, k, v, W, S, mask_lmk=True)
    log_z = pkg.exact_chunk_log_z_tl(q, k, chunk_size=S, window_size=W, mask_lmk=True)
    t = torch.arange(L, device=dev)
    lim = torch.div(t - W + 1, S, rounding_mode="floor").clamp_min(0)  # fully remote chunks per query
    idx = torch.arange(N, device=dev).view(1, 1, 1, N).expand(B, L, H, N)
    idx = torch.where(idx < lim.view(1, L, 1, 1), idx, torch.full_like(idx, -1)).to(torch.int32).contiguous()
    wts = torch.softmax(torch.cat([log_z, lse_swa.unsqueeze(-1)], -1), -1)
    o_sparse = pkg.HiLS_block_M_head(q, k, v, wts.bfloat16(), idx, block_size=S, is_training=False)
    o = o_sparse.float() + swa_o.float() * wts[..., N].bfloat16().float().unsqueeze(-1)
    keep = (t.view(1, L) <= t.view(L, 1)) & (((t + 1) % S) != 0).view(1, L)
    G = HQ // H
    qf, kf, vf = q.float().transpose(1, 2), k.float().repeat_interleave(G, 2).transpose(1, 2), \
        v.float().repeat_interleave(G, 2).transpose(1, 2)
    dense = F.scaled_dot_product_attention(qf, kf, vf, attn_mask=keep).transpose(1, 2)
    row_ok = keep.any(-1)  # query 63 with window 1 ... sees nothing but earlier chunks: still fine
    assert_close_bf16(o[:, row_ok].cpu(), dense[:, row_ok].cpu(), "local + remote == dense", max_abs=2e-2,
                      rel_l2=1.5e-2)
    s = torch.einsum("bhid,bhjd->bhij", qf, kf) / D ** 0.5
    full_lse = torch.logsumexp(s.masked_fill(~keep, float("-inf")), -1).transpose(1, 2)
    total = torch.logaddexp(torch.logsumexp(log_z, -1), lse_swa)
    fin = torch.isfinite(full_lse)
    assert (total[fin] - full_lse[fin]).abs().max().item() < 2e-3
