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


def test_swa_backward_raises_and_argument_errors(pkg, dev):
    q = torch.randn(1, 64, 2, 64, device=dev).bfloat16().requires_grad_()
    o, lse = pkg.flex_attn_tl(q, q.detach(), q.detach(), 16, 64)
    with pytest.raises(NotImplementedError):
        o.sum().backward()
    with pytest.raises(ValueError):
        pkg.flex_attn_tl(q, q, q, 16, 64, training=True, kv_start=5)
    with pytest.raises(RuntimeError):  # head dim the kernels do not cover
        x = torch.randn(1, 64, 2, 32, device=dev).bfloat16()
        pkg.flex_attn_tl(x, x, x, 16, 64)
