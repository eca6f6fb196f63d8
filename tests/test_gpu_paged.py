"""Decode over a paged cache (page = chunk = 64 tokens) against the same data kept token-major:
the kernels read other addresses, the arithmetic is the same, so everything must agree bit for bit."""
import math

import pytest
import torch

from util import assert_close_bf16, note

pytestmark = pytest.mark.gpu


def _paged_copy(k, v, lmk, dev, seed, spare=5):
    """Scatter a token-major cache (B, Lkv, H, D) into pages handed out in random order."""
    B, Lkv, H, D = k.shape
    n = Lkv // 64
    num_pages = B * n + spare
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(seed))[: B * n].view(B, n)
    k_pages = torch.randn(num_pages, H, 64, D).bfloat16()  # unmapped pages hold garbage
    v_pages = torch.randn(num_pages, H, 64, D).bfloat16()
    lmk_pages = torch.randn(num_pages, H, D).bfloat16()
    k_pages[perm] = k.view(B, n, 64, H, D).permute(0, 1, 3, 2, 4)
    v_pages[perm] = v.view(B, n, 64, H, D).permute(0, 1, 3, 2, 4)
    lmk_pages[perm] = lmk
    table = torch.full((B, n + 3), -1, dtype=torch.int32)
    table[:, :n] = perm.to(torch.int32)
    return k_pages.to(dev), v_pages.to(dev), lmk_pages.to(dev), table.to(dev)


@pytest.mark.parametrize("B,Lq,Lkv,HQ,H,D,K", [(32, 1, 32768, 32, 8, 128, 32), (16, 1, 16384, 8, 8, 64, 16),
                                               (50, 2, 20480, 4, 1, 128, 8),
                                               (64, 1, 32768, 16, 2, 64, 32), (20, 1, 32768, 40, 8, 128, 16),  # eight / five heads per KV head
                                               # short caches: the token-major call runs on other kernels
                                               (5, 1, 4096, 8, 2, 128, 16), (3, 2, 2048, 4, 4, 64, 8)])
def test_paged_decode_matches_contiguous(pkg, orc, dev, B, Lq, Lkv, HQ, H, D, K):
    note(f"paged decode B{B} Lq{Lq} Lkv{Lkv} HQ{HQ} H{H} D{D} K{K}")
    gen = torch.Generator().manual_seed(71)
    q = torch.randn(B, Lq, HQ, D, generator=gen).bfloat16()
    k = torch.randn(B, Lkv, H, D, generator=gen).bfloat16()
    v = torch.randn(B, Lkv, H, D, generator=gen).bfloat16()
    lse = torch.randn(B, Lq, HQ, generator=gen) * 3 + 5
    qd, kd, vd, lsed = q.to(dev), k.to(dev), v.to(dev), lse.to(dev)
    lmk = pkg.chunk_mean_pool(kd, 64)
    # the token-major cache through the same route (one launch where the shape allows it, else two calls)
    o0, w0, idx0, sc0 = pkg.decode_step(qd, lmk, kd, vd, lsed, K, 64, 1, q_offset=Lkv - Lq)
    k_pages, v_pages, lmk_pages, table = _paged_copy(k, v, lmk.cpu(), dev, seed=72)
    dbg = {}
    o1, w1, idx1 = pkg.paged_hils_attend(qd, k_pages, v_pages, lmk_pages, table, lsed, Lkv, K, 1, _debug=dbg)
    assert torch.equal(idx1, idx0), "indices differ between the paged and the token-major cache"
    same_kernels = Lkv // 64 >= 256 and B * Lq * H >= 96  # both on the one-launch kernel
    if same_kernels:
        assert torch.equal(dbg["scores"], sc0) and torch.equal(w1, w0)
        assert torch.equal(o1, o0), "attention output differs between the paged and the token-major cache"
    else:  # scores from another kernel: one bf16 step apart at most
        assert (dbg["scores"].float() - sc0.float()).abs().max().item() <= 2e-2
        assert (w1.float() - w0.float()).abs().max().item() <= 8e-3
        assert_close_bf16(o1, o0.float(), "paged vs token-major output")
    # and against the oracle (selection rule on the kernel's own logits, attention output)
    lim = orc.causal_chunk_limit(Lq, Lkv - Lq, 1, 64)
    want = orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim, K)
    assert torch.equal(idx1.cpu(), want)
    ref = orc.sparse_attn(q, k, v, w1.cpu(), idx1.cpu(), chunk_size=64)
    assert_close_bf16(o1, ref, "paged decode output")
    # a page that is not mapped is invisible: unmap the pages of chunk 3 and compare with a drop of chunk 3
    t2 = table.clone()
    t2[:, 3] = -1
    o2, w2, idx2 = pkg.paged_hils_attend(qd, k_pages, v_pages, lmk_pages, t2, lsed, Lkv, K, 1)
    assert not (idx2 == 3).any()


def test_paged_layer_appends_and_pools(pkg, orc, dev):
    """HiLSPagedLayer: prefill + token-by-token appends through a shuffled free list reproduce the
    contiguous cache (keys, values, mean-pooled chunk keys) and its remote branch."""
    note("HiLSPagedLayer")
    B, H, HQ, D, K = 3, 2, 8, 128, 8
    gen = torch.Generator().manual_seed(73)
    L0, steps = 700, 200
    k = torch.randn(B, L0 + steps, H, D, generator=gen).bfloat16().to(dev)
    v = torch.randn(B, L0 + steps, H, D, generator=gen).bfloat16().to(dev)
    order = torch.randperm(64, generator=gen).tolist()
    cache = pkg.HiLSPagedLayer(num_pages=64, batch=B, max_pages_per_seq=20, num_kv_heads=H, head_dim=D,
                               device=dev, page_order=order)
    cache.update(k[:, :L0], v[:, :L0])
    for t in range(L0, L0 + steps):
        cache.update(k[:, t:t + 1], v[:, t:t + 1])
    Lkv = L0 + steps
    kc, vc = cache.gather_contiguous()
    assert torch.equal(kc, k) and torch.equal(vc, v)
    lmk = pkg.chunk_mean_pool(k[:, : Lkv // 64 * 64].contiguous(), 64)
    got = cache.lmk_pages[cache.page_table[:, : Lkv // 64].long()]
    assert torch.equal(got, lmk), "pooled keys of the pages differ from the token-major mean pool"
    q = torch.randn(B, 1, HQ, D, generator=gen).bfloat16().to(dev)
    lse = (torch.randn(B, 1, HQ, generator=gen) * 2 + 4).to(dev)
    o1, w1, idx1 = cache.hils_attend(q, lse, K, 1)
    idx0, _, w0 = pkg.topk_chunk_weights(q, lmk, lse, K, 64, 1, q_offset=Lkv - 1)
    o0 = pkg.HiLS_block_M_head(q, k, v, w0, idx0, block_size=64, is_training=False)
    assert torch.equal(idx1, idx0) and torch.equal(w1, w0) and torch.equal(o1, o0)


def test_paged_layer_attention_pooled_prior(pkg, orc, dev):
    """With the chunks' prior queries the layer keeps attention-pooled chunk keys and the entropy bias
    per page, as the reference's per-layer prior cache does, filled incrementally."""
    note("HiLSPagedLayer prior")
    B, H, D = 2, 4, 64
    gen = torch.Generator().manual_seed(74)
    L = 64 * 5
    k = torch.randn(B, L, H, D, generator=gen).bfloat16().to(dev)
    v = torch.randn(B, L, H, D, generator=gen).bfloat16().to(dev)
    mu = torch.randn(B, 5, H, D, generator=gen).bfloat16().to(dev)
    cache = pkg.HiLSPagedLayer(num_pages=16, batch=B, max_pages_per_seq=8, num_kv_heads=H, head_dim=D, device=dev,
                               num_q_heads=H, chunk_pooling=False)
    cache.update(k[:, :128], v[:, :128], mu_q=mu[:, :2])      # two chunks at once
    for c in range(2, 5):                                      # then chunk by chunk, token by token
        for t in range(c * 64, c * 64 + 63):
            cache.update(k[:, t:t + 1], v[:, t:t + 1])
        t = c * 64 + 63
        cache.update(k[:, t:t + 1], v[:, t:t + 1], mu_q=mu[:, c:c + 1])
    lk, lb, _ = orc.chunk_attn_pool(mu.float().cpu(), k.view(B, 5, 64, H, D).float().cpu())
    pg = cache.page_table[:, :5].long()
    assert_close_bf16(cache.lmk_pages[pg], lk, "attention-pooled chunk keys per page")
    assert_close_bf16(cache.prior_b[pg], lb, "entropy bias per page", max_abs=2e-2)
