"""Decode cache with incrementally pooled chunk keys: every step on the in-place buffers must equal
the oracle run from scratch on the tokens seen so far."""
import pytest
import torch

from util import assert_close_bf16, note

pytestmark = pytest.mark.gpu


def test_incremental_cache_matches_recomputation(pkg, orc, dev):
    note("HiLSDynamicLayer: prefill 300 tokens, then 140 decode steps")
    B, HQ, H, D, S, K, W = 2, 8, 2, 64, 64, 4, 1
    gen = torch.Generator().manual_seed(5)
    L0, steps = 300, 140
    k_all = torch.randn(B, L0 + steps, H, D, generator=gen).bfloat16()
    v_all = torch.randn(B, L0 + steps, H, D, generator=gen).bfloat16()
    cache = pkg.HiLSDynamicLayer(chunk_size=S, capacity=128)  # forces two growth steps
    kk, vv = cache.update(k_all[:, :L0].to(dev), v_all[:, :L0].to(dev))
    assert kk.shape == (B, L0, H, D) and cache.get_seq_length() == L0 and cache.pooled_chunks == L0 // S
    for t in range(L0, L0 + steps):
        cache.update(k_all[:, t:t + 1].to(dev), v_all[:, t:t + 1].to(dev))
        if t % 23 and t not in (L0 + steps - 1, 319, 320, 383, 384):
            continue  # check around chunk boundaries and every 23rd step
        n = t + 1
        q = torch.randn(B, 1, HQ, D, generator=gen).bfloat16()
        lse = torch.randn(B, 1, HQ, generator=gen) * 2 + 3
        o, w, idx = cache.hils_attend(q.to(dev), lse.to(dev), K, W)
        assert cache.pooled_chunks == n // S
        # from scratch on the n tokens seen so far
        k_n, v_n = k_all[:, :n], v_all[:, :n]
        full = n // S
        lmk = orc.mean_pool(k_n[:, : full * S], S).bfloat16()
        assert torch.equal(cache.lmk_k[:, :full].cpu(), lmk)
        ridx, rsc = orc.online_softmax_topk_head(q.view(B, 1, H, HQ // H, D), lmk, lse, K, S, W, is_causal=True,
                                                 q_offset=n - 1)
        agree = (idx.cpu() == ridx).float().mean().item()
        assert agree >= 0.95, f"step {t}: index agreement {agree:.3f}"
        k_pad = torch.zeros(B, cache.capacity, H, D, dtype=k_n.dtype)
        v_pad = torch.zeros_like(k_pad)
        k_pad[:, :n], v_pad[:, :n] = k_n, v_n
        ref = orc.sparse_attn(q, k_pad, v_pad, w.cpu(), idx.cpu(), chunk_size=S)
        assert_close_bf16(o, ref, f"step {t} remote branch")
        lim = (n - 1 - W + 1) // S
        assert int(idx.max().item()) < max(lim, 1) and (idx >= 0).sum().item() == B * H * min(K, max(lim, 0))


def test_offloaded_cache_reads_host_memory_in_place(pkg, dev):
    """Past the offload point K and V live in pinned host memory and the kernels read the selected
    chunks and the local window from there: every step must equal the layer that keeps them on the
    GPU bit for bit (same kernels, same bytes).  Thresholds as the reference's, lowered for the test
    (utils/hils_cache_utils.py:4-5)."""
    import hils_attention_amd.utils.hils_cache_utils as cu
    note("HiLSDynamicLayer: offload at 200 tokens (pinned host K/V read in place) vs GPU-resident")
    B, HQ, H, D, S, K, W = 2, 8, 2, 64, 64, 4, 64
    gen = torch.Generator().manual_seed(6)
    L0, steps = 150, 120
    k_all = torch.randn(B, L0 + steps, H, D, generator=gen).bfloat16().to(dev)
    v_all = torch.randn(B, L0 + steps, H, D, generator=gen).bfloat16().to(dev)
    old = (cu._OFFLOAD_SEQ_THRESHOLD, cu._OFFLOAD_HIDDEN_DIM_THRESHOLD)
    cu._OFFLOAD_SEQ_THRESHOLD, cu._OFFLOAD_HIDDEN_DIM_THRESHOLD = 200, H * D
    try:
        host = pkg.HiLSDynamicLayer(chunk_size=S, capacity=128)
        gpu = pkg.HiLSDynamicLayer(chunk_size=S, capacity=128, offload=False)
        host.update(k_all[:, :L0], v_all[:, :L0])
        gpu.update(k_all[:, :L0], v_all[:, :L0])
        assert not host._offloading and host.keys.is_cuda
        for t in range(L0, L0 + steps):
            kh, vh = host.update(k_all[:, t:t + 1], v_all[:, t:t + 1])
            kg, vg = gpu.update(k_all[:, t:t + 1], v_all[:, t:t + 1])
            n = t + 1
            assert host._offloading == (n > 200)
            if host._offloading:
                assert kh.is_pinned() and vh.is_pinned() and not kh.is_cuda and host.lmk_k.is_cuda
            assert torch.equal(kh.to(dev), kg) and torch.equal(vh.to(dev), vg)
            assert torch.equal(host.lmk_k[:, : n // S], gpu.lmk_k[:, : n // S])
            if t % 17 and t not in (200, 201, 255, 256):
                continue
            q = torch.randn(B, 1, HQ, D, generator=gen).bfloat16().to(dev)
            # the local branch over the last window, read from wherever the cache lives
            lo = max(0, n - 2 * S)
            swa_h, lse_h = pkg.flex_attn_tl(q, kh[:, lo:], vh[:, lo:], window_size=W, chunk_size=S, training=False, kv_start=lo)
            swa_g, lse_g = pkg.flex_attn_tl(q, kg[:, lo:], vg[:, lo:], window_size=W, chunk_size=S, training=False, kv_start=lo)
            assert torch.equal(swa_h, swa_g) and torch.equal(lse_h, lse_g)
            oh, wh, ih = host.hils_attend(q, lse_h, K, W)
            og, wg, ig = gpu.hils_attend(q, lse_g, K, W)
            assert torch.equal(ih, ig) and torch.equal(wh, wg) and torch.equal(oh, og), f"step {t}"
        # a forced choice overrides the thresholds
        forced = pkg.HiLSDynamicLayer(chunk_size=S, offload=True)
        kf, _ = forced.update(k_all[:, :70], v_all[:, :70])
        assert kf.is_pinned() and torch.equal(forced.lmk_k[:, :1], gpu.lmk_k[:, :1])
    finally:
        cu._OFFLOAD_SEQ_THRESHOLD, cu._OFFLOAD_HIDDEN_DIM_THRESHOLD = old
