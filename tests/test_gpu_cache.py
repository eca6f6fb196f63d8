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
