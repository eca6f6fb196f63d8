"""The headline configurations at their full sizes (32K prefill, 128K decode), checked through
properties that do not need a full-size CPU run: index invariants over every row, the selection
rule and the attention output against the oracle on sampled queries, linearity in the weights,
independence of the slot order, the -1 convention."""
import math

import pytest
import torch

from util import assert_close_bf16, note

pytestmark = pytest.mark.gpu


def _index_invariants(idx, lim, K):
    """ascending, -1 padded at the end, below the causal limit, min(K, limit) entries."""
    ic = idx.long()
    valid = ic >= 0
    big = torch.where(valid, ic, torch.full_like(ic, 1 << 30))
    assert torch.all(big[..., 1:] >= big[..., :-1])
    assert torch.all((big[..., 1:] > big[..., :-1]) | ~valid[..., 1:])
    limv = lim.clamp_min(0).view(1, -1, 1, 1)
    assert torch.all(~valid | (ic < limv))
    assert torch.equal(valid.sum(-1), limv.clamp_max(K).expand(idx.shape[0], -1, idx.shape[2], 1).squeeze(-1))


def test_prefill_32k_properties(pkg, orc, dev):
    note("full size: prefill B1 L32768 hq32/hkv8 D128 top32")
    B, L, HQ, H, D, S, K, W = 1, 32768, 32, 8, 128, 64, 32, 1
    G, N = HQ // H, L // S
    gen = torch.Generator(device=dev).manual_seed(1003)
    q = torch.randn(B, L, HQ, D, device=dev, generator=gen).bfloat16()
    k = torch.randn(B, L, H, D, device=dev, generator=gen).bfloat16()
    v = torch.randn(B, L, H, D, device=dev, generator=gen).bfloat16()
    lse_swa = torch.randn(B, L, HQ, device=dev, generator=gen) * 2 + 6
    lmk = pkg.chunk_mean_pool(k, S)
    # mean pool: closed form on every chunk
    ref_lmk = k.view(B, N, S, H, D).float().mean(2)
    assert (lmk.float() - ref_lmk).abs().max().item() <= 8e-3
    # ---- top-k: invariants on all 262144 rows, the selection rule on sampled rows ----
    dbg = {}
    idx, scores = pkg.online_softmax_topk_head(q, lmk, lse_swa, K, S, W, is_training=False, _debug=dbg)
    torch.cuda.synchronize()
    lim = torch.div(torch.arange(L, device=dev) - W + 1, S, rounding_mode="floor")
    _index_invariants(idx, lim, K)
    idx_plain, scores_plain = pkg.online_softmax_topk_head(q, lmk, lse_swa, K, S, W, is_training=False)
    assert torch.equal(idx, idx_plain) and torch.equal(scores, scores_plain)  # both kernel variants agree
    ts = torch.randint(0, L, (192,), generator=torch.Generator().manual_seed(1)).sort().values
    ts[-1] = L - 1
    sel = dbg["sel_logits"][:, ts.to(dev)].cpu()
    lt = dbg["lse_total"][:, ts.to(dev)].cpu()
    want = orc.topk_select(sel, lt, lim.cpu()[ts], K)
    assert torch.equal(idx[:, ts.to(dev)].cpu(), want), "selection differs from the rule on the kernel's own logits"
    raw = torch.einsum("blhgd,bnhd->blhgn", q[:, ts.to(dev)].view(B, -1, H, G, D).float(), lmk.float()) / math.sqrt(D)
    assert (sel - raw.cpu()).abs()[torch.isfinite(sel)].max().item() <= 2e-3
    gathered = torch.gather(raw, 4, idx[:, ts.to(dev)].clamp_min(0).long().unsqueeze(3).expand(-1, -1, -1, G, -1))
    got = scores[:, ts.to(dev)].view(B, -1, H, G, K).float()
    ok = (idx[:, ts.to(dev)] >= 0).unsqueeze(3).expand_as(got)
    assert (got - gathered)[ok].abs().max().item() <= 6e-2 and torch.all(got[~ok] == float("-inf"))
    del dbg, sel, lt
    # ---- inter-chunk softmax + sparse attention ----
    w = pkg.chunk_weights(scores, lse_swa)
    assert (w.float().sum(-1) - 1).abs().max().item() < 2e-2
    o = pkg.HiLS_block_M_head(q, k, v, w, idx, block_size=S, is_training=False)
    tq = torch.tensor([0, 63, 64, 65, 127, 128, 129, 1000, 4095, 4096, 20000, L - 1])
    tq = torch.cat([tq, torch.randint(0, L, (20,), generator=torch.Generator().manual_seed(2))])
    ref = orc.sparse_attn(q[:, tq.to(dev)].cpu(), k.cpu(), v.cpu(), w[:, tq.to(dev)].cpu(), idx[:, tq.to(dev)].cpu(),
                          chunk_size=S)
    assert_close_bf16(o[:, tq.to(dev)], ref, "attention on sampled queries")
    assert torch.count_nonzero(o[:, :64]).item() == 0  # no remote chunk yet: the branch contributes nothing
    # slot order does not matter (integer accumulation): bit-identical output
    perm = torch.randperm(K, generator=torch.Generator().manual_seed(3)).to(dev)
    w_p = torch.cat([w[..., :K][..., perm], w[..., K:]], -1).contiguous()
    o_p = pkg.HiLS_block_M_head(q, k, v, w_p, idx[..., perm].contiguous(), block_size=S, is_training=False)
    assert torch.equal(o_p, o)
    # linear in the weights; a slot with index -1 is the same as a slot with weight 0
    half = (w.float() * 0.5).bfloat16()
    o_h = pkg.HiLS_block_M_head(q, k, v, half, idx, block_size=S, is_training=False)
    assert (o_h.float() * 2 - o.float()).abs().max().item() <= 3e-2
    drop = torch.rand(idx.shape, device=dev, generator=gen) < 0.3
    w_zero = torch.where(drop.repeat_interleave(G, 2), torch.zeros_like(w[..., :K]), w[..., :K])
    o_a = pkg.HiLS_block_M_head(q, k, v, torch.cat([w_zero, w[..., K:]], -1).contiguous(), idx, block_size=S,
                                is_training=False)
    o_b = pkg.HiLS_block_M_head(q, k, v, w, torch.where(drop, torch.full_like(idx, -1), idx), block_size=S,
                                is_training=False)
    assert (o_a.float() - o_b.float()).abs().max().item() <= 1e-2


def test_decode_128k_properties(pkg, orc, dev):
    note("full size: decode B32 Lkv131072 hq32/hkv8 D128 top32")
    B, Lkv, HQ, H, D, S, K, W = 32, 131072, 32, 8, 128, 64, 32, 1
    G, N = HQ // H, Lkv // S
    gen = torch.Generator(device=dev).manual_seed(1004)
    q = torch.randn(B, 1, HQ, D, device=dev, generator=gen).bfloat16()
    kc = torch.empty(B, Lkv, H, D, dtype=torch.bfloat16, device=dev).normal_(generator=gen)
    vc = torch.empty(B, Lkv, H, D, dtype=torch.bfloat16, device=dev).normal_(generator=gen)
    lse_swa = torch.randn(B, 1, HQ, device=dev, generator=gen) * 5 + 10
    lmk = pkg.chunk_mean_pool(kc, S)
    dbg = {}
    idx, scores = pkg.online_softmax_topk_head(q, lmk, lse_swa, K, S, W, q_offset=Lkv - 1, is_training=False,
                                               _debug=dbg)
    lim = torch.tensor([(Lkv - 1 - W + 1) // S], device=dev)
    _index_invariants(idx, lim, K)
    want = orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim.cpu(), K)
    assert torch.equal(idx.cpu(), want), "decode selection differs from the rule on the kernel's own logits"
    raw = torch.einsum("blhgd,bnhd->blhgn", q.view(B, 1, H, G, D).float(), lmk.float()) / math.sqrt(D)
    assert (dbg["sel_logits"] - raw).abs()[:, :, :, :, : int(lim.item())].max().item() <= 2e-3
    idx2, scores2, w = pkg.topk_chunk_weights(q, lmk, lse_swa, K, S, W, q_offset=Lkv - 1)
    assert torch.equal(idx2, idx) and torch.equal(scores2, scores)
    w_ref = orc.inter_chunk_softmax(scores.cpu(), lse_swa.cpu())
    assert (w.float().cpu() - w_ref).abs().max().item() <= 4e-3
    o = pkg.HiLS_block_M_head(q, kc, vc, w, idx, block_size=S, is_training=False)
    bs = [0, 7, 31]  # the oracle on three batch elements (their whole cache on the CPU)
    for b in bs:
        ref = orc.sparse_attn(q[b:b + 1].cpu(), kc[b:b + 1].cpu(), vc[b:b + 1].cpu(), w[b:b + 1].cpu(),
                              idx[b:b + 1].cpu(), chunk_size=S)
        assert_close_bf16(o[b:b + 1], ref, f"decode attention, batch element {b}")
    # -1 slots and zero weights agree; slot order does not matter
    drop = torch.rand(idx.shape, device=dev, generator=gen) < 0.3
    w_zero = torch.where(drop.repeat_interleave(G, 2), torch.zeros_like(w[..., :K]), w[..., :K])
    o_a = pkg.HiLS_block_M_head(q, kc, vc, torch.cat([w_zero, w[..., K:]], -1).contiguous(), idx, block_size=S,
                                is_training=False)
    o_b = pkg.HiLS_block_M_head(q, kc, vc, w, torch.where(drop, torch.full_like(idx, -1), idx), block_size=S,
                                is_training=False)
    assert (o_a.float() - o_b.float()).abs().max().item() <= 1e-2
    perm = torch.randperm(K, generator=torch.Generator().manual_seed(3)).to(dev)
    w_p = torch.cat([w[..., :K][..., perm], w[..., K:]], -1).contiguous()
    o_p = pkg.HiLS_block_M_head(q, kc, vc, w_p, idx[..., perm].contiguous(), block_size=S, is_training=False)
    assert (o_p.float() - o.float()).abs().max().item() <= 1e-2
