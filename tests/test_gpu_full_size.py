"""The headline configurations at their full sizes (32K prefill, 128K decode), checked through
properties that do not need a full-size CPU run: index invariants over every row, the selection
rule and the attention output against the oracle on sampled queries, linearity in the weights,
independence of the slot order, the -1 convention."""
import math

import pytest
import torch

import util
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


@pytest.mark.parametrize("recipe", ["plain", "bench"])
def test_prefill_32k_properties(pkg, orc, dev, recipe):
    """``plain``: N(0,1) inputs and a random lse_swa.  ``bench``: the benchmark's own inputs
    (per-head scale U[0.5,2] on q and k, which makes the chunk scores peaked, and the exact
    lse of the query's own chunk in bf16), so the figures bench.py prints are on checked data."""
    note(f"full size: prefill B1 L32768 hq32/hkv8 D128 top32, {recipe} inputs")
    B, L, HQ, H, D, S, K, W = 1, 32768, 32, 8, 128, 64, 32, 1
    G, N = HQ // H, L // S
    gen = torch.Generator(device=dev).manual_seed(1003)
    if recipe == "plain":
        q = torch.randn(B, L, HQ, D, device=dev, generator=gen).bfloat16()
        k = torch.randn(B, L, H, D, device=dev, generator=gen).bfloat16()
        v = torch.randn(B, L, H, D, device=dev, generator=gen).bfloat16()
        lse_swa = torch.randn(B, L, HQ, device=dev, generator=gen) * 2 + 6
    else:
        q, k, v, lse_swa = util.prefill_inputs(dev)
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
    # fp32 products of bf16 inputs summed in another order: a few ulp of the largest logit
    assert (sel - raw.cpu()).abs()[torch.isfinite(sel)].max().item() <= 2e-3 * max(1.0, raw.abs().max().item() / 8)
    gathered = torch.gather(raw, 4, idx[:, ts.to(dev)].clamp_min(0).long().unsqueeze(3).expand(-1, -1, -1, G, -1))
    got = scores[:, ts.to(dev)].view(B, -1, H, G, K).float()
    ok = (idx[:, ts.to(dev)] >= 0).unsqueeze(3).expand_as(got)
    bar = 6e-2 * max(1.0, gathered.abs().max().item() / 8)  # one bf16 step of the largest score
    assert (got - gathered)[ok].abs().max().item() <= bar and torch.all(got[~ok] == float("-inf"))
    del dbg, sel, lt
    # ---- inter-chunk softmax + sparse attention ----
    w = pkg.chunk_weights(scores, lse_swa)
    assert (w.float().sum(-1) - 1).abs().max().item() < 2e-2
    # the call the benchmark times (selection + weights in one call; with the benchmark's inputs lse_swa
    # is bf16 and the launches are the variants that read it as bf16): same indices, scores and weights
    idx_f, scores_f, w_f = pkg.topk_chunk_weights(q, lmk, lse_swa, K, S, W)
    assert torch.equal(idx_f, idx) and torch.equal(scores_f, scores)
    assert torch.equal(w_f, w), "fused weights differ from chunk_weights on the same scores"
    del idx_f, scores_f, w_f
    o = pkg.HiLS_block_M_head(q, k, v, w, idx, block_size=S, is_training=False)
    tq = torch.tensor([0, 63, 64, 65, 127, 128, 129, 1000, 4095, 4096, 20000, L - 1])
    tq = torch.cat([tq, torch.randint(0, L, (20,), generator=torch.Generator().manual_seed(2))])
    # rows whose remote weights are the smallest of the sequence (the output tile of a query block
    # is accumulated as fixed point scaled from the block's LARGEST weight sum)
    mass = w[0, 2048:, :, :K].float().sum(-1).amax(-1)
    low = torch.topk(mass, 12, largest=False).indices.cpu() + 2048
    tq = torch.cat([tq, low])
    ref = orc.sparse_attn(q[:, tq.to(dev)].cpu(), k.cpu(), v.cpu(), w[:, tq.to(dev)].cpu(), idx[:, tq.to(dev)].cpu(),
                          chunk_size=S)
    assert_close_bf16(o[:, tq.to(dev)], ref, "attention on sampled queries")
    got_low, ref_low = o[0, low.to(dev)].float().cpu(), ref[0, -12:]
    rel_low = ((got_low - ref_low).norm(dim=-1) / ref_low.norm(dim=-1).clamp_min(1e-30)).max().item()
    note(f"    lowest remote weight sums {mass[low - 2048].min().item():.3e}..{mass[low - 2048].max().item():.3e}: "
         f"worst per-row relative L2 error {rel_low:.3e}")
    assert rel_low <= 2e-2, "low-weight rows lose relative accuracy"
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
    del o_a, o_b, o_p, w_p, w_zero, drop
    # ---- the one-launch step (what the benchmark's decode figure times) on the same cache ----
    dbg1 = {}
    o1, w1, idx1, sc1 = pkg.decode_step(q, lmk, kc, vc, lse_swa, K, S, W, q_offset=Lkv - 1, _debug=dbg1)
    assert dbg1, "the one-launch kernel did not take the headline shape"
    want1 = orc.topk_select(dbg1["sel_logits"].cpu(), dbg1["lse_total"].cpu(), lim.cpu(), K)
    assert torch.equal(idx1.cpu(), want1), "one-launch selection differs from the rule on its own logits"
    assert torch.equal(idx1, idx) and torch.equal(sc1, scores) and torch.equal(w1, w)
    assert_close_bf16(o1, o.float(), "one launch vs two calls")
    for b in bs:
        ref = orc.sparse_attn(q[b:b + 1].cpu(), kc[b:b + 1].cpu(), vc[b:b + 1].cpu(), w1[b:b + 1].cpu(),
                              idx1[b:b + 1].cpu(), chunk_size=S)
        assert_close_bf16(o1[b:b + 1], ref, f"one-launch decode, batch element {b}")
    # chunk keys head-major (the layout this package's cache layers keep): other addresses, same arithmetic
    lmk_hm = pkg.head_major_chunk_keys(lmk)
    o2, w2, idx2, sc2 = pkg.decode_step(q, lmk_hm, kc, vc, lse_swa, K, S, W, q_offset=Lkv - 1, lmk_head_major=True)
    assert torch.equal(idx2, idx1) and torch.equal(sc2, sc1) and torch.equal(w2, w1) and torch.equal(o2, o1)
    del o2, w2, idx2, sc2, dbg1
    # ---- the same cache in pages handed out in random order ----
    num_pages = B * N + 7
    perm = torch.randperm(num_pages, device=dev, generator=gen)[: B * N].view(B, N)
    k_pages = torch.empty(num_pages, H, S, D, dtype=torch.bfloat16, device=dev).normal_(generator=gen)
    v_pages = torch.empty(num_pages, H, S, D, dtype=torch.bfloat16, device=dev).normal_(generator=gen)
    lmk_pages = torch.empty(num_pages, H, D, dtype=torch.bfloat16, device=dev).normal_(generator=gen)
    k_pages[perm] = kc.view(B, N, S, H, D).permute(0, 1, 3, 2, 4)
    v_pages[perm] = vc.view(B, N, S, H, D).permute(0, 1, 3, 2, 4)
    lmk_pages[perm] = lmk
    table = torch.full((B, N + 3), -1, dtype=torch.int32, device=dev)
    table[:, :N] = perm.to(torch.int32)
    dbgp = {}
    o3, w3, idx3 = pkg.paged_hils_attend(q, k_pages, v_pages, lmk_pages, table, lse_swa, Lkv, K, W, _debug=dbgp)
    wantp = orc.topk_select(dbgp["sel_logits"].cpu(), dbgp["lse_total"].cpu(), lim.cpu(), K)
    assert torch.equal(idx3.cpu(), wantp), "paged selection differs from the rule on its own logits"
    assert torch.equal(idx3, idx1) and torch.equal(dbgp["scores"], sc1) and torch.equal(w3, w1)
    assert torch.equal(o3, o1), "paged output differs from the token-major cache's"
    o4, w4, idx4 = pkg.paged_hils_attend(q, k_pages, v_pages, None, table, lse_swa, Lkv, K, W, lmk_dense=lmk_hm)
    assert torch.equal(idx4, idx1) and torch.equal(w4, w1) and torch.equal(o4, o1)


def _sampled_queries(L, n, seed):
    tq = torch.tensor([0, 63, 64, 65, 127, 128, 129, 1000, 4095, 4096, L - 1])
    return torch.cat([tq, torch.randint(0, L, (n,), generator=torch.Generator().manual_seed(seed))])


def test_prefill_config2_properties(pkg, orc, dev):
    """Config 2 (345M-shaped prefill forward, B4 L8192, 16 heads MHA, D64, top-32) on the
    benchmark's inputs: index invariants on every row, the selection rule and the scores on
    sampled rows, the inter-chunk softmax and the attention output against the oracle on sampled
    queries of every batch element."""
    note("full size: prefill B4 L8192 h16/16 D64 top32 (config 2)")
    B, L, HQ, H, D, S, K, W = 4, 8192, 16, 16, 64, 64, 32, 1
    G, N = 1, L // S
    q, k, v, lse_swa = util.config2_inputs(dev)
    lmk = pkg.chunk_mean_pool(k, S)
    assert (lmk.float() - k.view(B, N, S, H, D).float().mean(2)).abs().max().item() <= 8e-3
    dbg = {}
    idx, scores = pkg.online_softmax_topk_head(q, lmk, lse_swa, K, S, W, is_training=False, _debug=dbg)
    lim = torch.div(torch.arange(L, device=dev) - W + 1, S, rounding_mode="floor")
    _index_invariants(idx, lim, K)
    idx2, scores2, w = pkg.topk_chunk_weights(q, lmk, lse_swa, K, S, W)   # what the bench step calls
    assert torch.equal(idx2, idx) and torch.equal(scores2, scores)
    ts = _sampled_queries(L, 150, 11).sort().values
    tsd = ts.to(dev)
    sel, lt = dbg["sel_logits"][:, tsd].cpu(), dbg["lse_total"][:, tsd].cpu()
    assert torch.equal(idx[:, tsd].cpu(), orc.topk_select(sel, lt, lim.cpu()[ts], K)), \
        "selection differs from the rule on the kernel's own logits"
    raw = torch.einsum("blhgd,bnhd->blhgn", q[:, tsd].view(B, -1, H, G, D).float(), lmk.float()) / math.sqrt(D)
    assert (sel - raw.cpu()).abs()[torch.isfinite(sel)].max().item() <= 2e-3
    # lse_total = logaddexp(lse_swa, logsumexp of the visible logits)
    vis = torch.arange(N).view(1, 1, 1, 1, N) < lim.cpu()[ts].view(1, -1, 1, 1, 1)
    lt_ref = torch.logaddexp(lse_swa[:, tsd].float().cpu().view(B, -1, H, G),
                             torch.logsumexp(raw.cpu().masked_fill(~vis, float("-inf")), -1))
    assert (lt - lt_ref).abs().max().item() <= 1e-4 * max(1.0, lt_ref.abs().max().item())
    gathered = torch.gather(raw, 4, idx[:, tsd].clamp_min(0).long().unsqueeze(3))
    got = scores[:, tsd].view(B, -1, H, G, K).float()
    ok = (idx[:, tsd] >= 0).unsqueeze(3)
    assert (got - gathered)[ok].abs().max().item() <= 6e-2 and torch.all(got[~ok.expand_as(got)] == float("-inf"))
    del dbg, sel, lt
    w_ref = orc.inter_chunk_softmax(scores[:, tsd].cpu(), lse_swa[:, tsd].cpu())
    assert (w[:, tsd].float().cpu() - w_ref).abs().max().item() <= 4e-3
    ws = pkg.prepare_kv_workspace(L, k, v, HQ, K, S)
    o = pkg.HiLS_block_M_head(q, k, v, w, idx, block_size=S, is_training=False, kv_workspace=ws)
    tq = _sampled_queries(L, 40, 12)
    tqd = tq.to(dev)
    ref = orc.sparse_attn(q[:, tqd].cpu(), k.cpu(), v.cpu(), w[:, tqd].cpu(), idx[:, tqd].cpu(), chunk_size=S)
    assert_close_bf16(o[:, tqd], ref, "config 2 attention on sampled queries")
    assert torch.count_nonzero(o[:, :64]).item() == 0
    o_nows = pkg.HiLS_block_M_head(q, k, v, w, idx, block_size=S, is_training=False)
    assert torch.equal(o_nows, o), "packing K/V inside the call or ahead of it must not change the output"


def test_train_config5_forward_backward(pkg, orc, dev):
    """Config 5 (345M-shaped training layer, B8 L8192, 16 heads MHA, D64, top-32), the step
    bench.py times: mean pool -> top-k scores -> softmax over [scores, lse_swa] -> sparse
    attention, backward through every operator.

    * forward: index invariants on every row, output against the oracle on sampled queries;
    * the attention operator's backward on its own (dQ, dK, dV, dW) against the oracle's autograd
      on one batch element and two heads: every query of those heads goes through the oracle, so
      dK / dV of every chunk are complete sums, including the early chunks that thousands of
      queries select (their rows are also reported and checked on their own);
    * the gradients of the whole step (through the score gather, the softmax and the pooling)
      against the oracle's autograd of the same chain on the kernel's indices, same slice."""
    note("full size: train layer fwd+bwd B8 L8192 h16/16 D64 top32 (config 5)")
    B, L, HQ, H, D, S, K, W = 8, 8192, 16, 16, 64, 64, 32, 1
    N = L // S
    q, k, v, d_o, lse_swa = util.train_inputs(dev)
    o, idx, scores, w = util.train_forward(pkg, q, k, v, lse_swa, keep=True)
    o.backward(d_o)
    torch.cuda.synchronize()
    lim = torch.div(torch.arange(L, device=dev) - W + 1, S, rounding_mode="floor")
    _index_invariants(idx, lim, K)
    tq = _sampled_queries(L, 24, 21)
    tqd = tq.to(dev)
    ref = orc.sparse_attn(q[:, tqd].detach().cpu(), k.detach().cpu(), v.detach().cpu(), w[:, tqd].detach().cpu(),
                          idx[:, tqd].cpu(), chunk_size=S)
    assert_close_bf16(o[:, tqd], ref, "config 5 attention forward on sampled queries")

    # ---- the attention operator's backward in isolation ----
    b0, h0, nh = 3, 5, 2
    ql, kl, vl, wl = (t.detach().clone().requires_grad_() for t in (q, k, v, w))
    pkg.HiLS_block_M_head(ql, kl, vl, wl, idx, block_size=S, is_training=True).backward(d_o)
    torch.cuda.synchronize()
    hs = slice(h0, h0 + nh)

    def cpu_slice(t):
        return t[b0:b0 + 1, :, hs].detach().float().cpu()

    idx_s = idx[b0:b0 + 1, :, hs].cpu()
    do_s = cpu_slice(d_o)
    qf, kf, vf, wf = (cpu_slice(t).requires_grad_() for t in (q, k, v, w))
    for t0 in range(0, L, 1024):   # query blocks: dK / dV accumulate in the leaves' .grad
        sl = slice(t0, t0 + 1024)
        orc.sparse_attn(qf[:, sl], kf, vf, wf[:, sl], idx_s[:, sl], chunk_size=S).backward(do_s[:, sl])
    assert_close_bf16(ql.grad[b0:b0 + 1, :, hs], qf.grad, "attention dq (1 batch element, 2 heads, all queries)")
    assert_close_bf16(kl.grad[b0:b0 + 1, :, hs], kf.grad, "attention dk")
    assert_close_bf16(vl.grad[b0:b0 + 1, :, hs], vf.grad, "attention dv")
    valid = idx_s >= 0
    dw_ref = torch.zeros_like(wf.grad)
    dw_ref[..., :K] = torch.where(valid, wf.grad[..., :K], torch.zeros(()))
    assert_close_bf16(wl.grad[b0:b0 + 1, :, hs], dw_ref, "attention dw")
    # the chunks selected by the most queries
    counts = torch.zeros(nh, N + 1, dtype=torch.long)
    for j in range(nh):
        counts[j] = torch.bincount(idx_s[0, :, j].flatten().long() + 1, minlength=N + 1)
    counts = counts[:, 1:]
    for j in range(nh):
        hot = torch.topk(counts[j], 4).indices
        note(f"    head {h0 + j}: hottest chunks {hot.tolist()} selected by {counts[j][hot].tolist()} queries")
        assert counts[j][hot].min().item() >= 1000
        for c in hot.tolist():
            rows = slice(c * S, (c + 1) * S)
            assert_close_bf16(kl.grad[b0, rows, h0 + j], kf.grad[0, rows, j], f"dk of hot chunk {c}")
            assert_close_bf16(vl.grad[b0, rows, h0 + j], vf.grad[0, rows, j], f"dv of hot chunk {c}")
    del ql, kl, vl, wl

    # ---- the whole step's gradients ----
    lse_s = cpu_slice(lse_swa)
    qf, kf, vf = (cpu_slice(t).requires_grad_() for t in (q, k, v))
    for t0 in range(0, L, 1024):
        sl = slice(t0, t0 + 1024)
        lmk = orc.mean_pool(kf, S)
        logits = orc.topk_logits(qf[:, sl].view(1, 1024, nh, 1, D), lmk)          # (1,T,nh,1,N)
        sc = torch.gather(logits, 4, idx_s[:, sl].clamp_min(0).long().unsqueeze(3))
        sc = sc.masked_fill((idx_s[:, sl] < 0).unsqueeze(3), float("-inf")).view(1, 1024, nh, K)
        w_o = orc.inter_chunk_softmax(sc, lse_s[:, sl])
        orc.sparse_attn(qf[:, sl], kf, vf, w_o, idx_s[:, sl], chunk_size=S).backward(do_s[:, sl])
    assert_close_bf16(q.grad[b0:b0 + 1, :, hs], qf.grad, "step dq")
    assert_close_bf16(k.grad[b0:b0 + 1, :, hs], kf.grad, "step dk")
    assert_close_bf16(v.grad[b0:b0 + 1, :, hs], vf.grad, "step dv")
