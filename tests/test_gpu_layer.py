"""Whole HiLS layer forward (config 1: B1 L2048 h4/4 D64 chunk 64 top-8, causal) on the GPU
vs the CPU oracle: mean-pooled chunk keys -> top-k -> inter-chunk softmax -> sparse attention."""
import pytest
import torch

from util import assert_close_bf16, note

pytestmark = pytest.mark.gpu


def test_config1_layer_forward(pkg, orc, dev):
    note("config 1 layer forward")
    B, L, HQ, H, D, S, K, W = 1, 2048, 4, 4, 64, 64, 8, 1
    gen = torch.Generator().manual_seed(1001)
    q = torch.randn(B, L, HQ, D, generator=gen).bfloat16()
    k = torch.randn(B, L, H, D, generator=gen).bfloat16()
    v = torch.randn(B, L, H, D, generator=gen).bfloat16()
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    lmk = pkg.chunk_mean_pool(kd, S)
    ref = orc.hils_layer_forward(q.float(), k.float(), v.float(), chunk_size=S, topk=K, window_size=W,
                                 lmk_k=lmk.float().cpu())
    dbg = {}
    lse_swa = ref["lse_swa"].bfloat16()  # the layer hands lse_swa over in bf16
    ref = orc.hils_layer_forward(q.float(), k.float(), v.float(), chunk_size=S, topk=K, window_size=W,
                                 lmk_k=lmk.float().cpu())
    idx, scores = pkg.online_softmax_topk_head(qd, lmk, lse_swa.to(dev), K, S, W, _debug=dbg)
    lim = orc.causal_chunk_limit(L, 0, W, S)
    sel_idx = orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim, K)
    assert torch.equal(idx.cpu(), sel_idx), "indices not bit-exact from identical fp32 scores"
    w = orc.inter_chunk_softmax(scores.float().cpu(), lse_swa.float()).bfloat16()
    o_sparse = pkg.HiLS_block_M_head(qd, kd, vd, w.to(dev), idx, block_size=S, is_training=False)
    o = torch.addcmul(o_sparse.float().cpu(), ref["swa_o"].bfloat16().float(), w[..., K].float().unsqueeze(-1))
    # oracle on the kernel's own indices (near-tie flips against the fp32 oracle are allowed
    # to differ, everything downstream of the indices must agree)
    o_ref = orc.sparse_attn(q, k, v, w, idx.cpu(), chunk_size=S) + ref["swa_o"] * w[..., K].float().unsqueeze(-1)
    assert_close_bf16(o, o_ref, "layer output")
    agree = (idx.cpu() == ref["indices"]).float().mean().item()
    assert agree > 0.97, f"index agreement with the fp32 oracle {agree:.4f}"


def test_chunk_weights_kernel(pkg, orc, dev):
    """Fused inter-chunk softmax against the layer's torch glue restated in the oracle."""
    note("chunk_weights")
    torch.manual_seed(3)
    for K in (16, 32, 12):
        _chunk_weights_case(pkg, orc, dev, K)
    # long rows of queries: the backward's workgroups walk several tiles and add the bias gradients in LDS
    _chunk_weights_case(pkg, orc, dev, 32, dims=(3, 5000, 16, 2, 79))
    _chunk_weights_case(pkg, orc, dev, 8, dims=(1, 9001, 6, 3, 141))


def _chunk_weights_case(pkg, orc, dev, K, dims=(2, 301, 8, 2, 40)):
    B, L, HQ, H, N = dims
    scores = torch.randn(B, L, HQ, K).bfloat16()
    scores[:, :5, :, 7:] = float("-inf")
    lse = torch.randn(B, L, HQ).bfloat16()
    idx = torch.randint(-1, N, (B, L, H, K), dtype=torch.int32)
    pb = torch.randn(B, N, HQ)
    for prior, s1 in ((False, False), (True, False), (False, True), (True, True)):
        w = pkg.chunk_weights(scores.to(dev), lse.to(dev), pb.to(dev) if prior else None,
                              idx.to(dev) if prior else None, enable_softmax1=s1)
        ref = orc.inter_chunk_softmax(scores, lse, pb.bfloat16() if prior else None, idx if prior else None,
                                      softmax1=s1)
        assert w.dtype == torch.bfloat16 and w.shape == ref.shape
        assert_close_bf16(w, ref, f"chunk_weights prior={prior} softmax1={s1}", max_abs=8e-3)
    w32 = pkg.chunk_weights(scores.to(dev), lse.float().to(dev))
    assert torch.equal(w32, pkg.chunk_weights(scores.to(dev), lse.to(dev)))
    # backward: gradients of scores, lse_swa and prior_b against the oracle's autograd
    for prior, s1 in ((False, False), (True, True)):
        sc_d = scores.to(dev).requires_grad_()
        lse_d = lse.float().to(dev).requires_grad_()
        pb_d = pb.to(dev).requires_grad_() if prior else None
        w = pkg.chunk_weights(sc_d, lse_d, pb_d, idx.to(dev) if prior else None, enable_softmax1=s1)
        g = torch.randn(w.shape).bfloat16()
        w.backward(g.to(dev))
        sc_c = scores.float().requires_grad_()
        lse_c = lse.float().requires_grad_()
        pb_c = pb.bfloat16().float().requires_grad_() if prior else None
        ref = orc.inter_chunk_softmax(sc_c, lse_c, pb_c, idx if prior else None, softmax1=s1)
        ref.backward(g.float())
        assert sc_d.grad.dtype == torch.bfloat16 and lse_d.grad.dtype == torch.float32
        assert_close_bf16(sc_d.grad, sc_c.grad, f"d_scores prior={prior} softmax1={s1}", max_abs=8e-3)
        assert_close_bf16(lse_d.grad, lse_c.grad, "d_lse_swa", max_abs=8e-3)
        if prior:
            # empty slots gather (and scatter to) chunk 0 on both sides, as torch.gather on the clamped indices does
            assert_close_bf16(pb_d.grad, pb_c.grad, "d_prior_b", max_abs=2e-2)


@pytest.mark.parametrize("B,L,N,HQ,H,D,K,off", [(32, 1, 2048, 32, 8, 128, 32, 2048 * 64 - 1),
                                                (13, 1, 500, 8, 8, 64, 16, 300 * 64),
                                                (2, 3, 700, 8, 2, 128, 8, 700 * 64 - 3),
                                                (128, 1, 256, 4, 1, 64, 8, 64 * 2 + 1),
                                                # prefill shapes: two kernels behind the one call
                                                (1, 1024, 16, 8, 2, 128, 8, 0),
                                                (2, 1000, 16, 4, 4, 64, 16, 24),
                                                # eight and five query heads per KV head, decode and prefill
                                                (64, 1, 2048, 16, 2, 64, 32, 2048 * 64 - 1),
                                                (1, 2048, 32, 16, 2, 64, 16, 0), (1, 1500, 600, 10, 2, 128, 8, 600 * 64 - 1500),
                                                (1, 2048, 32, 4, 2, 128, 32, 0),
                                                (1, 512, 8, 8, 2, 64, 12, 0),
                                                (1, 777, 40, 6, 2, 128, 32, 1800),   # three heads per KV head
                                                (2, 515, 9, 4, 1, 64, 8, 64)])
def test_topk_with_fused_weights_matches_two_calls(pkg, dev, B, L, N, HQ, H, D, K, off):
    """One call for selection + inter-chunk softmax (the selection kernel writes the weights when
    it runs one workgroup per row, else a second kernel) against the two separate operators."""
    note(f"topk+weights B{B} L{L} N{N} HQ{HQ} H{H} D{D} K{K}")
    gen = torch.Generator().manual_seed(77)
    q = torch.randn(B, L, HQ, D, generator=gen).bfloat16().to(dev)
    lmk = torch.randn(B, N, H, D, generator=gen).bfloat16().to(dev)
    lse = (torch.randn(B, L, HQ, generator=gen) * 5 + 10).to(dev)
    idx0, sc0 = pkg.online_softmax_topk_head(q, lmk, lse, K, 64, 1, q_offset=off, is_training=False)
    w0 = pkg.chunk_weights(sc0, lse)
    idx1, sc1, w1 = pkg.topk_chunk_weights(q, lmk, lse, K, 64, 1, q_offset=off)
    assert torch.equal(idx0, idx1) and torch.equal(sc0, sc1)
    assert w1.shape == w0.shape and w1.dtype == torch.bfloat16
    assert (w1.float() - w0.float()).abs().max().item() <= 4e-3  # one bf16 step at weights below 1
    assert (w1.float().sum(-1) - 1).abs().max().item() < 2e-2
    assert torch.equal(w1[..., :K] == 0, w0[..., :K] == 0)  # empty slots carry exactly zero weight
    if L > 64:  # prefill: the softmax is the same arithmetic in the same order whichever kernel runs it
        assert torch.equal(w1.view(torch.int16), w0.view(torch.int16))


@pytest.mark.parametrize("L,N,HQ,H,D,K", [(3000, 47, 8, 2, 128, 16), (9000, 300, 3, 1, 64, 32),
                                          (2048, 32, 8, 4, 64, 8), (1500, 24, 16, 1, 128, 8),
                                          (4096, 64, 16, 2, 64, 32), (3000, 47, 10, 2, 128, 16)])
def test_topk_weights_reads_bf16_lse_in_place(pkg, dev, L, N, HQ, H, D, K):
    """lse_swa in bf16, as the layer hands it over: the one-pass prefill kernel reads it in place
    (other shapes convert it first); either way the result is that of the fp32 copy of the same values."""
    note(f"topk+weights bf16 lse L{L} N{N} HQ{HQ} H{H} D{D} K{K}")
    gen = torch.Generator().manual_seed(78)
    q = torch.randn(1, L, HQ, D, generator=gen).bfloat16().to(dev)
    lmk = torch.randn(1, N, H, D, generator=gen).bfloat16().to(dev)
    lse16 = (torch.randn(1, L, HQ, generator=gen) * 5 + 10).bfloat16().to(dev)
    off = max(0, N * 64 - L)
    idx0, sc0, w0 = pkg.topk_chunk_weights(q, lmk, lse16.float(), K, 64, 1, q_offset=off)
    idx1, sc1, w1 = pkg.topk_chunk_weights(q, lmk, lse16, K, 64, 1, q_offset=off)
    assert torch.equal(idx0, idx1)
    assert torch.equal(sc0.view(torch.int16), sc1.view(torch.int16))
    assert torch.equal(w0.view(torch.int16), w1.view(torch.int16))


def test_decode_step_replays_as_hip_graph(pkg, orc, dev):
    """The decode step (selection + inter-chunk softmax, then sparse attention) captured as one HIP
    graph: every replay, with eager work and synchronisations in between and with new inputs
    copied into the captured buffers, must reproduce the eager result bit for bit."""
    note("decode step as a HIP graph")
    B, Lkv, HQ, H, D, S, K = 32, 4096, 32, 8, 128, 64, 16
    gen = torch.Generator().manual_seed(91)
    q = torch.randn(B, 1, HQ, D, generator=gen).bfloat16().to(dev)
    kc = torch.randn(B, Lkv, H, D, generator=gen).bfloat16().to(dev)
    vc = torch.randn(B, Lkv, H, D, generator=gen).bfloat16().to(dev)
    lse = (torch.randn(B, 1, HQ, generator=gen) * 2 + 3).to(dev)
    lmk = pkg.chunk_mean_pool(kc, S)

    def step():
        idx, scores, w = pkg.topk_chunk_weights(q, lmk, lse, K, S, 1, q_offset=Lkv - 1)
        return idx, w, pkg.HiLS_block_M_head(q, kc, vc, w, idx, block_size=S, is_training=False)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_idx, g_w, g_o = step()
    for it in range(4):
        if it:
            q.copy_(torch.randn(B, 1, HQ, D, generator=gen).bfloat16())  # new query, same buffers
        e_idx, e_w, e_o = step()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_idx, e_idx), f"replay {it}: indices differ"
        assert torch.equal(g_w, e_w), f"replay {it}: weights differ"
        assert torch.equal(g_o, e_o), f"replay {it}: outputs differ"
    # and the eager result itself against the oracle
    ref = orc.sparse_attn(q.cpu(), kc.cpu(), vc.cpu(), e_w.cpu(), e_idx.cpu(), chunk_size=S)
    assert_close_bf16(e_o, ref, "decode step output")


@pytest.mark.parametrize("B,Lq,Lkv,HQ,H,D,K", [(32, 1, 32768, 32, 8, 128, 32), (16, 1, 16512, 8, 8, 64, 16),
                                               (50, 2, 20480, 4, 1, 128, 8), (24, 1, 65536, 12, 4, 64, 64),
                                               (64, 1, 32768, 16, 2, 64, 32), (20, 1, 65536, 40, 8, 128, 32),
                                               # not taken by the one-launch kernel (few rows): the two calls
                                               (2, 1, 4096, 8, 2, 128, 16)])
def test_decode_step_one_launch(pkg, orc, dev, B, Lq, Lkv, HQ, H, D, K):
    """decode_step (selection + inter-chunk softmax + attention of a row by one workgroup) against the
    two separate calls and against the oracle."""
    note(f"decode_step B{B} Lq{Lq} Lkv{Lkv} HQ{HQ} H{H} D{D} K{K}")
    gen = torch.Generator().manual_seed(81)
    q = torch.randn(B, Lq, HQ, D, generator=gen).bfloat16()
    k = torch.randn(B, Lkv, H, D, generator=gen).bfloat16()
    v = torch.randn(B, Lkv, H, D, generator=gen).bfloat16()
    lse = torch.randn(B, Lq, HQ, generator=gen) * 3 + 5
    qd, kd, vd, lsed = q.to(dev), k.to(dev), v.to(dev), lse.to(dev)
    N = Lkv // 64
    lmk = pkg.chunk_mean_pool(kd[:, : N * 64].contiguous(), 64)
    dbg = {}
    o1, w1, idx1, sc1 = pkg.decode_step(qd, lmk, kd, vd, lsed, K, 64, 1, q_offset=Lkv - Lq, _debug=dbg)
    idx0, sc0, w0 = pkg.topk_chunk_weights(qd, lmk, lsed, K, 64, 1, q_offset=Lkv - Lq)
    o0 = pkg.HiLS_block_M_head(qd, kd, vd, w0, idx0, block_size=64, is_training=False)
    assert torch.equal(idx1, idx0) and torch.equal(sc1, sc0) and torch.equal(w1, w0)
    assert_close_bf16(o1, o0.float(), "one launch vs two calls")
    if dbg:  # the one-launch kernel ran: selection rule on its own logits
        lim = orc.causal_chunk_limit(Lq, Lkv - Lq, 1, 64)
        want = orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim, K)
        assert torch.equal(idx1.cpu(), want)
    ref = orc.sparse_attn(q, k, v, w1.cpu(), idx1.cpu(), chunk_size=64)
    assert_close_bf16(o1, ref, "decode_step output")
    # twice the same call: bit-identical (the selection's log-sum-exp is summed in a fixed order)
    o2, w2, idx2, sc2 = pkg.decode_step(qd, lmk, kd, vd, lsed, K, 64, 1, q_offset=Lkv - Lq)
    assert torch.equal(o2, o1) and torch.equal(idx2, idx1) and torch.equal(w2, w1)


@pytest.mark.parametrize("q_pos", [10, 700, 1000, 5000])
def test_decode_step_on_a_mostly_empty_cache(pkg, orc, dev, q_pos):
    """A cache buffer far longer than the sequence (the in-place cache hands the kernels its whole
    buffers): only the chunks before the query are visible, fewer than topk of them or none at all."""
    note(f"decode_step with the query at position {q_pos} of a 32768-token buffer")
    B, Lq, Lkv, HQ, H, D, K = 12, 1, 32768, 16, 8, 128, 16
    gen = torch.Generator().manual_seed(83)
    q = torch.randn(B, Lq, HQ, D, generator=gen).bfloat16()
    k = torch.randn(B, Lkv, H, D, generator=gen).bfloat16()
    v = torch.randn(B, Lkv, H, D, generator=gen).bfloat16()
    lse = torch.randn(B, Lq, HQ, generator=gen) * 3 + 5
    qd, kd, vd, lsed = q.to(dev), k.to(dev), v.to(dev), lse.to(dev)
    lmk = pkg.chunk_mean_pool(kd, 64)
    dbg = {}
    o1, w1, idx1, sc1 = pkg.decode_step(qd, lmk, kd, vd, lsed, K, 64, 1, q_offset=q_pos, _debug=dbg)
    assert dbg, "this shape is meant to run on the one-launch kernel"
    lim = orc.causal_chunk_limit(Lq, q_pos, 1, 64)
    want = orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim, K)
    assert torch.equal(idx1.cpu(), want)
    nvis = int(lim[0])
    assert (idx1 >= 0).sum().item() == B * H * min(K, nvis) and int(idx1.max().item()) < max(nvis, 1)
    idx0, sc0, w0 = pkg.topk_chunk_weights(qd, lmk, lsed, K, 64, 1, q_offset=q_pos)
    assert torch.equal(idx1, idx0) and torch.equal(sc1, sc0) and torch.equal(w1, w0)
    ref = orc.sparse_attn(q, k, v, w1.cpu(), idx1.cpu(), chunk_size=64)
    assert_close_bf16(o1, ref, "decode_step output")
    if nvis == 0:  # nothing remote to attend to: all the weight on the local branch
        assert torch.count_nonzero(o1).item() == 0 and torch.all(w1[..., K].float() == 1.0)


@pytest.mark.parametrize("L,HQ,H,D,K,W", [(4096, 16, 2, 64, 16, 512), (2500, 32, 4, 128, 8, 512), (3000, 8, 4, 64, 8, 200)])
def test_default_mode_layer_forward_at_the_reference_head_counts(pkg, orc, dev, L, HQ, H, D, K, W):
    """The layer in the reference's default mode (models/FlashHiLS/hils_attention.py:361-416, 540-623: sliding
    window 512, attention-pooled chunk keys per query head, their entropy as prior bias of the selection and
    of the inter-chunk softmax, the local branch merged by its weight) at the head counts of its
    configurations (configs/hils_attention: 16 query / 2 KV heads of 64), every stage on the GPU, against the
    oracle's stages on the same inputs and on the kernel's own selection."""
    note(f"default-mode layer forward L{L} HQ{HQ} H{H} D{D} K{K} W{W}")
    B, S = 1, 64
    G, N = HQ // H, L // S
    gen = torch.Generator().manual_seed(1010)
    q = torch.randn(B, L, HQ, D, generator=gen).bfloat16()
    k = torch.randn(B, L, H, D, generator=gen).bfloat16()
    v = torch.randn(B, L, H, D, generator=gen).bfloat16()
    mu = torch.randn(B, N, HQ, D, generator=gen).bfloat16()  # the chunks' prior queries
    qd, kd, vd, mud = q.to(dev), k.to(dev), v.to(dev), mu.to(dev)
    # the GPU pipeline
    swa_o, lse_swa = pkg.flex_attn_tl(qd, kd, vd, W, S, training=False)
    lmk_k, lmk_b = pkg.chunk_attn_pool(mud, kd[:, : N * S].reshape(B, N, S, H, D))
    lse_h = lse_swa.bfloat16()  # the layer hands it over in its hidden dtype
    idx, sc, w = pkg.topk_chunk_weights(qd, lmk_k, lse_h, K, S, W, prior_b=lmk_b, num_kv_heads=H)
    o = pkg.HiLS_block_M_head(qd, kd, vd, w, idx, block_size=S, is_training=False, swa_o=swa_o)
    torch.cuda.synchronize()
    # the oracle's stages
    r_swa_o, r_lse = orc.swa(q, k, v, window_size=W, chunk_size=S, mask_lmk=True)
    assert_close_bf16(swa_o, r_swa_o, "local branch")
    fin = torch.isfinite(r_lse)
    assert torch.equal(torch.isfinite(lse_swa).cpu(), fin)
    assert (lse_swa.cpu() - r_lse)[fin].abs().max().item() <= 1e-3
    r_k, r_b, _ = orc.chunk_attn_pool(mu, k[:, : N * S].reshape(B, N, S, H, D).repeat_interleave(G, dim=3))
    assert_close_bf16(lmk_k, r_k, "attention-pooled chunk keys")
    assert (lmk_b.cpu() - r_b).abs().max().item() <= 1e-4
    # selection on the GPU's own chunk keys / bias / lse: agreement with the oracle's, exactness from the logits
    ridx, _, aux = orc.online_softmax_topk_head(q.view(B, L, H, G, D), lmk_k.cpu(), lse_h.float().cpu(), K, S, W,
                                                bias=lmk_b.cpu(), return_aux=True)
    assert (idx.cpu() == ridx).float().mean().item() >= 0.99
    dbg = {}
    idx_e, sc_e = pkg.online_softmax_topk_head(qd, lmk_k, lse_h.float(), K, S, W, is_training=False, bias=lmk_b, G=G,
                                               _debug=dbg)
    assert torch.equal(idx_e, idx) and torch.equal(sc_e.view(torch.int16), sc.view(torch.int16))
    lim = orc.causal_chunk_limit(L, 0, W, S)
    assert torch.equal(idx.cpu(), orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim, K))
    w_ref = orc.inter_chunk_softmax(sc.float().cpu(), lse_h.float().cpu(), lmk_b.cpu().bfloat16().float(), idx.cpu(),
                                    bf16_sum=True)
    assert_close_bf16(w, w_ref, "inter-chunk weights with the prior bias", max_abs=8e-3)
    o_ref = orc.sparse_attn(q, k, v, w.cpu(), idx.cpu(), chunk_size=S) + swa_o.float().cpu() * w[..., K].float().cpu().unsqueeze(-1)
    assert_close_bf16(o, o_ref, "layer output")
