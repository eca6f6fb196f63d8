"""The layer's default mode (``enable_prior_query``, models/FlashHiLS/hils_attention.py:361-416,
568-602) on the fast kernels: the prior bias of every chunk is the selection's additive bias and is
gathered into the inter-chunk softmax.  Prefill (one-pass selection kernel), decode (one launch per
step, token-major / head-major / paged chunk keys) and the two cache layers, against the oracle's
``online_softmax_topk_head(bias=)`` + ``inter_chunk_softmax(prior_b=)`` + ``sparse_attn``."""
import pytest
import torch

from util import assert_close_bf16, assert_close_f32, note

pytestmark = pytest.mark.gpu


def _oracle_step(orc, q, lmk, lse, pb, k, v, K, S, W, off, idx, scores_bf16):
    """Oracle outputs for the kernel's own indices and bf16 scores: weights and remote output."""
    w = orc.inter_chunk_softmax(scores_bf16.float(), lse, pb.bfloat16().float(), idx, bf16_sum=True)
    o = orc.sparse_attn(q, k, v, w.bfloat16(), idx, chunk_size=S)
    return w, o


@pytest.mark.parametrize("L,N,HQ,H,D,K,off", [(4096, 64, 8, 2, 128, 16, 0), (9000, 300, 3, 1, 64, 32, 300 * 64 - 9000),
                                             (2048, 32, 4, 4, 64, 8, 0), (6000, 500, 4, 1, 128, 32, 500 * 64 - 6000),
                                             (5000, 400, 16, 2, 64, 32, 400 * 64 - 5000), (3000, 47, 5, 1, 128, 16, 8),
                                             (5000, 400, 4, 2, 128, 32, 400 * 64 - 5000)])
def test_prefill_selection_with_prior_bias(pkg, orc, dev, L, N, HQ, H, D, K, off):
    """topk_chunk_weights(prior_b=) at prefill sizes: the one-pass selection kernel adds the bias to
    its logits, the softmax kernel gathers it.  Checked against the exporting variant of the operator
    (bit-exact selection from the exported biased logits), chunk_weights and the oracle; lse_swa in fp32
    and, as the layer hands it over, in bf16."""
    note(f"prefill selection with prior bias L{L} N{N} HQ{HQ} H{H} D{D} K{K}")
    B, S, W = 1, 64, 1
    G = HQ // H
    gen = torch.Generator().manual_seed(401)
    q = torch.randn(B, L, HQ, D, generator=gen).bfloat16()
    lmk = torch.randn(B, N, H, D, generator=gen).bfloat16()
    lse = (torch.randn(B, L, HQ, generator=gen) * 3 + 5).bfloat16().float()
    pb = torch.randn(B, N, HQ, generator=gen) * 2  # entropy-like magnitudes, both signs
    qd, lmkd, lsed, pbd = q.to(dev), lmk.to(dev), lse.to(dev), pb.to(dev)
    dbg = {}
    idx0, sc0 = pkg.online_softmax_topk_head(qd, lmkd, lsed, K, S, W, q_offset=off, is_training=False,
                                             bias=pbd, _debug=dbg)
    lim = orc.causal_chunk_limit(L, off, W, S)
    want = orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim, K)
    assert torch.equal(idx0.cpu(), want), "indices not bit-exact from the kernel's biased logits"
    ridx, rsc, aux = orc.online_softmax_topk_head(q.view(B, L, H, G, D), lmk, lse, K, S, W, q_offset=off,
                                                  bias=pb, return_aux=True)
    assert_close_f32(dbg["sel_logits"].cpu(), aux["sel_logits"], 2e-3, "biased selection logits")
    assert_close_f32(dbg["lse_total"].cpu(), aux["lse_total"], 1e-3, "lse_total")
    assert (idx0.cpu() == ridx).float().mean().item() >= 0.99
    # raw scores (no bias) at the kernel's indices
    safe = idx0.cpu().long().clamp_min(0).unsqueeze(3).expand(-1, -1, -1, G, -1)
    raw = torch.gather(aux["logits"], -1, safe).masked_fill((idx0.cpu() < 0).unsqueeze(3).expand(-1, -1, -1, G, -1),
                                                             float("-inf"))
    assert_close_bf16(sc0.view(B, L, H, G, K), raw, "scores carry no bias")
    w0 = pkg.chunk_weights(sc0, lsed, pbd, idx0)
    for lse_in in (lsed, lsed.bfloat16()):
        idx1, sc1, w1 = pkg.topk_chunk_weights(qd, lmkd, lse_in, K, S, W, q_offset=off, prior_b=pbd)
        assert torch.equal(idx1, idx0), "the inference launches and the exporting variant disagree"
        assert torch.equal(sc1.view(torch.int16), sc0.view(torch.int16))
        # (a kernel that writes the weights itself may differ from chunk_weights by one bf16 step)
        assert (w1.float() - w0.float()).abs().max().item() <= 4e-3
    w_ref = orc.inter_chunk_softmax(sc0.float().cpu(), lse, pb.bfloat16().float(), idx0.cpu(), bf16_sum=True)
    assert_close_bf16(w1, w_ref, "weights with prior bias", max_abs=8e-3)
    # the bias matters: without it another selection comes out
    idx_nb, _, _ = pkg.topk_chunk_weights(qd, lmkd, lsed, K, S, W, q_offset=off)
    assert not torch.equal(idx_nb, idx1)


@pytest.mark.parametrize("L,N,HQ,H,D,K", [(3000, 47, 8, 2, 128, 16), (5000, 400, 4, 1, 64, 32),
                                          (5000, 400, 16, 2, 64, 32), (3000, 47, 7, 1, 128, 16),
                                          (9000, 300, 12, 2, 128, 32), (5000, 400, 4, 2, 64, 32)])
def test_prefill_selection_with_a_key_per_query_head(pkg, orc, dev, L, N, HQ, H, D, K):
    """The layer's default pooling (attention-pooled chunk keys, one per query head, with their prior
    bias; models/FlashHiLS/hils_attention.py:391-416, 568-602) through topk_chunk_weights: same
    indices and scores as the operator, weights against chunk_weights and the oracle."""
    note(f"prefill selection, key per query head, L{L} N{N} HQ{HQ} H{H} D{D} K{K}")
    B, S, W = 1, 64, 1
    G = HQ // H
    off = N * S - L if N * S > L else 0
    gen = torch.Generator().manual_seed(402)
    q = torch.randn(B, L, HQ, D, generator=gen).bfloat16()
    lmk = torch.randn(B, N, HQ, D, generator=gen).bfloat16()
    lse = (torch.randn(B, L, HQ, generator=gen) * 3 + 5).bfloat16().float()
    pb = torch.randn(B, N, HQ, generator=gen) * 2
    qd, lmkd, lsed, pbd = q.to(dev), lmk.to(dev), lse.to(dev), pb.to(dev)
    dbg = {}
    idx0, sc0 = pkg.online_softmax_topk_head(qd, lmkd, lsed, K, S, W, q_offset=off, is_training=False,
                                             bias=pbd, G=G, _debug=dbg)
    lim = orc.causal_chunk_limit(L, off, W, S)
    want = orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim, K)
    assert torch.equal(idx0.cpu(), want), "indices not bit-exact from the kernel's biased logits"
    ridx, rsc, aux = orc.online_softmax_topk_head(q.view(B, L, H, G, D), lmk, lse, K, S, W, q_offset=off,
                                                  bias=pb, return_aux=True)
    assert_close_f32(dbg["sel_logits"].cpu(), aux["sel_logits"], 2e-3, "biased selection logits")
    assert (idx0.cpu() == ridx).float().mean().item() >= 0.99
    w0 = pkg.chunk_weights(sc0, lsed, pbd, idx0)
    for lse_in in (lsed, lsed.bfloat16()):
        idx1, sc1, w1 = pkg.topk_chunk_weights(qd, lmkd, lse_in, K, S, W, q_offset=off, prior_b=pbd, num_kv_heads=H)
        assert torch.equal(idx1, idx0) and torch.equal(sc1.view(torch.int16), sc0.view(torch.int16))
        assert (w1.float() - w0.float()).abs().max().item() <= 4e-3
    w_ref = orc.inter_chunk_softmax(sc0.float().cpu(), lse, pb.bfloat16().float(), idx0.cpu(), bf16_sum=True)
    assert (w0.float().cpu() - w_ref).abs().max().item() <= 8e-3


@pytest.mark.parametrize("B,Lq,Lkv,HQ,H,D,K", [(32, 1, 32768, 32, 8, 128, 32), (16, 1, 16512, 8, 8, 64, 16),
                                               (50, 2, 20480, 4, 1, 128, 8), (2, 1, 4096, 8, 2, 128, 16),
                                               (64, 1, 32768, 16, 2, 64, 32), (16, 1, 65536, 40, 8, 128, 16),
                                               # logits and bias of the row do not fit the LDS side by side: one array
                                               (48, 1, 131072, 16, 2, 64, 32), (12, 1, 196608, 32, 8, 128, 32)])
def test_decode_step_with_prior_bias(pkg, orc, dev, B, Lq, Lkv, HQ, H, D, K):
    """decode_step(prior_b=): one launch per step with the bias staged beside the logits; the chunk
    keys and the bias token-major (the reference's layout) and head-major (the cache layers')."""
    note(f"decode_step with prior bias B{B} Lq{Lq} Lkv{Lkv} HQ{HQ} H{H} D{D} K{K}")
    S, W = 64, 1
    G, N, off = HQ // H, Lkv // 64, Lkv - Lq
    gen = torch.Generator().manual_seed(402)
    q = torch.randn(B, Lq, HQ, D, generator=gen).bfloat16()
    k = torch.randn(B, Lkv, H, D, generator=gen).bfloat16()
    v = torch.randn(B, Lkv, H, D, generator=gen).bfloat16()
    lse = torch.randn(B, Lq, HQ, generator=gen) * 3 + 5
    pb = torch.randn(B, N, HQ, generator=gen) * 2
    qd, kd, vd, lsed, pbd = q.to(dev), k.to(dev), v.to(dev), lse.to(dev), pb.to(dev)
    lmkd = pkg.chunk_mean_pool(kd[:, : N * 64].contiguous(), 64)
    dbg = {}
    o1, w1, idx1, sc1 = pkg.decode_step(qd, lmkd, kd, vd, lsed, K, S, W, q_offset=off, prior_b=pbd, _debug=dbg)
    lim = orc.causal_chunk_limit(Lq, off, W, S)
    if dbg:  # the one-launch kernel ran: its biased logits, its selection rule
        want = orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim, K)
        assert torch.equal(idx1.cpu(), want)
        _, _, aux = orc.online_softmax_topk_head(q.view(B, Lq, H, G, D), lmkd.cpu(), lse, K, S, W, q_offset=off,
                                                 bias=pb, return_aux=True)
        assert_close_f32(dbg["sel_logits"].cpu(), aux["sel_logits"], 2e-3, "biased selection logits")
        assert_close_f32(dbg["lse_total"].cpu(), aux["lse_total"], 1e-3, "lse_total")
    # the same step as separate calls of the operators
    idx0, sc0 = pkg.online_softmax_topk_head(qd, lmkd, lsed, K, S, W, q_offset=off, is_training=False, bias=pbd)
    w0 = pkg.chunk_weights(sc0, lsed, pbd, idx0)
    assert torch.equal(idx1, idx0) and torch.equal(sc1, sc0)
    assert (w1.float() - w0.float()).abs().max().item() <= 4e-3
    w_ref, o_ref = _oracle_step(orc, q, lmkd.cpu(), lse, pb, k, v, K, S, W, off, idx1.cpu(), sc1.cpu())
    assert_close_bf16(w1, w_ref, "weights with prior bias", max_abs=8e-3)
    assert_close_bf16(o1, orc.sparse_attn(q, k, v, w1.cpu(), idx1.cpu(), chunk_size=S), "decode_step output")
    # head-major chunk keys and bias with spare capacity: the same bits
    from hils_attention_amd.ops.hils_glue import head_major_chunk_keys
    lmk_hm, pb_hm = head_major_chunk_keys(lmkd, pbd, capacity=N + 7)
    o2, w2, idx2, sc2 = pkg.decode_step(qd, lmk_hm, kd, vd, lsed, K, S, W, q_offset=off, prior_b=pb_hm,
                                        lmk_head_major=True, num_chunks=N)
    assert torch.equal(idx2, idx1) and torch.equal(sc2, sc1) and torch.equal(w2, w1) and torch.equal(o2, o1)
    o3, w3, idx3, _ = pkg.decode_step(qd, lmk_hm, kd, vd, lsed, K, S, W, q_offset=off, lmk_head_major=True,
                                      num_chunks=N)
    o4, w4, idx4, _ = pkg.decode_step(qd, lmkd, kd, vd, lsed, K, S, W, q_offset=off)
    assert torch.equal(idx3, idx4) and torch.equal(w3, w4) and torch.equal(o3, o4)
    assert not torch.equal(idx3, idx1), "the bias must change the selection"


@pytest.mark.parametrize("B,Lq,Lkv,HQ,H,D,K", [(32, 1, 32768, 32, 8, 128, 32), (50, 2, 20480, 4, 1, 128, 8),
                                               (24, 1, 65536, 12, 4, 64, 64), (48, 1, 16512, 6, 2, 64, 16),
                                               (48, 1, 16384, 4, 2, 64, 8), (64, 1, 32768, 16, 2, 64, 32),
                                               (48, 1, 65536, 14, 2, 128, 16),
                                               (48, 1, 131072, 16, 2, 64, 32)])  # bias and logits in one array
def test_decode_step_with_a_key_per_query_head(pkg, orc, dev, B, Lq, Lkv, HQ, H, D, K):
    """The layer's default pooling in decode: one attention-pooled chunk key per query head and its
    prior bias.  One launch per step; token-major, head-major and paged keys give the same bits; the
    selection rule holds on the kernel's own logits, which match the oracle's per-head products."""
    note(f"decode_step, key per query head, B{B} Lq{Lq} Lkv{Lkv} HQ{HQ} H{H} D{D} K{K}")
    S, W = 64, 1
    G, N, off = HQ // H, Lkv // 64, Lkv - Lq
    gen = torch.Generator().manual_seed(405)
    q = torch.randn(B, Lq, HQ, D, generator=gen).bfloat16()
    k = torch.randn(B, Lkv, H, D, generator=gen).bfloat16()
    v = torch.randn(B, Lkv, H, D, generator=gen).bfloat16()
    lmk = torch.randn(B, N, HQ, D, generator=gen).bfloat16()
    lse = torch.randn(B, Lq, HQ, generator=gen) * 3 + 5
    pb = torch.randn(B, N, HQ, generator=gen) * 2
    qd, kd, vd, lmkd, lsed, pbd = q.to(dev), k.to(dev), v.to(dev), lmk.to(dev), lse.to(dev), pb.to(dev)
    dbg = {}
    o1, w1, idx1, sc1 = pkg.decode_step(qd, lmkd, kd, vd, lsed, K, S, W, q_offset=off, prior_b=pbd, _debug=dbg)
    assert dbg, "the one-launch kernel did not take this shape"
    lim = orc.causal_chunk_limit(Lq, off, W, S)
    want = orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim, K)
    assert torch.equal(idx1.cpu(), want)
    ridx, _, aux = orc.online_softmax_topk_head(q.view(B, Lq, H, G, D), lmk, lse, K, S, W, q_offset=off, bias=pb,
                                                return_aux=True)
    assert_close_f32(dbg["sel_logits"].cpu(), aux["sel_logits"], 2e-3, "biased selection logits")
    assert_close_f32(dbg["lse_total"].cpu(), aux["lse_total"], 1e-3, "lse_total")
    assert (idx1.cpu() == ridx).float().mean().item() >= 0.99
    safe = idx1.cpu().long().clamp_min(0).unsqueeze(3).expand(-1, -1, -1, G, -1)
    raw = torch.gather(aux["logits"], -1, safe).masked_fill((idx1.cpu() < 0).unsqueeze(3).expand(-1, -1, -1, G, -1),
                                                             float("-inf"))
    assert_close_bf16(sc1.view(B, Lq, H, G, K), raw, "scores carry no bias")
    w_ref = orc.inter_chunk_softmax(sc1.float().cpu(), lse, pb.bfloat16().float(), idx1.cpu(), bf16_sum=True)
    assert_close_bf16(w1, w_ref, "weights with prior bias", max_abs=8e-3)
    assert_close_bf16(o1, orc.sparse_attn(q, k, v, w1.cpu(), idx1.cpu(), chunk_size=S), "decode_step output")
    # the operators one by one (the selection alone runs on the same row kernel)
    idx0, sc0 = pkg.online_softmax_topk_head(qd, lmkd, lsed, K, S, W, q_offset=off, is_training=False, bias=pbd, G=G)
    assert torch.equal(idx1, idx0) and torch.equal(sc1, sc0)
    w0 = pkg.chunk_weights(sc0, lsed, pbd, idx0)
    assert (w1.float() - w0.float()).abs().max().item() <= 4e-3
    # head-major keys and bias with spare capacity: the same bits
    lmk_hm, pb_hm = pkg.head_major_chunk_keys(lmkd, pbd, capacity=N + 5, num_kv_heads=H)
    o2, w2, idx2, sc2 = pkg.decode_step(qd, lmk_hm, kd, vd, lsed, K, S, W, q_offset=off, prior_b=pb_hm,
                                        lmk_head_major=True, num_chunks=N)
    assert torch.equal(idx2, idx1) and torch.equal(sc2, sc1) and torch.equal(w2, w1) and torch.equal(o2, o1)
    # pages: keys per page and per sequence
    if Lkv % 64 == 0:
        num_pages = B * N + 3
        perm = torch.randperm(num_pages, generator=gen)[: B * N].view(B, N).to(dev)
        k_pages = torch.randn(num_pages, H, 64, D, generator=gen).bfloat16().to(dev)
        v_pages = torch.randn(num_pages, H, 64, D, generator=gen).bfloat16().to(dev)
        lmk_pages = torch.randn(num_pages, HQ, D, generator=gen).bfloat16().to(dev)
        pb_pages = torch.randn(num_pages, HQ, generator=gen).to(dev)
        k_pages[perm] = kd.view(B, N, 64, H, D).permute(0, 1, 3, 2, 4)
        v_pages[perm] = vd.view(B, N, 64, H, D).permute(0, 1, 3, 2, 4)
        lmk_pages[perm] = lmkd
        pb_pages[perm] = pbd
        table = torch.full((B, N + 2), -1, dtype=torch.int32, device=dev)
        table[:, :N] = perm.to(torch.int32)
        o3, w3, idx3 = pkg.paged_hils_attend(qd, k_pages, v_pages, lmk_pages, table, lsed, Lkv, K, W, prior_pages=pb_pages)
        assert torch.equal(idx3, idx1) and torch.equal(w3, w1) and torch.equal(o3, o1)
        lmk_hm2, pb_hm2 = pkg.head_major_chunk_keys(lmkd, pbd, capacity=N + 2, num_kv_heads=H)
        o4, w4, idx4 = pkg.paged_hils_attend(qd, k_pages, v_pages, None, table, lsed, Lkv, K, W, lmk_dense=lmk_hm2,
                                             prior_dense=pb_hm2)
        assert torch.equal(idx4, idx1) and torch.equal(w4, w1) and torch.equal(o4, o1)


def test_paged_decode_with_prior_bias(pkg, orc, dev):
    """The paged cache: per-page chunk keys / bias and the per-sequence head-major ones give the bits
    of the token-major decode step."""
    note("paged decode with prior bias")
    B, Lkv, HQ, H, D, K, S, W = 16, 20480, 16, 4, 128, 16, 64, 1
    G, N = HQ // H, Lkv // 64
    gen = torch.Generator().manual_seed(403)
    q = torch.randn(B, 1, HQ, D, generator=gen).bfloat16().to(dev)
    k = torch.randn(B, Lkv, H, D, generator=gen).bfloat16().to(dev)
    v = torch.randn(B, Lkv, H, D, generator=gen).bfloat16().to(dev)
    lse = (torch.randn(B, 1, HQ, generator=gen) * 3 + 5).to(dev)
    pb = (torch.randn(B, N, HQ, generator=gen) * 2).to(dev)
    lmk = pkg.chunk_mean_pool(k, 64)
    o0, w0, idx0, _ = pkg.decode_step(q, lmk, k, v, lse, K, S, W, q_offset=Lkv - 1, prior_b=pb)
    num_pages = B * N + 5
    perm = torch.randperm(num_pages, generator=gen)[: B * N].to(dev)
    k_pages = torch.zeros(num_pages, H, 64, D, dtype=torch.bfloat16, device=dev)
    v_pages = torch.zeros_like(k_pages)
    k_pages[perm] = k.view(B, N, 64, H, D).permute(0, 1, 3, 2, 4).reshape(B * N, H, 64, D)
    v_pages[perm] = v.view(B, N, 64, H, D).permute(0, 1, 3, 2, 4).reshape(B * N, H, 64, D)
    lmk_pages = torch.zeros(num_pages, H, D, dtype=torch.bfloat16, device=dev)
    lmk_pages[perm] = lmk.reshape(B * N, H, D)
    prior_pages = torch.zeros(num_pages, HQ, device=dev)
    prior_pages[perm] = pb.reshape(B * N, HQ)
    table = perm.view(B, N).to(torch.int32).contiguous()
    dbg = {}
    o1, w1, idx1 = pkg.paged_hils_attend(q, k_pages, v_pages, lmk_pages, table, lse, Lkv, K, W,
                                         prior_pages=prior_pages, _debug=dbg)
    assert dbg and torch.equal(idx1, idx0) and torch.equal(w1, w0) and torch.equal(o1, o0)
    from hils_attention_amd.ops.hils_glue import head_major_chunk_keys
    lmk_hm, pb_hm = head_major_chunk_keys(lmk, pb, capacity=N + 3)
    o2, w2, idx2 = pkg.paged_hils_attend(q, k_pages, v_pages, None, table, lse, Lkv, K, W, lmk_dense=lmk_hm,
                                         prior_dense=pb_hm)
    assert torch.equal(idx2, idx0) and torch.equal(w2, w0) and torch.equal(o2, o0)
    # few rows: the separate calls (row-per-workgroup selection with the paged bias, then attention)
    o3, w3, idx3 = pkg.paged_hils_attend(q[:2], k_pages, v_pages, lmk_pages, table[:2].contiguous(), lse[:2], Lkv,
                                         K, W, prior_pages=prior_pages)
    o4, w4, idx4, _ = pkg.decode_step(q[:2], lmk[:2], k[:2], v[:2], lse[:2], K, S, W, q_offset=Lkv - 1, prior_b=pb[:2])
    assert torch.equal(idx3, idx4)
    assert (w3.float() - w4.float()).abs().max().item() <= 4e-3
    assert_close_bf16(o3, o4.float(), "paged two-call path vs dense two-call path")


@pytest.mark.parametrize("G,chunk_pooling", [(4, True), (1, False), (2, False), (4, False), (8, False), (8, True)])
def test_cache_layers_keep_and_use_the_prior(pkg, orc, dev, G, chunk_pooling):
    """HiLSDynamicLayer / HiLSPagedLayer filled incrementally with the chunks' prior queries: the
    entropy bias (and, without chunk pooling, the attention-pooled keys) match the oracle's attention
    pool, and hils_attend equals the oracle's step with bias= / prior_b= on the tokens seen so far."""
    note(f"cache layers with prior queries, G{G} chunk_pooling={chunk_pooling}")
    B, H, D, S, K, W = 2, 2, 64, 64, 4, 1
    HQ = H * G
    gen = torch.Generator().manual_seed(404 + G)
    L0, steps = 64 * 5 + 20, 150
    Lt = L0 + steps
    k = torch.randn(B, Lt, H, D, generator=gen).bfloat16()
    v = torch.randn(B, Lt, H, D, generator=gen).bfloat16()
    mu = torch.randn(B, Lt // S, HQ, D, generator=gen).bfloat16()
    kd, vd, mud = k.to(dev), v.to(dev), mu.to(dev)
    dyn = pkg.HiLSDynamicLayer(chunk_size=S, capacity=256, chunk_pooling=chunk_pooling)
    paged = None
    if True:
        paged = pkg.HiLSPagedLayer(num_pages=40, batch=B, max_pages_per_seq=12, num_kv_heads=H, head_dim=D,
                                   device=dev, num_q_heads=HQ, chunk_pooling=chunk_pooling,
                                   page_order=torch.randperm(40, generator=gen).tolist())
    layers = [c for c in (dyn, paged) if c is not None]
    for c in layers:
        c.update(kd[:, :L0], vd[:, :L0], mu_q=mud[:, : L0 // S])
    for t in range(L0, Lt):
        n = t + 1
        new_full = n // S - t // S
        mq = mud[:, t // S: n // S] if new_full else None
        for c in layers:
            c.update(kd[:, t:n], vd[:, t:n], mu_q=mq)
        if t % 31 and t not in (Lt - 1, 383, 384):
            continue
        full = n // S
        lk, lb, _ = orc.chunk_attn_pool(mu[:, :full].float(), k[:, : full * S].view(B, full, S, H, D)
                                        .repeat_interleave(G, dim=3).float())
        lmk_ref = orc.mean_pool(k[:, : full * S], S).bfloat16() if chunk_pooling else lk.bfloat16()
        assert_close_bf16(dyn.prior_b[:, :full], lb, "entropy bias of the cache", max_abs=2e-2)
        assert_close_bf16(dyn.lmk_k[:, :full], lmk_ref.float(), "chunk keys of the cache")
        q = torch.randn(B, 1, HQ, D, generator=gen).bfloat16()
        lse = torch.randn(B, 1, HQ, generator=gen) * 2 + 3
        pb_layer = dyn.prior_b[:, :full].contiguous().cpu()          # what the layer keeps (fp32)
        lmk_layer = dyn.lmk_k[:, :full].contiguous().cpu()
        lim = orc.causal_chunk_limit(1, n - 1, W, S)
        outs = []
        for c in layers:
            dbg = {}
            o, w, idx = c.hils_attend(q.to(dev), lse.to(dev), K, W, _debug=dbg)
            outs.append((o, w, idx))
            if "sel_logits" in dbg:
                want = orc.topk_select(dbg["sel_logits"].cpu()[..., :full], dbg["lse_total"].cpu(), lim, K)
                assert torch.equal(idx.cpu(), want), f"step {t}: selection rule"
            # the oracle's step on the layer's own chunk keys and bias
            qg = q.view(B, 1, H, G, D)
            ridx, rsc = orc.online_softmax_topk_head(qg, lmk_layer, lse, K, S, W, q_offset=n - 1, bias=pb_layer)
            assert (idx.cpu() == ridx).float().mean().item() >= 0.9, f"step {t}: indices"
            safe = idx.cpu().long().clamp_min(0).unsqueeze(3).expand(-1, -1, -1, G, -1)
            sc = torch.gather(orc.topk_logits(qg, lmk_layer), -1, safe).masked_fill(
                (idx.cpu() < 0).unsqueeze(3).expand(-1, -1, -1, G, -1), float("-inf")).reshape(B, 1, HQ, K)
            w_ref = orc.inter_chunk_softmax(sc.bfloat16().float(), lse, pb_layer.bfloat16().float(), idx.cpu(), bf16_sum=True)
            assert_close_bf16(w, w_ref, f"step {t}: weights", max_abs=1e-2)
            k_pad = torch.zeros(B, ((n + S - 1) // S + 1) * S, H, D, dtype=k.dtype)
            v_pad = torch.zeros_like(k_pad)
            k_pad[:, :n], v_pad[:, :n] = k[:, :n], v[:, :n]
            o_ref = orc.sparse_attn(q, k_pad, v_pad, w.cpu(), idx.cpu(), chunk_size=S)
            assert_close_bf16(o, o_ref, f"step {t}: remote branch")
        if len(outs) == 2 and chunk_pooling:  # same chunk keys, same bias: the two layers agree
            assert torch.equal(outs[0][2], outs[1][2])
            assert (outs[0][1].float() - outs[1][1].float()).abs().max().item() <= 4e-3
