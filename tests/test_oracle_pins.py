"""Pins for the CPU oracle: closed forms, library routines and brute force on tiny inputs.

The reference stores no golden vectors for this path, so every oracle function is pinned
by independent mathematics chosen so that a dropped term, a wrong sign/index or a
transposed operand fails at least one check.
"""
import itertools
import math

import pytest
import torch
import torch.nn.functional as F

from util import rand_indices


# ------------------------------------------------------------------ pooling
def test_mean_pool_closed_form(orc):
    k = torch.arange(2 * 128 * 3 * 4, dtype=torch.float32).view(2, 128, 3, 4)
    out = orc.mean_pool(k, 64)
    assert out.shape == (2, 2, 3, 4)
    # mean of an arithmetic progression = midpoint of first and last token of the chunk
    assert torch.allclose(out[1, 1], (k[1, 64] + k[1, 127]) / 2)


def test_attn_pool_special_cases(orc):
    torch.manual_seed(0)
    B, N, S, H, D = 1, 3, 64, 2, 16
    # all keys equal -> lmk_k = that key, entropy = ln 63
    key = torch.randn(B, N, 1, H, D)
    k = key.expand(B, N, S, H, D).contiguous()
    mu = torch.randn(B, N, H, D)
    lk, lb, p = orc.chunk_attn_pool(mu, k)
    assert torch.allclose(lk, key[:, :, 0], atol=1e-5)
    assert torch.allclose(lb, torch.full_like(lb, math.log(63)), atol=1e-5)
    assert torch.all(p[:, :, -1] == 0)
    # mu = 0 -> uniform mean over the first 63 tokens (landmark excluded)
    k = torch.randn(B, N, S, H, D)
    lk, lb, _ = orc.chunk_attn_pool(torch.zeros(B, N, H, D), k)
    assert torch.allclose(lk, k[:, :, :63].mean(2), atol=1e-5)
    # one dominant key -> entropy -> 0 and lmk_k -> that key
    k = torch.randn(B, N, S, H, D) * 0.01
    k[:, :, 5] = mu * 50
    lk, lb, _ = orc.chunk_attn_pool(mu, k)
    assert lb.abs().max() < 1e-3
    assert torch.allclose(lk, k[:, :, 5], atol=1e-3)


def test_attn_pool_vs_library(orc):
    torch.manual_seed(1)
    B, N, S, H, D = 2, 4, 64, 3, 32
    mu = torch.randn(B, N, H, D)
    k = torch.randn(B, N, S, H, D)
    lk, lb, p = orc.chunk_attn_pool(mu, k, 0.37)
    qq = mu.reshape(B * N, H, 1, D)
    kk = k[:, :, :63].permute(0, 1, 3, 2, 4).reshape(B * N, H, 63, D)
    ref = F.scaled_dot_product_attention(qq, kk, kk, scale=0.37).reshape(B, N, H, D)
    assert torch.allclose(lk, ref, atol=1e-5)
    ent = torch.distributions.Categorical(probs=p[:, :, :63].permute(0, 1, 3, 2)).entropy()
    assert torch.allclose(lb, ent, atol=1e-5)
    # a different scale must change the result (scale is not silently dropped)
    assert not torch.allclose(lk, orc.chunk_attn_pool(mu, k)[0], atol=1e-3)


# ------------------------------------------------------------------ top-k
def brute_topk(q, lmks, lse_swa, topk, S, W, q_offset=0, bias=None, drop=None):
    """Enumerate all chunks in pure Python; order by (-score, index)."""
    B, L, h_kv, G, D = q.shape
    N = lmks.shape[1]
    scale = 1.0 / math.sqrt(D)
    out = torch.full((B, L, h_kv, topk), -1, dtype=torch.int32)
    for b, t, h in itertools.product(range(B), range(L), range(h_kv)):
        tg = t + q_offset
        lim = (tg - W + 1) // S if W > 0 else tg // S
        vis = [c for c in range(N) if c < lim]
        if not vis:
            continue
        pooled = {}
        lt = []
        for g in range(G):
            lg = torch.tensor([float(torch.dot(q[b, t, h, g], lmks[b, c, h])) * scale
                               + (float(bias[b, c, h * G + g]) if bias is not None else 0.0) for c in vis],
                              dtype=torch.float64)
            lt.append(torch.logaddexp(lse_swa[b, t, h * G + g].double(), torch.logsumexp(lg, 0)))
            for i, c in enumerate(vis):
                pooled[c] = max(pooled.get(c, -float("inf")), float(lg[i] - lt[g]))
        cand = [c for c in vis if drop is None or drop[b, t, c] == 0]
        cand.sort(key=lambda c: (-pooled[c], c))
        sel = sorted(cand[:topk])
        out[b, t, h, :len(sel)] = torch.tensor(sel, dtype=torch.int32)
    return out


def test_topk_brute_force_tiny(orc):
    torch.manual_seed(2)
    B, L, h_kv, G, D, N, S, topk = 1, 40, 2, 2, 8, 10, 4, 3
    q = torch.randn(B, L, h_kv, G, D)
    lmks = torch.randn(B, N, h_kv, D)
    lse = torch.randn(B, L, h_kv * G)
    bias = torch.randn(B, N, h_kv * G)
    drop = (torch.rand(B, L, N) < 0.2).int()
    for W, off, b_, d_ in [(1, 0, None, None), (3, 0, bias, None), (0, 0, None, drop), (2, 5, bias, drop)]:
        idx, scores = orc.online_softmax_topk_head(q, lmks, lse, topk, S, W, q_offset=off, bias=b_, drop_mask=d_)
        assert torch.equal(idx, brute_topk(q, lmks, lse, topk, S, W, off, b_, d_))
        # returned scores are the raw scaled qk at the chosen chunks, -inf at -1
        for t in (9, 23, 39):
            for h in range(h_kv):
                for j, c in enumerate(idx[0, t, h].tolist()):
                    for g in range(G):
                        want = float(torch.dot(q[0, t, h, g], lmks[0, c, h])) / math.sqrt(D) if c >= 0 else -math.inf
                        assert scores[0, t, h, g, j].item() == pytest.approx(want, abs=1e-5)


def test_topk_invariants_and_reduction_to_torch_topk(orc):
    torch.manual_seed(3)
    B, L, h_kv, D, N, S, topk = 2, 64, 1, 16, 16, 4, 5
    q = torch.randn(B, L, h_kv, 1, D)
    lmks = torch.randn(B, N, h_kv, D)
    lse = torch.full((B, L, h_kv), float("-inf"))
    idx, _, aux = orc.online_softmax_topk_head(q, lmks, lse, topk, S, 1, return_aux=True)
    lim = orc.causal_chunk_limit(L, 0, 1, S)
    for b in range(B):
        for t in range(L):
            nv = int(lim[t])
            row = [c for c in idx[b, t, 0].tolist() if c >= 0]
            assert row == sorted(row) and len(set(row)) == len(row)
            assert len(row) == min(topk, max(nv, 0))
            assert idx[b, t, 0].tolist()[len(row):] == [-1] * (topk - len(row))
            if nv > 0:
                want = torch.topk(aux["logits"][b, t, 0, 0, :nv], min(topk, nv)).indices.sort().values.tolist()
                assert row == want
    # lse_total is logaddexp of the two branches
    lse2 = torch.randn(B, L, h_kv)
    _, _, aux2 = orc.online_softmax_topk_head(q, lmks, lse2, topk, S, 1, return_aux=True)
    t = 40
    manual = torch.logaddexp(lse2[0, t, 0], torch.logsumexp(aux2["logits"][0, t, 0, 0, :int(lim[t])], 0))
    assert aux2["lse_total"][0, t, 0, 0].item() == pytest.approx(manual.item(), abs=1e-5)


def test_topk_tie_break_and_permutation_equivariance(orc):
    torch.manual_seed(4)
    B, L, D, N, S, topk = 1, 32, 8, 8, 4, 3
    q = torch.randn(B, L, 1, 1, D)
    lmks = torch.randn(B, N, 1, D)
    lmks[:, 1::2] = lmks[:, 0::2]  # chunks 2j and 2j+1 tie exactly
    lse = torch.zeros(B, L, 1)
    idx, _ = orc.online_softmax_topk_head(q, lmks, lse, topk, S, 1)
    for t in range(L):
        row = [c for c in idx[0, t, 0].tolist() if c >= 0]
        for c in row:
            if c % 2 == 1:
                assert c - 1 in row, "a tie must be won by the lower chunk index"
    # permuting the chunks (non-causal, distinct keys) permutes the selected set
    lmks = torch.randn(B, N, 1, D)
    perm = torch.randperm(N)
    a, _ = orc.online_softmax_topk_head(q, lmks, lse, topk, S, 1, is_causal=False)
    b, _ = orc.online_softmax_topk_head(q, lmks[:, perm], lse, topk, S, 1, is_causal=False)
    inv = torch.argsort(perm)
    for t in range(L):
        assert sorted(inv[a[0, t, 0].long()].tolist()) == b[0, t, 0].tolist()


def test_topk_select_is_exact_on_given_scores(orc):
    """topk_select on hand-made scores: max over g, -inf and NaN never selected, ties by index."""
    sel = torch.tensor([[[[[1.0, 5.0, 5.0, float("-inf"), 2.0, float("nan")],
                           [0.0, 0.0, 7.0, float("-inf"), 2.5, 1.0]]]]])  # (1,1,1,G=2,N=6)
    lt = torch.tensor([[[[0.0, 1.0]]]])
    # pooled = max(g0 - 0, g1 - 1) = [1, 5, 6, -inf, 2, 0]
    assert orc.topk_select(sel, lt, None, 3).tolist() == [[[[1, 2, 4]]]]
    assert orc.topk_select(sel, lt, None, 6).tolist() == [[[[0, 1, 2, 4, 5, -1]]]]
    assert orc.topk_select(sel, lt, torch.tensor([2]), 3).tolist() == [[[[0, 1, -1]]]]
    tie = torch.tensor([[[[[3.0, 3.0, 3.0, 3.0]]]]])
    assert orc.topk_select(tie, torch.zeros(1, 1, 1, 1), None, 2).tolist() == [[[[0, 1]]]]


def test_topk_gumbel_and_per_qhead_keys_brute_force(orc):
    """Two option branches of the selection, each against a pure-Python enumeration.

    Gumbel noise g[h_q, c] is added to the scaled logit of (query head, chunk) before both the
    LSE and the selection (ops/topk_head_softmax.py:47-52 in the torch reference), the returned
    scores stay raw.  Per-q-head chunk keys (B,N,h_kv*G,D): head h*G+g of the keys scores query
    head (h, g); selection is still per KV head with the max over g."""
    torch.manual_seed(21)
    B, L, h_kv, G, D, N, S, topk, W = 1, 36, 2, 3, 8, 9, 4, 3, 1
    scale = 1.0 / math.sqrt(D)
    q = torch.randn(B, L, h_kv, G, D)
    lse = torch.randn(B, L, h_kv * G)
    shared = torch.randn(B, N, h_kv, D)
    per_head = torch.randn(B, N, h_kv * G, D)
    # the noise is large against the logits' spread, so it changes most selections
    noise = torch.randn(1, 1, h_kv * G, N) * 3

    def brute(lmks, per_qhead, gum):
        out = torch.full((B, L, h_kv, topk), -1, dtype=torch.int32)
        raw = torch.full((B, L, h_kv, G, N), float("nan"), dtype=torch.float64)
        for t, h in itertools.product(range(L), range(h_kv)):
            vis = list(range(max(0, (t - W + 1) // S)))
            if not vis:
                continue
            pooled = {c: -math.inf for c in vis}
            for g in range(G):
                hq = h * G + g
                lg = []
                for c in vis:
                    key = lmks[0, c, hq] if per_qhead else lmks[0, c, h]
                    r = float(torch.dot(q[0, t, h, g].double(), key.double())) * scale
                    raw[0, t, h, g, c] = r
                    lg.append(r + (float(gum[0, 0, hq, c]) if gum is not None else 0.0))
                lt = math.log(math.exp(float(lse[0, t, hq])) + sum(math.exp(x) for x in lg))
                for c, x in zip(vis, lg):
                    pooled[c] = max(pooled[c], x - lt)
            sel = sorted(sorted(vis, key=lambda c: (-pooled[c], c))[:topk])
            out[0, t, h, :len(sel)] = torch.tensor(sel, dtype=torch.int32)
        return out, raw

    plain, _ = orc.online_softmax_topk_head(q, shared, lse, topk, S, W)
    for lmks, per_qhead, gum in [(shared, False, noise), (per_head, True, None), (per_head, True, noise)]:
        idx, scores = orc.online_softmax_topk_head(q, lmks, lse, topk, S, W, gumbel_noise=gum)
        want, raw = brute(lmks, per_qhead, gum)
        assert torch.equal(idx, want), (per_qhead, gum is not None)
        for t in (17, 35):
            for h, g in itertools.product(range(h_kv), range(G)):
                for j, c in enumerate(idx[0, t, h].tolist()):
                    if c >= 0:  # raw scaled product: no noise in the returned score
                        assert scores[0, t, h, g, j].item() == pytest.approx(raw[0, t, h, g, c].item(), abs=1e-5)
    assert not torch.equal(orc.online_softmax_topk_head(q, shared, lse, topk, S, W, gumbel_noise=noise)[0], plain), \
        "the noise must take part in the selection"
    # a per-head key tensor that repeats the shared keys selects what the shared keys select
    rep = shared.repeat_interleave(G, dim=2)
    assert torch.equal(orc.online_softmax_topk_head(q, rep, lse, topk, S, W)[0], plain)
    # swapping two heads' keys inside a group must matter (head h*G+g belongs to (h, g), not (g, h))
    swapped = per_head.clone()
    swapped[:, :, [0, 1]] = per_head[:, :, [1, 0]]
    assert not torch.equal(orc.online_softmax_topk_head(q, swapped, lse, topk, S, W)[0],
                           orc.online_softmax_topk_head(q, per_head, lse, topk, S, W)[0])


# ------------------------------------------------------------------ sparse attention
def test_sparse_attn_textbook_and_properties(orc):
    torch.manual_seed(5)
    B, L, HQ, H, D, S, K = 1, 128, 4, 2, 16, 32, 3
    q, k, v = torch.randn(B, L, HQ, D), torch.randn(B, L, H, D), torch.randn(B, L, H, D)
    # K = 1, w = 1 -> SDPA over the chunk's first S-1 tokens
    idx = torch.full((B, L, H, 1), 2, dtype=torch.int32)
    o = orc.sparse_attn(q, k, v, torch.ones(B, L, HQ, 1), idx, chunk_size=S)
    kc = k[:, 64:95].repeat_interleave(2, 2).permute(0, 2, 1, 3)
    vc = v[:, 64:95].repeat_interleave(2, 2).permute(0, 2, 1, 3)
    ref = F.scaled_dot_product_attention(q.permute(0, 2, 1, 3), kc, vc).permute(0, 2, 1, 3)
    assert torch.allclose(o, ref, atol=1e-5)
    # without the landmark mask all S tokens take part
    o2 = orc.sparse_attn(q, k, v, torch.ones(B, L, HQ, 1), idx, chunk_size=S, mask_last_token=False)
    kc = k[:, 64:96].repeat_interleave(2, 2).permute(0, 2, 1, 3)
    vc = v[:, 64:96].repeat_interleave(2, 2).permute(0, 2, 1, 3)
    ref2 = F.scaled_dot_product_attention(q.permute(0, 2, 1, 3), kc, vc).permute(0, 2, 1, 3)
    assert torch.allclose(o2, ref2, atol=1e-5)
    # -1 slots contribute nothing; output is linear in the weights; extra weight columns are ignored
    gen = torch.Generator().manual_seed(6)
    idx = rand_indices(B, L, H, K, S, gen, fill_prob=0.6)
    w1, w2 = torch.rand(B, L, HQ, K + 2), torch.rand(B, L, HQ, K + 2)
    o1 = orc.sparse_attn(q, k, v, w1, idx, chunk_size=S)
    o2 = orc.sparse_attn(q, k, v, w2, idx, chunk_size=S)
    o3 = orc.sparse_attn(q, k, v, 2 * w1 - 3 * w2, idx, chunk_size=S)
    assert torch.allclose(o3, 2 * o1 - 3 * o2, atol=1e-4)
    assert torch.count_nonzero(o1[:, :S]).item() == 0
    w1b = w1.clone()
    w1b[..., K:] = 123.0
    assert torch.equal(orc.sparse_attn(q, k, v, w1b, idx, chunk_size=S), o1)
    # brute-force one (t, head) including the per-chunk LSE
    o1, lse = orc.sparse_attn(q, k, v, w1, idx, chunk_size=S, return_lse=True)
    t, hq = 100, 3
    acc = torch.zeros(D)
    for j, c in enumerate(idx[0, t, hq // 2].tolist()):
        if c < 0:
            assert lse[0, t, hq, j] == float("-inf")
            continue
        s = (k[0, c * S:c * S + S - 1, hq // 2] @ q[0, t, hq]) / math.sqrt(D)
        assert lse[0, t, hq, j].item() == pytest.approx(torch.logsumexp(s, 0).item(), abs=1e-5)
        acc += w1[0, t, hq, j] * (torch.softmax(s, 0) @ v[0, c * S:c * S + S - 1, hq // 2])
    assert torch.allclose(o1[0, t, hq], acc, atol=1e-5)


def test_sparse_attn_slope_brute_force(orc):
    """ALiBi-like slope inside a chunk: -slope[h_q] * max(0, (S - 2) - s) is added to the raw
    q.k of token s BEFORE the scale (ops/hils_fwd_bwd_head.py:68-76), so the last unmasked token
    (s = S - 2) gets no penalty and token 0 the largest.  Pure-Python loop per (query, head)."""
    torch.manual_seed(22)
    B, L, HQ, H, D, S, K = 1, 96, 4, 2, 8, 16, 2
    G = HQ // H
    q, k, v = torch.randn(B, L, HQ, D), torch.randn(B, L, H, D), torch.randn(B, L, H, D)
    slope = torch.tensor([0.05, 0.2, 0.7, 1.5])
    gen = torch.Generator().manual_seed(23)
    idx = rand_indices(B, L, H, K, S, gen, fill_prob=0.8)
    w = torch.rand(B, L, HQ, K)
    scale = 0.3
    for mask_last in (True, False):
        o, lse = orc.sparse_attn(q, k, v, w, idx, chunk_size=S, sm_scale=scale, slope=slope,
                                 mask_last_token=mask_last, return_lse=True)
        for t in (20, 50, 95):
            for hq in range(HQ):
                acc = [0.0] * D
                for j, c in enumerate(idx[0, t, hq // G].tolist()):
                    if c < 0:
                        continue
                    ntok = S - 1 if mask_last else S
                    logit = []
                    for s_ in range(ntok):
                        dot = sum(float(q[0, t, hq, d]) * float(k[0, c * S + s_, hq // G, d]) for d in range(D))
                        logit.append((dot - float(slope[hq]) * max(0, S - 2 - s_)) * scale)
                    m = max(logit)
                    z = sum(math.exp(x - m) for x in logit)
                    assert lse[0, t, hq, j].item() == pytest.approx(m + math.log(z), abs=1e-4)
                    for s_ in range(ntok):
                        p = math.exp(logit[s_] - m) / z
                        for d in range(D):
                            acc[d] += float(w[0, t, hq, j]) * p * float(v[0, c * S + s_, hq // G, d])
                assert torch.allclose(o[0, t, hq], torch.tensor(acc), atol=1e-4)
    # slope 0 is the plain operator; a large slope concentrates the mass on the last unmasked token
    o0 = orc.sparse_attn(q, k, v, w, idx, chunk_size=S, sm_scale=scale, slope=torch.zeros(HQ))
    assert torch.allclose(o0, orc.sparse_attn(q, k, v, w, idx, chunk_size=S, sm_scale=scale), atol=1e-6)
    one = torch.full((B, L, H, 1), 1, dtype=torch.int32)
    o_big = orc.sparse_attn(q, k, v, torch.ones(B, L, HQ, 1), one, chunk_size=S, sm_scale=scale,
                            slope=torch.full((HQ,), 1e4))
    want = v[0, S + S - 2].repeat_interleave(G, 0)  # token S-2 of chunk 1
    assert torch.allclose(o_big[0, 40], want, atol=1e-4)


def test_factorised_equals_dense_when_weights_are_true_masses(orc):
    """Select all visible chunks with w = softmax(log Z_c, lse_swa): equals dense softmax
    attention over the kept tokens ("equivalent when Z' = Z")."""
    torch.manual_seed(7)
    B, L, HQ, H, D, S, W = 1, 96, 4, 2, 8, 16, 5
    N = L // S
    q, k, v = torch.randn(B, L, HQ, D), torch.randn(B, L, H, D), torch.randn(B, L, H, D)
    lim = orc.causal_chunk_limit(L, 0, W, S)
    idx = torch.arange(N).view(1, 1, 1, N).expand(B, L, H, N).clone()
    idx = torch.where(idx < lim.view(1, L, 1, 1), idx, torch.full_like(idx, -1)).to(torch.int32)
    lz = orc.exact_chunk_log_z(q, k, chunk_size=S, window_size=W, mask_lmk=True)
    swa_o, lse_swa = orc.swa(q, k, v, window_size=W, chunk_size=S, mask_lmk=True)
    w = torch.softmax(torch.cat([lz, lse_swa.unsqueeze(-1)], -1), -1)
    o = orc.sparse_attn(q, k, v, w, idx, chunk_size=S) + swa_o * w[..., N:]
    dense, lse_dense = orc.dense_hils_attention(q, k, v, chunk_size=S, window_size=W, indices=idx)
    assert torch.allclose(o, dense, atol=1e-5)
    total = torch.logaddexp(torch.logsumexp(lz, -1), lse_swa)
    assert torch.allclose(total, lse_dense, atol=1e-5)
    # dense equivalent on its own: plain causal attention with landmark keys removed
    s = torch.einsum("bihd,bjhd->bhij", q, k.repeat_interleave(2, 2)) / math.sqrt(D)
    keep = torch.ones(L, L).tril().bool() & (((torch.arange(L) + 1) % S) != 0).view(1, L)
    ref = torch.einsum("bhij,bjhd->bihd", torch.softmax(s.masked_fill(~keep, float("-inf")), -1).nan_to_num(0),
                       v.repeat_interleave(2, 2))
    assert torch.allclose(dense, ref, atol=1e-5)


# ------------------------------------------------------------------ exact log Z
def test_logz_brute_force_and_mask_pattern(orc):
    torch.manual_seed(8)
    B, L, HQ, H, D, S = 1, 50, 2, 1, 8, 8
    q, k = torch.randn(B, L, HQ, D), torch.randn(B, L, H, D)
    for W, lmk in [(1, False), (5, False), (0, False), (3, True)]:
        lz = orc.exact_chunk_log_z(q, k, chunk_size=S, window_size=W, mask_lmk=lmk)
        N = (L + S - 1) // S
        assert lz.shape == (B, L, HQ, N)
        for t in range(L):
            for c in range(N):
                toks = [j for j in range(c * S, min((c + 1) * S, L))
                        if j <= t and not (lmk and (j + 1) % S == 0)]
                if t < (c + 1) * S + W - 1 or not toks:
                    assert lz[0, t, 1, c] == float("-inf"), (W, t, c)
                else:
                    s = torch.stack([torch.dot(q[0, t, 1], k[0, j, 0]) for j in toks]) / math.sqrt(D)
                    assert lz[0, t, 1, c].item() == pytest.approx(torch.logsumexp(s, 0).item(), abs=1e-5)


def test_logz_total_mass_invariant(orc):
    torch.manual_seed(9)
    B, L, HQ, H, D, S, W = 2, 64, 4, 2, 8, 8, 6
    q, k = torch.randn(B, L, HQ, D), torch.randn(B, L, H, D)
    lz = orc.exact_chunk_log_z(q, k, chunk_size=S, window_size=W)
    _, lse_swa = orc.swa(q, k, k, window_size=W, chunk_size=S, mask_lmk=False)
    s = torch.einsum("bihd,bjhd->bhij", q, k.repeat_interleave(2, 2)) / math.sqrt(D)
    full = torch.logsumexp(s.masked_fill(torch.ones(L, L).triu(1).bool(), float("-inf")), -1).permute(0, 2, 1)
    assert torch.allclose(torch.logaddexp(torch.logsumexp(lz, -1), lse_swa), full, atol=1e-5)


# ------------------------------------------------------------------ HSA and SWA
def test_hsa_brute_force(orc):
    torch.manual_seed(10)
    Z, L, HQ, H, D, S, K, QX = 1, 32, 4, 2, 8, 8, 2, 4
    q, k, v = torch.randn(Z, L, HQ, D), torch.randn(Z, L, H, D), torch.randn(Z, L, H, D)
    idx = torch.randint(0, L // S, (Z, L // QX, H, K), dtype=torch.int32)
    w = torch.rand(Z, L // QX, H, K)
    o = orc.hsa(q, k, v, w, idx, 1.0, S, None)
    t, hq = 13, 3
    acc = torch.zeros(D)
    for j in range(K):
        c = int(idx[0, t // QX, hq // 2, j])
        s = (k[0, c * S:(c + 1) * S, hq // 2] @ q[0, t, hq]) / math.sqrt(D)
        p = torch.exp(s) / (torch.exp(s).sum() + 1.0)  # softmax with one extra unit of mass
        acc += w[0, t // QX, hq // 2, j] * (p @ v[0, c * S:(c + 1) * S, hq // 2])
    assert torch.allclose(o[0, t, hq], acc, atol=1e-5)
    # sm_n = 0 is the plain per-chunk softmax without landmark mask
    o0 = orc.hsa(q, k, v, w, idx, 0.0, S, None)
    ref = orc.sparse_attn(q, k, v, w.repeat_interleave(QX, 1).repeat_interleave(2, 2),
                          idx.repeat_interleave(QX, 1), chunk_size=S, mask_last_token=False)
    assert torch.allclose(o0, ref, atol=1e-6)


def test_swa_brute_force(orc):
    torch.manual_seed(11)
    B, L, HQ, H, D, S, W = 1, 40, 2, 1, 8, 8, 3
    q, k, v = torch.randn(B, L, HQ, D), torch.randn(B, L, H, D), torch.randn(B, L, H, D)
    o, lse = orc.swa(q, k, v, window_size=W, chunk_size=S)
    for t in (0, 7, 8, 9, 23, 39):
        start = ((t - W + 1) // S) * S
        toks = [j for j in range(max(start, 0), t + 1) if (j + 1) % S != 0]
        if not toks:
            assert lse[0, t, 0] == float("-inf")
            continue
        s = torch.stack([torch.dot(q[0, t, 0], k[0, j, 0]) for j in toks]) / math.sqrt(D)
        assert lse[0, t, 0].item() == pytest.approx(torch.logsumexp(s, 0).item(), abs=1e-5)
        assert torch.allclose(o[0, t, 0], torch.softmax(s, 0) @ v[0, toks, 0], atol=1e-5)


def test_swa_reduces_to_sdpa_and_positions(orc):
    """Without chunk expansion and landmark mask the window is a plain banded causal mask
    (F.scaled_dot_product_attention); with a cache, the queries are the last Lq positions and
    a truncated cache only shifts absolute positions (brute force)."""
    import torch.nn.functional as F
    torch.manual_seed(13)
    B, L, HQ, H, D, W = 1, 50, 2, 2, 8, 7
    q, k, v = torch.randn(B, L, HQ, D), torch.randn(B, L, H, D), torch.randn(B, L, H, D)
    o, lse = orc.swa(q, k, v, window_size=W, chunk_size=16, mask_lmk=False, expand_to_chunk=False)
    i, j = torch.arange(L).view(L, 1), torch.arange(L).view(1, L)
    band = (j <= i) & (j >= i - W + 1)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                         attn_mask=band).transpose(1, 2)
    assert torch.allclose(o, ref, atol=1e-5)
    # inference: 5 queries at the end of a cache of 50 keys whose first key is position 11
    S, kv0, Lq = 8, 11, 5
    o2, lse2 = orc.swa(q[:, -Lq:], k, v, window_size=W, chunk_size=S, kv_start=kv0)
    for t in range(Lq):
        pos = kv0 + L - Lq + t
        start = ((pos - W + 1) // S) * S
        toks = [jj for jj in range(L) if start <= kv0 + jj <= pos and (kv0 + jj + 1) % S != 0]
        sc = torch.stack([torch.dot(q[0, L - Lq + t, 1], k[0, jj, 1]) for jj in toks]) / math.sqrt(D)
        assert lse2[0, t, 1].item() == pytest.approx(torch.logsumexp(sc, 0).item(), abs=1e-5)
        assert torch.allclose(o2[0, t, 1], torch.softmax(sc, 0) @ v[0, toks, 1], atol=1e-5)


def test_inter_chunk_softmax(orc):
    torch.manual_seed(12)
    B, L, HQ, H, K, N = 1, 6, 4, 2, 3, 5
    scores = torch.randn(B, L, HQ, K)
    lse = torch.randn(B, L, HQ)
    idx = torch.randint(0, N, (B, L, H, K), dtype=torch.int32)
    pb = torch.randn(B, N, HQ)
    w = orc.inter_chunk_softmax(scores, lse, pb, idx)
    t, hq = 4, 3
    row = torch.cat([scores[0, t, hq] + pb[0, idx[0, t, hq // 2].long(), hq], lse[0, t, hq:hq + 1]])
    assert torch.allclose(w[0, t, hq], torch.softmax(row, 0), atol=1e-6)
    w1 = orc.inter_chunk_softmax(scores, lse, softmax1=True)
    assert w1.shape[-1] == K + 2 and torch.allclose(w1.sum(-1), torch.ones(B, L, HQ))


def test_rope_is_a_rotation(orc):
    """rope == x*cos + rotate_half(x)*sin for tables with equal halves; angle 0 is the identity,
    90 degrees maps (x1, x2) to (-x2, x1), angles add, pair norms are preserved."""
    torch.manual_seed(21)
    B, L, H, D = 2, 5, 3, 8
    x = torch.randn(B, L, H, D)
    ang = torch.rand(L, D // 2) * 6.0
    ang2 = torch.rand(L, D // 2) * 6.0
    full = lambda a: (torch.cat([a.cos(), a.cos()], -1), torch.cat([a.sin(), a.sin()], -1))
    cos, sin = full(ang)
    out = orc.rope(x, cos, sin)
    rot_half = torch.cat([-x[..., D // 2:], x[..., :D // 2]], -1)
    assert torch.allclose(out, x * cos.view(1, L, 1, D) + rot_half * sin.view(1, L, 1, D), atol=1e-6)
    assert torch.allclose(out, orc.rope(x, cos, sin, lo_only=True), atol=0)  # equal halves: same thing
    z = torch.zeros(L, D // 2)
    assert torch.equal(orc.rope(x, *full(z)), x)
    assert torch.allclose(orc.rope(x, *full(z + math.pi / 2)), rot_half, atol=1e-6)
    assert torch.allclose(orc.rope(out, *full(ang2)), orc.rope(x, *full(ang + ang2)), atol=1e-5)
    n_in = x[..., :D // 2] ** 2 + x[..., D // 2:] ** 2
    n_out = out[..., :D // 2] ** 2 + out[..., D // 2:] ** 2
    assert torch.allclose(n_in, n_out, atol=1e-5)
    # tables whose halves differ: the single-tensor form uses each half for its own output
    c, s_ = torch.randn(L, D), torch.randn(L, D)
    o2 = orc.rope(x, c, s_)
    t, h, d = 3, 1, 2
    assert o2[1, t, h, d].item() == pytest.approx((x[1, t, h, d] * c[t, d] - x[1, t, h, d + 4] * s_[t, d]).item(), abs=1e-6)
    assert o2[1, t, h, d + 4].item() == pytest.approx((x[1, t, h, d + 4] * c[t, d + 4] + x[1, t, h, d] * s_[t, d + 4]).item(), abs=1e-6)


def test_norm_rope_pool_pieces(orc):
    """rms_norm against torch's own F.rms_norm and the unit-RMS property; rope_hf against complex
    multiplication by e^{i angle} (the two halves are real and imaginary parts) and against the fp32
    kernel formula of ``rope``; the pooled keys against a python loop."""
    torch.manual_seed(31)
    B, L, H, D, S = 2, 70, 3, 16, 8
    x = torch.randn(B, L, H, D, dtype=torch.float64)
    w = torch.rand(D, dtype=torch.float64) + 0.5
    y = orc.rms_norm(x, w, 1e-6)
    assert torch.allclose(y, torch.nn.functional.rms_norm(x, (D,), w, 1e-6), atol=1e-12)
    assert torch.allclose((y / w).pow(2).mean(-1), torch.ones(B, L, H, dtype=torch.float64), atol=1e-5)
    ang = torch.rand(L, D // 2, dtype=torch.float64) * 6.0
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1), torch.cat([ang.sin(), ang.sin()], -1)
    r = orc.rope_hf(x, cos, sin)
    z = torch.complex(x[..., :D // 2], x[..., D // 2:]) * torch.polar(torch.ones_like(ang), ang).view(1, L, 1, D // 2)
    assert torch.allclose(r, torch.cat([z.real, z.imag], -1), atol=1e-12)
    assert torch.allclose(r.float(), orc.rope(x.float(), cos.float(), sin.float()), atol=1e-5)
    out, lmk = orc.norm_rope_pool(x, w, cos, sin, S, 1e-6)
    assert torch.allclose(out, orc.rope_hf(orc.rms_norm(x, w, 1e-6), cos, sin), atol=0)
    assert lmk.shape == (B, L // S, H, D)
    for b in range(B):
        for n in range(L // S):
            want = sum(out[b, n * S + s_] for s_ in range(S)) / S
            assert torch.allclose(lmk[b, n], want, atol=1e-12)
    # without norm and rotation it is the plain chunk mean
    out2, lmk2 = orc.norm_rope_pool(x, None, None, None, S)
    assert out2 is x and torch.allclose(lmk2, orc.mean_pool(x, S).to(torch.float64), atol=1e-6)
