"""HIP top-k chunk selection vs the CPU oracle, through the C ABI.

Index parity is bit-exact: the kernel exports the fp32 selection logits and lse_total it
selected from, and the oracle's selection rule applied to those must give identical
indices.  The logits themselves (bf16 MFMA, fp32 accumulation) are checked against the
oracle's fp32 einsum within 1e-3.  Shapes follow the reference's in-file tests
(ops/topk_head_softmax.py:1807-1816, :2431-2479).
"""
import pytest
import torch

from util import assert_close_bf16, assert_close_f32, note

pytestmark = pytest.mark.gpu


def run_case(pkg, orc, dev, B, L, N, h_kv, G, D, topk, S, W, seed=42, q_offset=0, training=True,
             use_bias=False, use_gumbel=False, use_drop=False, per_qhead=False, lse_mode="rand",
             dup_keys=False, is_causal=True, one_kernel=False):
    note(f"topk B{B} L{L} N{N} hkv{h_kv} G{G} D{D} k{topk} S{S} W{W} off{q_offset} "
         f"bias{use_bias} gum{use_gumbel} drop{use_drop} pq{per_qhead} lse={lse_mode} dup{dup_keys}")
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, L, h_kv, G, D, generator=gen).bfloat16()
    lmk_h = h_kv * G if per_qhead else h_kv
    lmks = torch.randn(B, N, lmk_h, D, generator=gen).bfloat16()
    if dup_keys:  # identical chunk keys -> exact score ties
        lmks[:, 1::2] = lmks[:, 0::2][:, : lmks[:, 1::2].shape[1]]
    if lse_mode == "rand":
        lse_swa = torch.randn(B, L, h_kv * G, generator=gen) * 5 + 10
    elif lse_mode == "neginf":
        lse_swa = torch.full((B, L, h_kv * G), float("-inf"))
    else:
        lse_swa = torch.zeros(B, L, h_kv * G)
    bias = torch.randn(B, N, h_kv * G, generator=gen) if use_bias else None
    gumbel = None
    if use_gumbel:
        u = torch.rand(1, 1, h_kv * G, N, generator=gen).clamp_(1e-20, 1 - 1e-7)
        gumbel = -torch.log(-torch.log(u))
    drop = (torch.rand(B, L, N, generator=gen) < 0.3).to(torch.int32) if use_drop else None
    dbg = {"no_workspace": True} if one_kernel else {}
    q_in = q if not per_qhead else q
    idx, scores = pkg.online_softmax_topk_head(
        q_in.to(dev), lmks.to(dev), lse_swa.to(dev), topk, S, W, is_causal=is_causal,
        q_offset=q_offset, is_training=training,
        drop_mask=None if drop is None else drop.to(dev),
        bias=None if bias is None else bias.to(dev),
        gumbel_noise=None if gumbel is None else gumbel.to(dev),
        G=G if per_qhead else 1, _debug=dbg)
    torch.cuda.synchronize()
    assert idx.dtype == torch.int32 and idx.shape == (B, L, h_kv, topk)
    assert scores.dtype == torch.bfloat16 and scores.shape == (B, L, h_kv * G, topk)
    eff_off = 0 if training else q_offset
    ridx, rscores, aux = orc.online_softmax_topk_head(
        q, lmks, lse_swa, topk, S, W, is_causal=is_causal, q_offset=eff_off, drop_mask=drop,
        bias=bias, gumbel_noise=gumbel, return_aux=True)
    sel = dbg["sel_logits"].cpu()
    lt = dbg["lse_total"].cpu()
    # 1. fp32 logits and LSE against the oracle's fp32 arithmetic
    assert_close_f32(sel, aux["sel_logits"], 2e-3, "selection logits")
    assert_close_f32(lt, aux["lse_total"], 1e-3, "lse_total")
    # 2. bit-exact selection from identical fp32 scores
    lim = aux["limit"]
    idx_from_kernel_scores = orc.topk_select(sel, lt, lim, topk, drop)
    assert torch.equal(idx.cpu(), idx_from_kernel_scores), "indices not bit-exact"
    # 3. invariants: ascending, -1 tail, visible only, count
    ic = idx.cpu().long()
    valid = ic >= 0
    srt = torch.where(valid, ic, torch.full_like(ic, 1 << 30))
    assert torch.all(srt[..., 1:] >= srt[..., :-1])
    assert torch.all((srt[..., 1:] > srt[..., :-1]) | ~valid[..., 1:])
    if lim is not None:
        assert torch.all(~valid | (ic < lim.view(1, L, 1, 1)))
        cnt = torch.minimum(lim.clamp_min(0), torch.tensor(topk)).view(1, L, 1)
        if drop is None:
            assert torch.equal(valid.sum(-1), cnt.expand(B, L, h_kv))
    # 4. agreement with the oracle's own indices (its logits differ in the last bits, so
    #    near-ties may flip: require >= 99 %, the reference's own bar)
    match = (idx.cpu() == ridx).float().mean().item()
    assert match >= 0.99, f"index agreement with the fp32 oracle only {match:.4f}"
    # 5. scores: raw scaled qk at the kernel's indices
    safe = ic.clamp_min(0).unsqueeze(3).expand(-1, -1, -1, G, -1)
    want = torch.gather(aux["logits"], -1, safe).masked_fill(~valid.unsqueeze(3).expand(-1, -1, -1, G, -1),
                                                              float("-inf"))
    assert_close_bf16(scores.view(B, L, h_kv, G, topk), want, "scores")
    if (per_qhead or use_bias) and not one_kernel:
        # without the logit export other launches run (queries bucketed by visible chunks, the variants
        # without per-element options): same results
        idx2, scores2 = pkg.online_softmax_topk_head(
            q_in.to(dev), lmks.to(dev), lse_swa.to(dev), topk, S, W, is_causal=is_causal,
            q_offset=q_offset, is_training=training,
            drop_mask=None if drop is None else drop.to(dev),
            bias=None if bias is None else bias.to(dev),
            gumbel_noise=None if gumbel is None else gumbel.to(dev), G=G if per_qhead else 1)
        assert torch.equal(idx2, idx) and torch.equal(scores2, scores), "export and plain launches differ"
    return idx, scores


def test_topk_reference_shape(pkg, orc, dev):
    # (B, L, S_chunks...) of test_topk_correctness_robust, reduced L for CPU oracle time
    run_case(pkg, orc, dev, B=2, L=1024, N=16, h_kv=2, G=8, D=64, topk=16, S=64, W=64)


@pytest.mark.parametrize("G,D", [(1, 64), (2, 128), (4, 128), (8, 64), (16, 64), (3, 64)])
def test_topk_group_sizes(pkg, orc, dev, G, D):
    run_case(pkg, orc, dev, B=1, L=640, N=10, h_kv=2, G=G, D=D, topk=4, S=64, W=1)
    # and without a workspace: the kernel that reads the chunk keys as they are
    run_case(pkg, orc, dev, B=1, L=640, N=10, h_kv=2, G=G, D=D, topk=4, S=64, W=1, one_kernel=True)


@pytest.mark.parametrize("L", [999, 1023, 1100, 17])
def test_topk_ragged_lengths(pkg, orc, dev, L):
    run_case(pkg, orc, dev, B=1, L=L, N=(L + 63) // 64, h_kv=2, G=4, D=64, topk=8, S=64, W=32)


def test_topk_window_zero_and_noncausal(pkg, orc, dev):
    run_case(pkg, orc, dev, B=1, L=512, N=8, h_kv=1, G=4, D=64, topk=4, S=64, W=0)
    run_case(pkg, orc, dev, B=1, L=96, N=24, h_kv=2, G=2, D=64, topk=8, S=64, W=0, is_causal=False)


def test_topk_bias_gumbel_drop(pkg, orc, dev):
    run_case(pkg, orc, dev, B=2, L=512, N=8, h_kv=2, G=4, D=64, topk=4, S=64, W=16, use_bias=True)
    run_case(pkg, orc, dev, B=1, L=512, N=8, h_kv=2, G=4, D=64, topk=4, S=64, W=16, use_gumbel=True)
    run_case(pkg, orc, dev, B=1, L=512, N=8, h_kv=2, G=4, D=64, topk=4, S=64, W=16, use_drop=True)
    run_case(pkg, orc, dev, B=1, L=512, N=8, h_kv=2, G=2, D=128, topk=4, S=64, W=16, use_bias=True,
             use_gumbel=True, use_drop=True)


def test_topk_per_qhead_lmks(pkg, orc, dev):
    run_case(pkg, orc, dev, B=1, L=512, N=8, h_kv=2, G=4, D=64, topk=4, S=64, W=1, per_qhead=True)
    run_case(pkg, orc, dev, B=1, L=300, N=5, h_kv=1, G=2, D=128, topk=8, S=64, W=1, per_qhead=True,
             use_bias=True)
    # the one-pass kernel's form for a key per query head (G = 3, 4; N <= 512, topk <= 32): ragged query
    # counts, every bucket of visible chunks, with and without the bias, another head dim, batch > 1
    run_case(pkg, orc, dev, B=1, L=777, N=13, h_kv=2, G=4, D=128, topk=8, S=64, W=1, per_qhead=True)
    run_case(pkg, orc, dev, B=2, L=2100, N=500, h_kv=1, G=4, D=64, topk=32, S=4, W=1, per_qhead=True,
             use_bias=True, training=False)
    run_case(pkg, orc, dev, B=1, L=1030, N=260, h_kv=2, G=3, D=128, topk=16, S=4, W=3, per_qhead=True,
             use_bias=True)
    run_case(pkg, orc, dev, B=1, L=70, N=300, h_kv=3, G=4, D=64, topk=32, S=64, W=0, per_qhead=True,
             is_causal=False)


def test_topk_chunked_prefill_and_decode(pkg, orc, dev):
    # chunked prefill: q_offset=1024; decode: q_len=1, kv=2049 (reference :2431-2479)
    run_case(pkg, orc, dev, B=1, L=256, N=20, h_kv=2, G=4, D=64, topk=8, S=64, W=64, q_offset=1024,
             training=False)
    run_case(pkg, orc, dev, B=2, L=1, N=32, h_kv=2, G=4, D=128, topk=8, S=64, W=64, q_offset=2048,
             training=False)


def test_topk_many_chunks_multi_segment(pkg, orc, dev):
    # more chunks than one LDS selection segment (512): exercises the candidate carry-over
    run_case(pkg, orc, dev, B=1, L=2, N=1500, h_kv=2, G=4, D=64, topk=32, S=64, W=1,
             q_offset=1500 * 64, training=False)
    run_case(pkg, orc, dev, B=1, L=1, N=2048, h_kv=1, G=4, D=128, topk=64, S=64, W=1,
             q_offset=2048 * 64, training=False, dup_keys=True)


def test_topk_prefill_beyond_512_chunks_with_bias(pkg, orc, dev):
    """Long prefill (more chunks than the one-pass kernel holds) with the additive bias: the general
    kernel loads a block's bias together with its keys."""
    run_case(pkg, orc, dev, B=1, L=4000, N=700, h_kv=1, G=4, D=128, topk=32, S=64, W=1, q_offset=700 * 64 - 4000,
             training=False, use_bias=True)
    run_case(pkg, orc, dev, B=2, L=2500, N=530, h_kv=2, G=3, D=64, topk=16, S=64, W=1, q_offset=530 * 64 - 2500,
             training=False, use_bias=True, dup_keys=True)
    run_case(pkg, orc, dev, B=1, L=3000, N=600, h_kv=2, G=2, D=128, topk=8, S=64, W=1, q_offset=600 * 64 - 3000,
             training=False, use_bias=True)
    run_case(pkg, orc, dev, B=1, L=2000, N=520, h_kv=1, G=1, D=64, topk=8, S=64, W=0, is_causal=False,
             training=True, use_bias=True, use_gumbel=True)
    # five to eight query heads on shared keys: walked head by head
    run_case(pkg, orc, dev, B=1, L=3000, N=600, h_kv=2, G=8, D=64, topk=32, S=64, W=1, q_offset=600 * 64 - 3000,
             training=False, use_bias=True)
    run_case(pkg, orc, dev, B=1, L=2100, N=530, h_kv=1, G=6, D=128, topk=40, S=64, W=1, q_offset=530 * 64 - 2100,
             training=False, dup_keys=True)


def test_topk_prefill_beyond_512_chunks_key_per_query_head(pkg, orc, dev):
    """Long prefill with one chunk key per query head (outside the one-pass kernel: more than 512 chunks,
    more than 32 winners, noise, a drop mask): the two-pass kernel walks the heads of a KV head."""
    run_case(pkg, orc, dev, B=1, L=4000, N=700, h_kv=1, G=4, D=128, topk=32, S=64, W=1, q_offset=700 * 64 - 4000,
             training=False, per_qhead=True)
    run_case(pkg, orc, dev, B=2, L=2500, N=530, h_kv=2, G=8, D=64, topk=16, S=64, W=1, q_offset=530 * 64 - 2500,
             training=False, per_qhead=True, use_bias=True, dup_keys=True)
    run_case(pkg, orc, dev, B=1, L=3001, N=1100, h_kv=2, G=2, D=128, topk=8, S=64, W=70, q_offset=1100 * 64 - 3001,
             training=False, per_qhead=True, use_bias=True)
    run_case(pkg, orc, dev, B=1, L=1000, N=40, h_kv=1, G=3, D=64, topk=48, S=16, W=1, training=True,
             per_qhead=True, use_bias=True, use_gumbel=True, use_drop=True)
    run_case(pkg, orc, dev, B=1, L=777, N=300, h_kv=2, G=5, D=64, topk=40, S=64, W=0, is_causal=False,
             per_qhead=True)


def test_topk_one_kernel_path_many_chunks(pkg, orc, dev):
    """The one-kernel path with more chunks than a selection segment, ragged query count,
    exact ties, and every optional input (winners carried across segments)."""
    run_case(pkg, orc, dev, B=1, L=21, N=1100, h_kv=2, G=4, D=128, topk=32, S=64, W=1,
             q_offset=1100 * 64 - 21, training=False, dup_keys=True, one_kernel=True)
    run_case(pkg, orc, dev, B=2, L=13, N=700, h_kv=1, G=2, D=64, topk=64, S=64, W=0, is_causal=False,
             training=True, use_bias=True, use_gumbel=True, use_drop=True, one_kernel=True)
    run_case(pkg, orc, dev, B=1, L=9, N=530, h_kv=1, G=3, D=64, topk=16, S=64, W=0, is_causal=False,
             one_kernel=True)


@pytest.mark.parametrize("G,D,L,N,topk,W,S", [(4, 128, 2050, 33, 32, 1, 64), (2, 64, 777, 13, 8, 64, 64),
                                              (3, 128, 300, 5, 4, 1, 64), (4, 64, 40, 600, 16, 1, 64),
                                              (3, 64, 9000, 150, 9, 1, 64),
                                              # a chunk size that is no power of two (visibility by division)
                                              (4, 128, 6000, 125, 16, 1, 48), (1, 64, 5000, 50, 7, 30, 100)])
def test_topk_inference_variant_matches_export_variant(pkg, dev, G, D, L, N, topk, W, S):
    """The kernel variant without logit export / bias / noise / drop mask (the one inference
    runs) must give the same indices and scores as the exporting variant checked above."""
    note(f"topk plain-vs-export G{G} D{D} L{L} N{N} k{topk} W{W} S{S}")
    gen = torch.Generator().manual_seed(123)
    h_kv = 2
    q = torch.randn(1, L, h_kv, G, D, generator=gen).bfloat16().to(dev)
    lmks = torch.randn(1, N, h_kv, D, generator=gen).bfloat16()
    lmks[:, 1::2] = lmks[:, 0::2][:, : lmks[:, 1::2].shape[1]]  # exact ties
    lmks = lmks.to(dev)
    lse = (torch.randn(1, L, h_kv * G, generator=gen) * 3 + 5).to(dev)
    off = max(0, N * S - L)
    outs = []
    for dbg in ({"no_workspace": True}, None):
        if dbg is None:
            from hils_attention_amd.ops import _cabi
            idx = torch.empty(1, L, h_kv, topk, dtype=torch.int32, device=dev)
            sc = torch.empty(1, L, h_kv, G, topk, dtype=torch.bfloat16, device=dev)
            _cabi.call("hils_topk_fwd", _cabi.ptr(q), _cabi.ptr(lmks), _cabi.ptr(lse.view(1, L, h_kv, G).contiguous()),
                       None, None, None, _cabi.ptr(idx), _cabi.ptr(sc), None, None, None, 0, 1, L, N, h_kv, G, D,
                       topk, S, W, 1, off, 0, D ** -0.5)
        else:
            idx, sc = pkg.online_softmax_topk_head(q, lmks, lse, topk, S, W, q_offset=off,
                                                   is_training=False, _debug=dbg)
            sc = sc.view(1, L, h_kv, G, topk)
        torch.cuda.synchronize()
        outs.append((idx.cpu(), sc.float().cpu()))
    assert torch.equal(outs[0][0], outs[1][0]), "indices differ between kernel variants"
    assert torch.equal(outs[0][1], outs[1][1]), "scores differ between kernel variants"


def test_topk_tie_break_lower_index_wins(pkg, orc, dev):
    """Duplicated chunk keys give exactly equal scores; the lower index must win."""
    idx, _ = run_case(pkg, orc, dev, B=1, L=1024, N=16, h_kv=1, G=1, D=64, topk=3, S=64, W=1,
                      dup_keys=True, lse_mode="neginf")
    # with pairs (2j, 2j+1) identical and an odd k, whenever exactly one member of a pair is
    # selected it must be the even (lower) one
    ic = idx.cpu().long()
    for t in range(128, 1024, 37):
        sel = set(ic[0, t, 0][ic[0, t, 0] >= 0].tolist())
        for c in sel:
            if c % 2 == 1:
                assert (c - 1) in sel, f"t={t}: chunk {c} chosen without its identical twin {c - 1}"


def test_topk_reduces_to_torch_topk(pkg, orc, dev):
    """lse_swa = -inf and G = 1: the selection is plain top-k of the logits."""
    B, L, N, D, topk, S = 1, 768, 12, 64, 4, 64
    torch.manual_seed(9)
    q = torch.randn(B, L, 1, D).bfloat16()
    lmks = torch.randn(B, N, 1, D).bfloat16()
    lse = torch.full((B, L, 1), float("-inf"))
    dbg = {}
    idx, _ = pkg.online_softmax_topk_head(q.to(dev), lmks.to(dev), lse.to(dev), topk, S, 1, _debug=dbg)
    sel = dbg["sel_logits"].cpu().view(B, L, N)
    for t in range(0, L, 13):
        nv = t // S
        got = [c for c in idx[0, t, 0].cpu().tolist() if c >= 0]
        assert len(got) == min(topk, nv)
        if nv > 0:
            want = torch.topk(sel[0, t, :nv], min(topk, nv)).indices.sort().values.tolist()
            assert got == want


@pytest.mark.parametrize("B,L,N,h_kv,G,D,topk", [(1, 512, 8, 2, 4, 64, 4),        # dense-tile kernel, one tile
                                                 (1, 8320, 130, 1, 2, 128, 16),   # two chunk tiles, ragged last row block
                                                 (2, 200, 3, 2, 3, 64, 2)])       # group size not a divisor of 128: inverse-index kernels
def test_topk_backward(pkg, orc, dev, B, L, N, h_kv, G, D, topk):
    S = 64
    note(f"topk backward B{B} L{L} N{N} h_kv{h_kv} G{G} D{D} top{topk}")
    torch.manual_seed(11)
    for per_qhead in (False, True):
        q = torch.randn(B, L, h_kv * G, D).bfloat16()
        lmks = torch.randn(B, N, h_kv * G if per_qhead else h_kv, D).bfloat16()
        lse = torch.randn(B, L, h_kv * G)
        gs = torch.randn(B, L, h_kv * G, topk).bfloat16()
        q_d = q.to(dev).requires_grad_()
        l_d = lmks.to(dev).requires_grad_()
        idx, scores = pkg.online_softmax_topk_head(q_d, l_d, lse.to(dev), topk, S, 1,
                                                   G=G if per_qhead else 1)
        valid = (idx >= 0).repeat_interleave(G, dim=2)
        gs_d = torch.where(valid, gs.to(dev), torch.zeros_like(gs.to(dev)))
        scores.backward(gs_d)
        # oracle: autograd through a gather of the fp32 logits at the same indices
        q_f = q.float().view(B, L, h_kv, G, D).requires_grad_()
        l_f = lmks.float().requires_grad_()
        logits = orc.topk_logits(q_f, l_f)
        ic = idx.cpu().long()
        safe = ic.clamp_min(0).unsqueeze(3).expand(-1, -1, -1, G, -1)
        picked = torch.gather(logits, -1, safe)
        g_ref = gs_d.float().cpu().view(B, L, h_kv, G, topk)
        (picked * g_ref).sum().backward()
        assert_close_bf16(q_d.grad.view(B, L, h_kv, G, D), q_f.grad, f"dq pq={per_qhead}")
        assert_close_bf16(l_d.grad, l_f.grad, f"dlmk pq={per_qhead}")


def test_topk_argument_errors(pkg, dev):
    q = torch.randn(1, 64, 4, 64, device=dev).bfloat16()
    lmks = torch.randn(1, 1, 3, 64, device=dev).bfloat16()
    lse = torch.zeros(1, 64, 4, device=dev)
    with pytest.raises(AssertionError):
        pkg.online_softmax_topk_head(q, lmks, lse, 4, 64, 1)
    with pytest.raises(TypeError):
        pkg.online_softmax_topk_head(q.float(), lmks[:, :, :2].float(), lse, 4, 64, 1)
    with pytest.raises(RuntimeError):
        pkg.online_softmax_topk_head(q, lmks[:, :, :2], lse, 100, 64, 1)


def test_topk_split_path_options(pkg, orc, dev):
    """Few queries and many chunks take the two-kernel path (logits spread over workgroups,
    then selection); cover bias / Gumbel / drop mask / per-q-head keys / ragged N there."""
    run_case(pkg, orc, dev, B=2, L=3, N=600, h_kv=2, G=4, D=64, topk=16, S=64, W=64, q_offset=600 * 64,
             training=False, use_bias=True, use_drop=True)
    run_case(pkg, orc, dev, B=1, L=1, N=1000, h_kv=2, G=2, D=128, topk=8, S=64, W=1, q_offset=70000,
             training=False, per_qhead=True)
    run_case(pkg, orc, dev, B=1, L=20, N=700, h_kv=1, G=3, D=64, topk=32, S=64, W=1, q_offset=700 * 64 - 20,
             training=False, use_bias=True)
    run_case(pkg, orc, dev, B=1, L=2, N=513, h_kv=1, G=1, D=64, topk=4, S=64, W=0, is_causal=False,
             training=True, use_gumbel=True)


@pytest.mark.parametrize("B,L,N,h_kv,G,D,topk,off", [
    (16, 1, 2048, 8, 4, 128, 32, 2048 * 64), (12, 1, 1000, 8, 2, 64, 64, 1000 * 64 - 1),
    (100, 1, 300, 1, 1, 128, 8, 200 * 64), (3, 5, 4096, 8, 4, 64, 16, 4096 * 64 - 5),
    (24, 1, 777, 4, 3, 128, 32, 500 * 64 + 7),
    (40, 2, 1536, 8, 4, 128, 32, 1536 * 64 - 2),  # more rows than compute units: 8-wavefront workgroups
    (128, 1, 256, 1, 4, 64, 8, 10),           # no chunk visible yet: all -1
    (64, 2, 300, 2, 2, 128, 8, 64 * 3 + 5),   # fewer visible chunks than topk
    # five to eight query heads per KV head: eight head slots per row
    (64, 1, 2048, 2, 8, 64, 32, 2048 * 64), (20, 1, 2500, 8, 6, 128, 16, 2500 * 64 - 3),
    (300, 1, 700, 1, 5, 128, 8, 700 * 64)])
def test_topk_workgroup_per_row_path(pkg, orc, dev, B, L, N, h_kv, G, D, topk, off):
    """About one (query, KV head) row per compute unit: one 16-wavefront workgroup per row streams the
    chunk keys, keeps the logits in LDS and selects (ragged N, limits below N, exact ties)."""
    run_case(pkg, orc, dev, B=B, L=L, N=N, h_kv=h_kv, G=G, D=D, topk=topk, S=64, W=1, q_offset=off,
             training=False, dup_keys=(N == 1000))


def test_topk_workgroup_per_row_path_bias_shares_the_logit_array(pkg, orc, dev):
    """More chunks than the LDS holds logits and bias side by side for: the bias is staged in the logits'
    array and a winner's bias is read again from global memory."""
    run_case(pkg, orc, dev, B=12, L=1, N=3500, h_kv=8, G=4, D=128, topk=32, S=64, W=1, q_offset=3500 * 64 - 1,
             training=False, use_bias=True)
    run_case(pkg, orc, dev, B=100, L=1, N=4096, h_kv=1, G=3, D=64, topk=64, S=64, W=1, q_offset=4096 * 64 - 1,
             training=False, use_bias=True, dup_keys=True)
    run_case(pkg, orc, dev, B=30, L=2, N=3000, h_kv=2, G=6, D=128, topk=16, S=64, W=1, q_offset=3000 * 64 - 2,
             training=False, use_bias=True)  # (eight head slots: over the in-place limit too, the two-kernel path)


@pytest.mark.parametrize("B,L,N,h_kv,G,D,topk,bias", [(64, 1, 1500, 2, 8, 64, 32, True), (100, 1, 1024, 1, 7, 128, 16, False),
                                                     (48, 2, 600, 2, 5, 128, 8, True),
                                                     (48, 1, 2048, 2, 8, 64, 32, True)])  # bias and logits in one array
def test_topk_workgroup_per_row_path_key_per_query_head(pkg, orc, dev, B, L, N, h_kv, G, D, topk, bias):
    """The same kernel with one chunk key per query head and five to eight heads per KV head."""
    run_case(pkg, orc, dev, B=B, L=L, N=N, h_kv=h_kv, G=G, D=D, topk=topk, S=64, W=1, q_offset=N * 64 - L,
             training=False, per_qhead=True, use_bias=bias)


def test_topk_split_and_fused_paths_agree(pkg, dev):
    from hils_attention_amd.ops import _cabi
    B, L, N, h_kv, G, D, topk = 2, 4, 1024, 2, 4, 128, 32
    gen = torch.Generator().manual_seed(5)
    q = torch.randn(B, L, h_kv, G, D, generator=gen).bfloat16().to(dev)
    lmks = torch.randn(B, N, h_kv, D, generator=gen).bfloat16().to(dev)
    lse = (torch.randn(B, L, h_kv, G, generator=gen) * 5 + 10).to(dev)
    ws = _cabi.topk_fwd_workspace(dev, B, L, N, h_kv, G)
    assert ws is not None
    outs = []
    for w in (None, ws):
        idx = torch.empty(B, L, h_kv, topk, dtype=torch.int32, device=dev)
        sc = torch.empty(B, L, h_kv, G, topk, dtype=torch.bfloat16, device=dev)
        _cabi.call("hils_topk_fwd", _cabi.ptr(q), _cabi.ptr(lmks), _cabi.ptr(lse), None, None, None,
                   _cabi.ptr(idx), _cabi.ptr(sc), None, None, _cabi.ptr(w), _cabi.nbytes(w), B, L, N, h_kv, G, D, topk, 64, 1, 1,
                   N * 64, 0, D ** -0.5)
        torch.cuda.synchronize()
        outs.append((idx.cpu(), sc.float().cpu()))
    assert torch.equal(outs[0][0], outs[1][0])
    assert (outs[0][1] - outs[1][1]).abs().max().item() <= 2e-2


@pytest.mark.parametrize("L,N,h_kv,G,D,topk,dup", [
    (8192, 128, 2, 1, 64, 32, False),    # MHA, config-2-like rows (16 queries per wavefront)
    (4100, 64, 2, 2, 128, 16, False),    # G = 2, ragged length
    (8192, 128, 1, 4, 128, 32, True),    # pairs of identical chunk keys: ties at the threshold
    (4096, 64, 1, 3, 64, 5, True),       # G = 3 (one padding head row), odd k, ties
    (2048, 32, 2, 4, 64, 1, False),      # a single winner
    (32768, 512, 1, 4, 128, 32, False),  # the full 512 chunks of the headline shape, one KV head
    (16384, 256, 1, 1, 128, 31, True),   # k not a power of two, ties, G = 1
    # five to eight query heads per KV head: two wavefronts per four queries trade their heads' scores
    (8192, 128, 2, 8, 64, 32, False), (5000, 79, 1, 5, 128, 16, True), (4096, 64, 2, 7, 64, 5, True),
    (16384, 256, 1, 8, 128, 32, True),
    # two query heads per KV head: two queries a lane
    (8192, 128, 2, 2, 128, 32, True), (5000, 79, 3, 2, 64, 7, False), (32768, 512, 1, 2, 64, 32, False),
])
def test_topk_one_pass_prefill_kernel(pkg, orc, dev, L, N, h_kv, G, D, topk, dup):
    """The one-pass prefill kernel (chunk keys repacked into the workspace, up to 512 chunks and 32
    winners): logits, lse_total, bit-exact selection, order, scores, across its head groupings."""
    run_case(pkg, orc, dev, B=1, L=L, N=N, h_kv=h_kv, G=G, D=D, topk=topk, S=64, W=1, seed=61,
             dup_keys=dup, training=False)


@pytest.mark.parametrize("G,D,L,N,topk,W,S,h_kv", [
    (4, 128, 12800, 200, 32, 1, 64, 2),   # queries of the 8- and 16-block launches
    (4, 64, 32000, 500, 32, 1, 64, 1),    # all four launches
    (1, 128, 22000, 343, 32, 1, 64, 1),   # the 24-block launch without head grouping
    (3, 64, 24000, 375, 16, 1, 64, 1),    # ... and with a padding head row
    (1, 64, 9000, 250, 16, 1, 64, 2),     # 16 queries per wavefront
    (3, 128, 7000, 140, 9, 64, 64, 1),    # a padding head row, odd k, a wide window
    (4, 128, 6000, 125, 16, 1, 48, 1),    # chunk sizes that are no power of two (visibility by division)
    (1, 64, 5000, 50, 7, 30, 100, 2),
    (8, 64, 32000, 500, 32, 1, 64, 1),    # eight heads per KV head, all four launches
    (6, 128, 20000, 313, 16, 1, 64, 2), (5, 64, 7000, 140, 9, 64, 48, 1),
    (2, 128, 32000, 500, 32, 1, 64, 2), (2, 64, 9000, 250, 5, 30, 100, 1)])  # two heads per KV head
def test_topk_one_pass_kernel_launches_match_export_variant(pkg, dev, G, D, L, N, topk, W, S, h_kv):
    """The one-pass prefill kernel as inference launches it (one instantiation per range of visible
    chunk counts, no logit export) against its exporting instantiation, which the cases above check
    against the oracle; pairs of identical chunk keys put exact ties at the threshold."""
    note(f"one-pass top-k launches G{G} D{D} L{L} N{N} k{topk} W{W} S{S}")
    gen = torch.Generator().manual_seed(321)
    q = torch.randn(1, L, h_kv * G, D, generator=gen).bfloat16().to(dev)
    lmks = torch.randn(1, N, h_kv, D, generator=gen).bfloat16()
    lmks[:, 1::2] = lmks[:, 0::2][:, : lmks[:, 1::2].shape[1]]
    lmks = lmks.to(dev)
    lse = (torch.randn(1, L, h_kv * G, generator=gen) * 3 + 5).to(dev)
    off = max(0, N * S - L)
    dbg = {}
    idx0, sc0 = pkg.online_softmax_topk_head(q, lmks, lse, topk, S, W, q_offset=off, is_training=False, _debug=dbg)
    idx1, sc1 = pkg.online_softmax_topk_head(q, lmks, lse, topk, S, W, q_offset=off, is_training=False)
    assert torch.equal(idx0, idx1), "indices differ between the launches and the exporting variant"
    assert torch.equal(sc0.view(torch.int16), sc1.view(torch.int16)), "scores differ"
    lim = torch.div(torch.arange(L, device=dev) + off - W + 1, S, rounding_mode="floor").clamp(0, N)
    assert torch.equal((idx1 >= 0).sum(-1), lim.clamp_max(topk).view(1, L, 1).expand(1, L, h_kv))


def test_topk_one_pass_kernel_all_scores_equal(pkg, orc, dev):
    """Every chunk key identical: all visible chunks tie, far more keys reach the lane bound than the
    compaction holds (the search over all keys runs) and the winners are the lowest indices."""
    note("one-pass top-k: all chunk keys equal")
    B, L, N, h_kv, G, D, topk, S = 1, 16384, 256, 1, 4, 128, 16, 64
    gen = torch.Generator().manual_seed(62)
    q = torch.randn(B, L, h_kv * G, D, generator=gen).bfloat16()
    lmks = torch.randn(1, 1, h_kv, D, generator=gen).bfloat16().expand(B, N, h_kv, D).contiguous()
    lse = torch.zeros(B, L, h_kv * G)
    dbg = {}
    idx, scores = pkg.online_softmax_topk_head(q.to(dev), lmks.to(dev), lse.to(dev), topk, S, 1,
                                               is_training=False, _debug=dbg)
    lim = orc.causal_chunk_limit(L, 0, 1, S)
    want = torch.arange(topk).view(1, 1, 1, topk).expand(B, L, h_kv, topk).clone()
    want = torch.where(want < lim.view(1, L, 1, 1), want, torch.full_like(want, -1)).to(torch.int32)
    assert torch.equal(idx.cpu(), want), "with all scores equal the lowest chunk indices must win"
    assert torch.equal(idx.cpu(), orc.topk_select(dbg["sel_logits"].cpu(), dbg["lse_total"].cpu(), lim, topk))


@pytest.mark.parametrize("G,D,per_qhead", [(4, 128, False), (8, 64, False), (5, 128, False), (4, 64, True), (7, 64, True)])
def test_topk_one_pass_kernel_rows_without_any_mass(pkg, orc, dev, G, D, per_qhead):
    """Rows whose lse_swa is -inf (the local branch saw no key: a landmark row with window 1) through
    the one-pass prefill kernel, both launch variants.  In the first chunk such a row sees no chunk
    either: lse_total is -inf, nothing is selected (indices -1, scores -inf) and no NaN is formed;
    later rows select from the chunk logits alone."""
    note("one-pass top-k: rows with lse_swa = -inf")
    B, L, N, h_kv, topk, S, W = 1, 4096, 64, 2, 8, 64, 1
    gen = torch.Generator().manual_seed(63)
    q = torch.randn(B, L, h_kv * G, D, generator=gen).bfloat16()
    lmks = torch.randn(B, N, h_kv * G if per_qhead else h_kv, D, generator=gen).bfloat16()
    lse = torch.randn(B, L, h_kv * G, generator=gen) * 3 + 5
    lse[:, S - 1::S] = float("-inf")   # every landmark row
    lse[:, :S:7] = float("-inf")       # and some more rows of the first chunk
    lim = orc.causal_chunk_limit(L, 0, W, S)
    outs = []
    for dbg in ({}, None):
        idx, scores = pkg.online_softmax_topk_head(q.to(dev), lmks.to(dev), lse.to(dev), topk, S, W,
                                                   is_training=False, G=G if per_qhead else 1, _debug=dbg)
        torch.cuda.synchronize()
        outs.append((idx.cpu(), scores.float().cpu()))
        assert torch.all(idx[:, :S] == -1), "rows that see no chunk must select nothing"
        assert torch.all(scores[:, :S].float() == float("-inf"))
        assert not torch.isnan(scores.float()).any()
        if dbg is not None:
            lt = dbg["lse_total"].cpu()
            assert torch.all(lt.view(B, L, -1)[:, :S][lse[:, :S] == float("-inf")] == float("-inf"))
            want = orc.topk_select(dbg["sel_logits"].cpu(), lt, lim, topk)
            assert torch.equal(idx.cpu(), want), "indices not bit-exact"
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    assert torch.equal((outs[0][0] >= 0).sum(-1), lim.clamp(0, topk).view(1, L, 1).expand(B, L, h_kv))
