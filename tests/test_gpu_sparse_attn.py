"""HIP sparse attention (forward + backward) vs the CPU oracle, through the C ABI."""
import math

import pytest
import torch
import torch.nn.functional as F

from util import LSE_TOL, assert_close_bf16, assert_close_f32, note, rand_indices

pytestmark = pytest.mark.gpu


def make_case(B, L, HQ, H, D, Dv, K, S, seed=42, extra_w=1, fill_prob=1.0, Lkv=None):
    gen = torch.Generator().manual_seed(seed)
    Lkv = Lkv or L
    q = (torch.randn(B, L, HQ, D, generator=gen)).bfloat16()
    k = (torch.randn(B, Lkv, H, D, generator=gen)).bfloat16()
    v = (torch.randn(B, Lkv, H, Dv, generator=gen)).bfloat16()
    w = torch.softmax(torch.randn(B, L, HQ, K + extra_w, generator=gen), dim=-1).bfloat16()
    idx = rand_indices(B, L, H, K, S, gen, causal=(Lkv == L), n_chunks=Lkv // S, fill_prob=fill_prob)
    return q, k, v, w, idx


def fwd_check(pkg, orc, dev, q, k, v, w, idx, S, **kw):
    o = pkg.HiLS_block_M_head(q.to(dev), k.to(dev), v.to(dev), w.to(dev), idx.to(dev),
                              block_size=S, is_training=False, **kw)
    torch.cuda.synchronize()
    okw = {}
    if "sm_scale" in kw and kw["sm_scale"] is not None:
        okw["sm_scale"] = kw["sm_scale"]
    if "mask_last_token" in kw:
        okw["mask_last_token"] = kw["mask_last_token"]
    if kw.get("slope") is not None:
        okw["slope"] = kw["slope"]
    ref = orc.sparse_attn(q, k, v, w, idx, chunk_size=S, **okw)
    assert o.dtype == torch.bfloat16
    assert_close_bf16(o, ref, "o")
    return o


SHAPES = [
    # B, L, HQ, H, D, Dv, K, S
    (1, 1024, 8, 1, 64, 64, 4, 32),   # the reference's fp32 correctness shape (hils_fwd_bwd_head.py:1045-1053)
    (2, 512, 4, 4, 64, 64, 8, 64),    # MHA, G = 1
    (1, 512, 8, 2, 128, 128, 8, 64),  # GQA 4:1, D = 128
    (1, 320, 16, 1, 64, 64, 4, 64),   # G = 16
    (1, 256, 6, 2, 64, 128, 3, 64),   # G = 3, Dv != D, K not a power of two
    (1, 200, 4, 2, 32, 32, 4, 16),    # ragged L, small chunks
]


@pytest.mark.parametrize("B,L,HQ,H,D,Dv,K,S", SHAPES)
def test_sparse_attn_fwd(pkg, orc, dev, B, L, HQ, H, D, Dv, K, S):
    note(f"sparse_attn_fwd B{B} L{L} HQ{HQ} H{H} D{D} Dv{Dv} K{K} S{S}")
    q, k, v, w, idx = make_case(B, L, HQ, H, D, Dv, K, S)
    fwd_check(pkg, orc, dev, q, k, v, w, idx, S)


def test_sparse_attn_fwd_options(pkg, orc, dev):
    q, k, v, w, idx = make_case(1, 384, 8, 2, 64, 64, 4, 64, seed=3, fill_prob=0.5)
    note("sparse_attn options: partial fill / no mask / scale / slope")
    fwd_check(pkg, orc, dev, q, k, v, w, idx, 64)
    fwd_check(pkg, orc, dev, q, k, v, w, idx, 64, mask_last_token=False)
    fwd_check(pkg, orc, dev, q, k, v, w, idx, 64, sm_scale=0.2)
    fwd_check(pkg, orc, dev, q, k, v, w, idx, 64, slope=torch.rand(8) * 0.1)


def test_sparse_attn_unsorted_and_empty(pkg, orc, dev):
    """Unsorted index rows give the same result; all-empty rows give exact zeros."""
    q, k, v, w, idx = make_case(1, 384, 4, 2, 64, 64, 4, 64, seed=4)
    o1 = fwd_check(pkg, orc, dev, q, k, v, w, idx, 64)
    perm = torch.tensor([2, 0, 3, 1])
    w2 = w.clone()
    w2[..., :4] = w[..., :4][..., perm]
    o2 = fwd_check(pkg, orc, dev, q, k, v, w2, idx[..., perm].contiguous(), 64)
    assert_close_bf16(o2, o1.float().cpu(), "permuted slots", max_abs=1e-2)
    assert torch.count_nonzero(o1[0, :64]).item() == 0  # queries of chunk 0 see no chunk


def test_sparse_attn_textbook_k1(pkg, dev):
    """K = 1, w = 1: softmax(q K_c[:63]^T) V_c[:63] = F.scaled_dot_product_attention."""
    torch.manual_seed(5)
    B, L, H, D, S = 1, 256, 2, 64, 64
    q = torch.randn(B, L, H, D).bfloat16()
    k = torch.randn(B, L, H, D).bfloat16()
    v = torch.randn(B, L, H, D).bfloat16()
    idx = torch.full((B, L, H, 1), 1, dtype=torch.int32)
    w = torch.ones(B, L, H, 1).bfloat16()
    o = pkg.HiLS_block_M_head(q.to(dev), k.to(dev), v.to(dev), w.to(dev), idx.to(dev), is_training=False)
    kc = k[:, 64:127].float().permute(0, 2, 1, 3)
    vc = v[:, 64:127].float().permute(0, 2, 1, 3)
    ref = F.scaled_dot_product_attention(q.float().permute(0, 2, 1, 3), kc, vc).permute(0, 2, 1, 3)
    assert_close_bf16(o, ref, "K=1 textbook")


def test_sparse_attn_linear_in_weights(pkg, dev):
    q, k, v, w, idx = make_case(1, 256, 4, 2, 64, 64, 4, 64, seed=6)
    args = (q.to(dev), k.to(dev), v.to(dev))
    w1 = w.to(dev)
    w2 = torch.softmax(torch.randn(w.shape), -1).bfloat16().to(dev)
    o1 = pkg.HiLS_block_M_head(*args, w1, idx.to(dev), is_training=False).float()
    o2 = pkg.HiLS_block_M_head(*args, w2, idx.to(dev), is_training=False).float()
    o3 = pkg.HiLS_block_M_head(*args, ((w1.float() + w2.float()) / 2).bfloat16(), idx.to(dev),
                               is_training=False).float()
    assert_close_bf16(o3, (o1 + o2) / 2, "linearity", max_abs=2e-2)


def test_sparse_attn_equals_dense_when_weights_are_chunk_masses(pkg, orc, dev):
    """Select every causal chunk with w = softmax(log Z_c, lse_swa): the factorised form must
    equal ordinary softmax attention over the kept tokens."""
    torch.manual_seed(7)
    B, L, HQ, H, D, S, W = 1, 512, 4, 2, 64, 64, 1
    N = L // S
    q = (torch.randn(B, L, HQ, D) * 0.5).bfloat16()
    k = (torch.randn(B, L, H, D) * 0.5).bfloat16()
    v = torch.randn(B, L, H, D).bfloat16()
    lim = orc.causal_chunk_limit(L, 0, W, S)
    idx = torch.arange(N).view(1, 1, 1, N).expand(B, L, H, N).clone()
    idx = torch.where(idx < lim.view(1, L, 1, 1), idx, torch.full_like(idx, -1)).to(torch.int32)
    log_z = orc.exact_chunk_log_z(q, k, chunk_size=S, window_size=W, mask_lmk=True)
    swa_o, lse_swa = orc.swa(q, k, v, window_size=W, chunk_size=S, mask_lmk=True)
    wts = torch.softmax(torch.cat([log_z, lse_swa.unsqueeze(-1)], -1), -1)
    o_sparse = pkg.HiLS_block_M_head(q.to(dev), k.to(dev), v.to(dev), wts.bfloat16().to(dev),
                                     idx.to(dev), is_training=False).float().cpu()
    o = o_sparse + swa_o * wts[..., N].bfloat16().float().unsqueeze(-1)
    dense, _ = orc.dense_hils_attention(q, k, v, chunk_size=S, window_size=W, indices=idx)
    assert_close_bf16(o, dense, "factorised == dense", max_abs=2e-2, rel_l2=1.5e-2)


def run_bwd(pkg, orc, dev, B, L, HQ, H, D, Dv, K, S, seed=42, **kw):
    q, k, v, w, idx = make_case(B, L, HQ, H, D, Dv, K, S, seed=seed)
    gen = torch.Generator().manual_seed(seed + 1)
    do = torch.randn(B, L, HQ, Dv, generator=gen).bfloat16()
    qd, kd, vd, wd = (t.to(dev).requires_grad_() for t in (q, k, v, w))
    o = pkg.HiLS_block_M_head(qd, kd, vd, wd, idx.to(dev), block_size=S, is_training=True, **kw)
    o.backward(do.to(dev))
    torch.cuda.synchronize()
    qf, kf, vf, wf = (t.float().requires_grad_() for t in (q, k, v, w))
    okw = {kk: vv for kk, vv in kw.items() if kk in ("sm_scale", "mask_last_token", "slope")}
    ref, lse_ref = orc.sparse_attn(qf, kf, vf, wf, idx, chunk_size=S, return_lse=True, **okw)
    ref.backward(do.float())
    assert_close_bf16(o, ref, "o")
    assert_close_bf16(qd.grad, qf.grad, "dq")
    assert_close_bf16(kd.grad, kf.grad, "dk")
    assert_close_bf16(vd.grad, vf.grad, "dv")
    # dw is defined for the first K columns of valid slots; everything else must be zero
    valid = (idx >= 0).repeat_interleave(HQ // H, dim=2)
    dw_ref = torch.zeros_like(wf.grad)
    dw_ref[..., :K] = torch.where(valid, wf.grad[..., :K], torch.zeros(()))
    assert wd.grad.dtype == torch.bfloat16
    assert_close_bf16(wd.grad, dw_ref, "dw")


BWD_SHAPES = [(1, 1024, 8, 1, 64, 64, 4, 32), (1, 384, 8, 2, 128, 128, 4, 64), (2, 256, 4, 4, 64, 64, 8, 64),
              (1, 256, 6, 2, 64, 128, 3, 64)]


@pytest.mark.parametrize("B,L,HQ,H,D,Dv,K,S", BWD_SHAPES)
def test_sparse_attn_bwd(pkg, orc, dev, B, L, HQ, H, D, Dv, K, S):
    note(f"sparse_attn_bwd B{B} L{L} HQ{HQ} H{H} D{D} Dv{Dv} K{K} S{S}")
    run_bwd(pkg, orc, dev, B, L, HQ, H, D, Dv, K, S)


def test_sparse_attn_bwd_options(pkg, orc, dev):
    note("sparse_attn_bwd options")
    run_bwd(pkg, orc, dev, 1, 256, 4, 2, 64, 64, 4, 64, seed=8, mask_last_token=False)
    run_bwd(pkg, orc, dev, 1, 256, 4, 2, 64, 64, 4, 64, seed=9, slope=torch.rand(4) * 0.1, sm_scale=0.2)
    # slope on the MFMA backward with grouped 128-wide heads and with ungrouped 64-wide ones (rows staged in LDS)
    run_bwd(pkg, orc, dev, 1, 384, 8, 2, 128, 128, 4, 64, seed=12, slope=torch.rand(8) * 0.2)
    run_bwd(pkg, orc, dev, 2, 320, 4, 4, 64, 64, 4, 64, seed=13, slope=torch.rand(4) * 0.2)
    run_bwd(pkg, orc, dev, 1, 200, 4, 2, 32, 32, 4, 16, seed=14, slope=torch.rand(4) * 0.2)  # shape-generic kernel


def test_sparse_attn_per_chunk_lse(pkg, orc, dev):
    """The saved per-chunk LSE (log2 domain) equals logsumexp of the 63 masked logits."""
    from hils_attention_amd.ops import _cabi
    q, k, v, w, idx = make_case(1, 256, 4, 2, 64, 64, 4, 64, seed=10)
    B, L, HQ, D = q.shape
    o = torch.empty(B, L, HQ, 64, dtype=torch.bfloat16, device=dev)
    lse = torch.empty(B, L, HQ, 4, dtype=torch.float32, device=dev)
    t = [x.to(dev) for x in (q, k, v, w, idx)]
    _cabi.call("hils_sparse_attn_fwd", *[_cabi.ptr(x) for x in t], None, None, _cabi.ptr(o), _cabi.ptr(lse), None, 0, 0,
               B, L, L, HQ, 2, D, 64, 4, w.shape[-1], HQ, 1, 64, 1 / math.sqrt(D), 1, 0.0, 0)
    _, lse_ref = orc.sparse_attn(q, k, v, w, idx, chunk_size=64, return_lse=True)
    assert_close_f32(lse.cpu() / 1.4426950408889634, lse_ref, LSE_TOL, "per-chunk LSE")


def test_sparse_attn_inference_backward_raises(pkg, dev):
    q, k, v, w, idx = make_case(1, 128, 4, 2, 64, 64, 2, 64)
    qd = q.to(dev).requires_grad_()
    o = pkg.HiLS_block_M_head(qd, k.to(dev), v.to(dev), w.to(dev), idx.to(dev), is_training=False)
    with pytest.raises(RuntimeError):
        o.sum().backward()


def test_sparse_attn_decode_shape(pkg, orc, dev):
    """One query per sequence against a long KV cache (decode)."""
    note("sparse_attn decode B4 Lq1 Lkv4096")
    q, k, v, w, idx = make_case(4, 1, 8, 2, 128, 128, 8, 64, seed=12, Lkv=4096)
    fwd_check(pkg, orc, dev, q, k, v, w, idx, 64)


@pytest.mark.parametrize("B,HQ,H,D,K,Lkv", [(32, 32, 8, 128, 32, 4096), (64, 8, 4, 64, 16, 2048),
                                            (256, 4, 1, 128, 24, 2048)])
def test_sparse_attn_decode_one_workgroup_per_row(pkg, orc, dev, B, HQ, H, D, K, Lkv):
    """Decode with a multiple of 256 (query, KV head) rows: one workgroup per row,
    slots spread over its wavefronts and summed in LDS (no split over workgroups)."""
    note(f"sparse_attn decode rows B{B} HQ{HQ} H{H} D{D} K{K} Lkv{Lkv}")
    q, k, v, w, idx = make_case(B, 1, HQ, H, D, D, K, 64, seed=13, Lkv=Lkv, fill_prob=0.9)
    fwd_check(pkg, orc, dev, q, k, v, w, idx, 64)


@pytest.mark.parametrize("B,Lq,HQ,H,D,K,Lkv,mask_last", [
    (3, 1, 16, 2, 64, 5, 2048, True),       # 8 query heads per KV head, fewer slots than wavefronts
    (2, 2, 32, 2, 128, 40, 4096, True),     # 16 heads per KV head, two queries
    (1, 3, 8, 8, 64, 128, 16384, False),    # the most slots the row kernel takes, last token not masked
    (5, 1, 12, 4, 128, 1, 1024, True),      # 3 heads per KV head, a single slot
    (300, 1, 6, 2, 64, 16, 1024, True)])    # more rows than compute units
def test_sparse_attn_decode_group_sizes_and_slot_counts(pkg, orc, dev, B, Lq, HQ, H, D, K, Lkv, mask_last):
    """The decode kernel at its other group sizes (up to 16 query heads in the matrix columns), slot
    counts (1 ... 128) and workgroup layouts (slots split over workgroups / one workgroup per row)."""
    note(f"sparse_attn decode B{B} Lq{Lq} HQ{HQ} H{H} D{D} K{K} Lkv{Lkv}")
    q, k, v, w, idx = make_case(B, Lq, HQ, H, D, D, K, 64, seed=14, Lkv=Lkv, fill_prob=0.85)
    fwd_check(pkg, orc, dev, q, k, v, w, idx, 64, mask_last_token=mask_last)


@pytest.mark.parametrize("B,L,HQ,H,D,Dv,K", [(1, 1024, 8, 2, 128, 128, 8), (2, 512, 4, 4, 64, 64, 16),
                                              (1, 700, 16, 1, 64, 128, 4), (1, 512, 8, 4, 128, 64, 32),
                                              (1, 300, 16, 2, 64, 64, 8),
                                              # query blocks with fewer 16-byte query pieces than the workgroup
                                              # stages per round, D = 128 with Dv = 64 (the staged queries fill
                                              # the output tile exactly) and the other head-dim pairs
                                              (2, 128, 4, 2, 128, 64, 8), (1, 256, 8, 4, 128, 64, 16),
                                              (3, 192, 8, 8, 128, 64, 4), (1, 128, 16, 4, 64, 128, 8),
                                              # an odd number of weight elements: the tensor's last one has no aligned dword
                                              (1, 129, 3, 3, 64, 64, 8), (1, 67, 1, 1, 64, 64, 4)])
def test_sparse_attn_mfma_path_matches_generic_path(pkg, orc, dev, B, L, HQ, H, D, Dv, K):
    """The chunk-regrouped MFMA kernel (workspace given) against the shape-generic kernel
    (workspace NULL) and the oracle, output and per-chunk LSE, through the C ABI."""
    from hils_attention_amd.ops import _cabi
    note(f"sparse_attn mfma-vs-generic B{B} L{L} HQ{HQ} H{H} D{D} Dv{Dv} K{K}")
    q, k, v, w, idx = make_case(B, L, HQ, H, D, Dv, K, 64, seed=21, fill_prob=0.8)
    t = [x.to(dev) for x in (q, k, v, w, idx)]
    outs = []
    ws = _cabi.sparse_attn_fwd_workspace(dev, B, L, L, HQ, H, D, Dv, K, HQ, 1, 64, 0.0)
    assert ws is not None, "this shape must be covered by the MFMA path"
    for use_ws in (False, True):
        o = torch.empty(B, L, HQ, Dv, dtype=torch.bfloat16, device=dev)
        lse = torch.empty(B, L, HQ, K, dtype=torch.float32, device=dev)
        _cabi.call("hils_sparse_attn_fwd", *[_cabi.ptr(x) for x in t], None, None, _cabi.ptr(o), _cabi.ptr(lse),
                   _cabi.ptr(ws) if use_ws else None, _cabi.nbytes(ws), 0,
                   B, L, L, HQ, H, D, Dv, K, w.shape[-1], HQ, 1, 64, 1 / math.sqrt(D), 1, 0.0, 0)
        torch.cuda.synchronize()
        outs.append((o.cpu(), lse.cpu()))
    ref, lse_ref = orc.sparse_attn(q, k, v, w, idx, chunk_size=64, return_lse=True)
    for name, (o, lse) in zip(("generic", "mfma"), outs):
        assert_close_bf16(o, ref, f"{name} o")
        assert_close_f32(lse / 1.4426950408889634, lse_ref, LSE_TOL, f"{name} lse")
    assert_close_bf16(outs[1][0], outs[0][0].float(), "mfma vs generic", max_abs=1e-2, rel_l2=5e-3)


@pytest.mark.parametrize("B,L,HQ,H,D,Dv,K,mask_last", [(1, 1100, 8, 2, 128, 128, 6, 1), (2, 640, 4, 4, 64, 64, 16, 1),
                                                        (1, 700, 16, 1, 64, 128, 4, 0), (1, 2048, 8, 4, 128, 64, 32, 1)])
def test_sparse_attn_bwd_mfma_path_matches_generic_path(pkg, dev, B, L, HQ, H, D, Dv, K, mask_last):
    """The MFMA backward (inverse index + chunk-major dK/dV kernel + query-block-major dQ/dW
    kernel; workspace given) against the shape-generic backward (workspace NULL), through the
    C ABI: ragged lengths, partly filled index rows, extra weight columns, many rows per chunk."""
    from hils_attention_amd.ops import _cabi
    note(f"sparse_attn bwd mfma-vs-generic B{B} L{L} HQ{HQ} H{H} D{D} Dv{Dv} K{K} mask{mask_last}")
    q, k, v, w, idx = make_case(B, L, HQ, H, D, Dv, K, 64, seed=31, fill_prob=0.8)
    gen = torch.Generator().manual_seed(32)
    do = torch.randn(B, L, HQ, Dv, generator=gen).bfloat16()
    NW = w.shape[-1]
    t = [x.to(dev) for x in (q, k, v, w, idx)]
    o = torch.empty(B, L, HQ, Dv, dtype=torch.bfloat16, device=dev)
    lse = torch.empty(B, L, HQ, K, dtype=torch.float32, device=dev)
    scale = 1 / math.sqrt(D)
    _cabi.call("hils_sparse_attn_fwd", *[_cabi.ptr(x) for x in t], None, None, _cabi.ptr(o), _cabi.ptr(lse), None, 0, 0,
               B, L, L, HQ, H, D, Dv, K, NW, HQ, 1, 64, scale, mask_last, 0.0, 0)
    ws = _cabi.sparse_attn_bwd_workspace(dev, B, L, L, HQ, H, D, Dv, K, HQ, 1, 64, 0.0)
    assert ws is not None, "this shape must be covered by the MFMA backward"
    res = []
    for use_ws, kv16 in ((False, 0), (True, 0), (True, 1)):  # kv16: dk / dv written once as bf16
        dq = torch.empty_like(t[0])
        if kv16:
            dk, dv = torch.full_like(t[1], float("nan")), torch.full_like(t[2], float("nan"))
        else:
            dk = torch.zeros(t[1].shape, dtype=torch.float32, device=dev)
            dv = torch.zeros(t[2].shape, dtype=torch.float32, device=dev)
        dw = torch.zeros(B, L, HQ, NW, dtype=torch.float32, device=dev)
        _cabi.call("hils_sparse_attn_bwd", *[_cabi.ptr(x) for x in t], None, _cabi.ptr(lse), _cabi.ptr(do.to(dev)),
                   _cabi.ptr(dq), _cabi.ptr(dk), _cabi.ptr(dv), _cabi.ptr(dw), _cabi.ptr(ws) if use_ws else None, _cabi.nbytes(ws),
                   B, L, L, HQ, H, D, Dv, K, NW, HQ, 1, 64, scale, mask_last, 0.0, None, None, 0, kv16)
        torch.cuda.synchronize()
        res.append([x.float().cpu() for x in (dq, dk, dv, dw)])
    for name, a, b in zip(("dq", "dk", "dv", "dw"), res[1], res[0]):
        assert_close_bf16(a, b, f"{name} mfma vs generic")
    for name, a, b in zip(("dk", "dv"), res[2][1:3], res[1][1:3]):
        assert torch.isfinite(a).all(), f"{name}: the bf16 output mode must write every element"
        assert_close_bf16(a, b.bfloat16().float(), f"{name} written as bf16 vs accumulated in fp32")
    assert torch.count_nonzero(res[1][3][..., K:]).item() == 0  # weight columns beyond K get no gradient


@pytest.mark.parametrize("B,L,HQ,H,D,Dv,K,extra_w,col", [(1, 512, 8, 2, 128, 128, 8, 1, None),   # MFMA path, column K
                                                         (2, 320, 4, 4, 64, 64, 4, 2, -2),        # softmax-1 sink column behind
                                                         (1, 200, 4, 2, 32, 32, 4, 1, None),      # shape-generic path
                                                         (8, 1, 8, 2, 128, 128, 8, 1, None)])     # decode path
def test_sparse_attn_merges_local_branch(pkg, orc, dev, B, L, HQ, H, D, Dv, K, extra_w, col):
    """HiLS_block_M_head(..., swa_o=...) returns hils_o + swa_o * weights[..., col] (the layer's
    addcmul merge) with gradients to swa_o and to that weight column, against the oracle."""
    note(f"sparse_attn + merge B{B} L{L} HQ{HQ} H{H} D{D} K{K} col{col}")
    S = 64 if D >= 64 else 16
    Lkv = L if L > 1 else 2048
    q, k, v, w, idx = make_case(B, L, HQ, H, D, Dv, K, S, seed=51, extra_w=extra_w, Lkv=Lkv)
    gen = torch.Generator().manual_seed(52)
    swa = torch.randn(B, L, HQ, Dv, generator=gen).bfloat16()
    do = torch.randn(B, L, HQ, Dv, generator=gen).bfloat16()
    train = L > 1
    qd, kd, vd, wd, sd = (t.to(dev).requires_grad_(train) for t in (q, k, v, w, swa))
    o = pkg.HiLS_block_M_head(qd, kd, vd, wd, idx.to(dev), block_size=S, is_training=train, swa_o=sd,
                              swa_weight_index=col)
    wcol = K if col is None else w.shape[-1] + col
    qf, kf, vf, wf, sf = (t.float().requires_grad_(train) for t in (q, k, v, w, swa))
    ref = orc.sparse_attn(qf, kf, vf, wf, idx, chunk_size=S) + sf * wf[..., wcol].unsqueeze(-1)
    assert_close_bf16(o, ref, "merged o")
    if not train:
        return
    o.backward(do.to(dev))
    ref.backward(do.float())
    assert_close_bf16(sd.grad, sf.grad, "d_swa_o")
    assert_close_bf16(qd.grad, qf.grad, "dq")
    assert_close_bf16(kd.grad, kf.grad, "dk")
    assert_close_bf16(vd.grad, vf.grad, "dv")
    valid = (idx >= 0).repeat_interleave(HQ // H, dim=2)
    dw_ref = torch.zeros_like(wf.grad)
    dw_ref[..., :K] = torch.where(valid, wf.grad[..., :K], torch.zeros(()))
    dw_ref[..., wcol] = wf.grad[..., wcol]
    assert_close_bf16(wd.grad, dw_ref, "dw (slots and the local branch's column)")


@pytest.mark.parametrize("B,L,HQ,H,D,K,S,slope", [(1, 1024, 8, 1, 64, 4, 32, False),   # the reference's own fp32 test shape
                                                  (2, 384, 8, 2, 128, 6, 64, True)])
def test_sparse_attn_fp32_mode(pkg, orc, dev, B, L, HQ, H, D, K, S, slope):
    """dtype="float32": fp32 tensors in and out, everything computed in fp32.  The reference runs its
    fp32 correctness test in this mode (ops/hils_fwd_bwd_head.py:1045-1126: B1 L1024 H1 HQ8 D64, 4 slots,
    chunk 32; bars 5e-3 on o and 5e-3 RMS ratio on every gradient); here the bars are 1e-4 (fp32 sums in
    another order)."""
    note(f"sparse_attn fp32 mode B{B} L{L} HQ{HQ} H{H} D{D} K{K} S{S} slope={slope}")
    gen = torch.Generator().manual_seed(42)
    q = torch.randn(B, L, HQ, D, generator=gen)
    k = torch.randn(B, L, H, D, generator=gen)
    v = torch.randn(B, L, H, D, generator=gen)
    idx = rand_indices(B, L, H, K, S, gen, causal=True, n_chunks=L // S)
    logits = torch.randn(B, L, HQ, K, generator=gen)
    logits.masked_fill_(idx.repeat_interleave(HQ // H, dim=2) < 0, float("-inf"))
    w = torch.nan_to_num(torch.softmax(logits, dim=-1), 0.0)
    do = torch.randn(B, L, HQ, D, generator=gen)
    sl = torch.rand(HQ, generator=gen) * 0.2 if slope else None
    kw = {"slope": sl} if slope else {}
    qd, kd, vd, wd = (t.to(dev).requires_grad_() for t in (q, k, v, w))
    o = pkg.HiLS_block_M_head(qd, kd, vd, wd, idx.to(dev), block_size=S, mask_last_token=True, dtype="float",
                              accum_dtype="float", block_M=2, num_threads=64, is_training=True, **kw)
    assert o.dtype == torch.float32
    o.backward(do.to(dev))
    torch.cuda.synchronize()
    qf, kf, vf, wf = (t.clone().requires_grad_() for t in (q, k, v, w))
    ref = orc.sparse_attn(qf, kf, vf, wf, idx, chunk_size=S, **kw)
    ref.backward(do)

    def ratio(a, b):
        return ((a.cpu() - b).square().mean().sqrt() / b.square().mean().sqrt().clamp_min(1e-30)).item()

    worst = (o.detach().cpu() - ref.detach()).abs().max().item()
    note(f"    o max-abs {worst:.3e}")
    assert worst <= 1e-4
    for name, got, want in (("dq", qd.grad, qf.grad), ("dk", kd.grad, kf.grad), ("dv", vd.grad, vf.grad),
                            ("dw", wd.grad, wf.grad)):
        assert got.dtype == torch.float32
        r = ratio(got, want)
        note(f"    {name} RMS error ratio {r:.3e}")
        assert r <= 1e-4, name
    with pytest.raises(TypeError):
        pkg.HiLS_block_M_head(qd.detach().bfloat16(), kd.detach(), vd.detach(), wd.detach(), idx.to(dev), block_size=S,
                              dtype="float32")
