"""The entry point that allocates nothing (`hils_topk_fwd_noalloc`, scratch in a device array inside
the library) against `hils_topk_fwd` with a caller-allocated workspace, through the C ABI: two calls
in a row, the second with a smaller input, on both kinds of scratch use (repacked chunk keys for a
prefill-sized call, parked logits for the two-kernel decode path)."""
import ctypes
import math

import pytest
import torch

from util import note


def _call(_cabi, name, q, lmk, lse, bias, idx, sc, ws, B, L, N, h_kv, G, D, K, off):
    args = [_cabi.ptr(q), _cabi.ptr(lmk), _cabi.ptr(lse), _cabi.ptr(bias), None, None, _cabi.ptr(idx),
            _cabi.ptr(sc), None, None]
    if name == "hils_topk_fwd":
        args += [_cabi.ptr(ws), _cabi.nbytes(ws)]
    _cabi.call(name, *args, B, L, N, h_kv, G, D, K, 64, 1, 1, off, 0, 1.0 / math.sqrt(D))


def _case(pkg, dev, B, L, N, h_kv, G, D, K, off, with_bias, seed):
    from hils_attention_amd.ops import _cabi
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, L, h_kv, G, D, generator=gen).bfloat16().to(dev)
    lmk = torch.randn(B, N, h_kv, D, generator=gen).bfloat16().to(dev)
    lse = (torch.randn(B, L, h_kv, G, generator=gen) * 2 + 3).to(dev)
    bias = torch.randn(B, N, h_kv, G, generator=gen).to(dev) if with_bias else None
    need = _cabi.load().hils_topk_fwd_workspace(B, L, N, h_kv, G)
    assert 0 < need <= _cabi.load().hils_topk_fwd_noalloc_max_workspace(), "the case must use the scratch"
    out = []
    for name in ("hils_topk_fwd", "hils_topk_fwd_noalloc"):
        idx = torch.full((B, L, h_kv, K), -7, dtype=torch.int32, device=dev)
        sc = torch.zeros((B, L, h_kv, G, K), dtype=torch.bfloat16, device=dev)
        ws = torch.empty(need, dtype=torch.uint8, device=dev) if name == "hils_topk_fwd" else None
        note(f"    {name} B{B} L{L} N{N} h_kv{h_kv} G{G} D{D} top{K} bias={with_bias}")
        _call(_cabi, name, q, lmk, lse, bias, idx, sc, ws, B, L, N, h_kv, G, D, K, off)
        torch.cuda.synchronize()
        out.append((idx, sc))
    assert torch.equal(out[0][0], out[1][0]), "indices differ"
    assert torch.equal(out[0][1].view(torch.int16), out[1][1].view(torch.int16)), "scores differ"
    assert (out[1][0] >= -1).all()


@pytest.mark.gpu
def test_no_alloc_topk_matches_workspace_entry_point(pkg, dev):
    note("hils_topk_fwd_noalloc vs hils_topk_fwd")
    # prefill-sized: the chunk keys are repacked into the scratch; then a smaller call
    _case(pkg, dev, 1, 4096, 64, 8, 4, 128, 16, 0, False, 5)
    _case(pkg, dev, 1, 2048, 32, 8, 2, 64, 8, 0, False, 6)
    # decode with a bias: logits parked in the scratch between two kernels; then a smaller call
    _case(pkg, dev, 4, 1, 2048, 8, 4, 128, 32, 2048 * 64 - 1, True, 7)
    _case(pkg, dev, 2, 1, 512, 4, 4, 64, 16, 512 * 64 - 1, True, 8)


def test_no_alloc_topk_rejects_oversize(pkg):
    from hils_attention_amd.ops import _cabi
    lib = _cabi.load()
    buf = ctypes.c_void_p(16)
    cap = lib.hils_topk_fwd_noalloc_max_workspace()
    assert cap == 8 << 20
    B, L, N, h_kv, G = 64, 1, 16384, 8, 4
    assert lib.hils_topk_fwd_workspace(B, L, N, h_kv, G) > cap
    rc = lib.hils_topk_fwd_noalloc(buf, buf, buf, None, None, None, buf, buf, None, None,
                                   B, L, N, h_kv, G, 128, 32, 64, 1, 1, N * 64 - 1, 0, 0.1, None)
    assert rc == 1 and b"built-in buffer" in lib.hils_last_error()
