"""CPU checks of the boundary: the C-ABI library loads and exports every symbol the header
declares, the Python binding agrees with the header, argument errors are reported, and the
product refuses to run without the GPU library path (no CPU fallback)."""
import ctypes
import os
import re

import pytest
import torch

import __graft_entry__ as entry

HEADER = os.path.join(entry.ROOT, "include", "hils_amd.h")


def header_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(?:int|size_t)\s+(hils_\w+)\s*\(([^)]*)\)\s*;", text):
        params = [p.strip() for p in m.group(2).split(",") if p.strip() and p.strip() != "void"]
        out[m.group(1)] = params
    return out


def test_library_exports_every_declared_symbol(pkg):
    lib = ctypes.CDLL(os.path.join(entry.PKG_DIR, "libhils_amd.so"))
    fns = header_functions()
    assert len(fns) >= 12
    for name in list(fns) + ["hils_last_error"]:
        assert hasattr(lib, name), f"{name} declared in include/hils_amd.h but not exported"


def test_binding_matches_header(pkg):
    from hils_attention_amd.ops import _cabi
    fns = header_functions()
    fns.pop("hils_version")
    fns.pop("hils_sparse_attn_fwd_workspace")
    fns.pop("hils_sparse_attn_bwd_workspace")
    fns.pop("hils_topk_bwd_workspace")
    fns.pop("hils_topk_fwd_workspace")
    assert set(_cabi.SIGNATURES) == set(fns)
    for name, params in fns.items():
        argtypes = _cabi.SIGNATURES[name]
        assert len(argtypes) == len(params), name
        for p, a in zip(params, argtypes):
            if "*" in p:
                assert a is ctypes.c_void_p, (name, p)
            elif p.startswith("float"):
                assert a is ctypes.c_float, (name, p)
            else:
                assert a is ctypes.c_int, (name, p)


def test_argument_errors_are_reported_without_a_gpu(pkg):
    from hils_attention_amd.ops import _cabi
    lib = _cabi.load()
    assert lib.hils_mean_pool_fwd(None, None, 1, 64, 1, 64, 64, None) == 1
    assert b"null pointer" in lib.hils_last_error()
    buf = ctypes.c_void_p(16)
    assert lib.hils_mean_pool_fwd(buf, buf, 1, 100, 1, 64, 64, None) == 1
    assert b"multiple" in lib.hils_last_error()
    assert lib.hils_topk_fwd(buf, buf, buf, None, None, None, buf, buf, None, None, None,
                             1, 16, 4, 1, 1, 64, 1000, 64, 1, 1, 0, 0, 0.125, None) == 1
    assert b"topk" in lib.hils_last_error()
    assert lib.hils_sparse_attn_fwd(buf, buf, buf, buf, buf, None, buf, None, None, 0,
                                    1, 16, 64, 3, 2, 64, 64, 4, 4, 3, 1, 64, 0.125, 1, 0.0, None) == 1
    assert b"multiple of H" in lib.hils_last_error()


def test_no_cpu_fallback(pkg):
    q = torch.randn(1, 128, 4, 64).bfloat16()
    k = torch.randn(1, 128, 2, 64).bfloat16()
    with pytest.raises(RuntimeError, match="no CPU path"):
        pkg.chunk_mean_pool(k, 64)
    with pytest.raises(RuntimeError, match="no CPU path"):
        pkg.exact_chunk_log_z_tl(q, k, chunk_size=64, window_size=1)
    w = torch.rand(1, 128, 4, 2).bfloat16()
    idx = torch.zeros(1, 128, 2, 2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="no CPU path"):
        pkg.HiLS_block_M_head(q, k, k, w, idx)
    with pytest.raises(RuntimeError, match="no CPU path"):
        pkg.online_softmax_topk_head(q, k[:, :2], torch.zeros(1, 128, 4), 2, 64, 1)


def test_wrapper_shape_checks_mirror_the_reference(pkg):
    q = torch.randn(1, 64, 4, 64).bfloat16()
    with pytest.raises(AssertionError, match="divisible"):
        pkg.online_softmax_topk_head(q, torch.randn(1, 2, 3, 64).bfloat16(), torch.zeros(1, 64, 4), 2, 64, 1)
    with pytest.raises(AssertionError, match="when G>1"):
        pkg.online_softmax_topk_head(q, torch.randn(1, 2, 2, 64).bfloat16(), torch.zeros(1, 64, 4), 2, 64, 1, G=2)
    with pytest.raises(AssertionError, match="head_dim"):
        pkg.HiLS_block_M_head(q, torch.randn(1, 64, 2, 32).bfloat16(), q, q, q)
    with pytest.raises(AssertionError, match="shared_k"):
        pkg.chunk_attn_pool_tilelang_shared_k(torch.randn(1, 2, 8, 64).bfloat16(),
                                              torch.randn(1, 2, 64, 8, 64).bfloat16())


def test_package_does_not_import_the_oracle():
    import sys
    for root, _, files in os.walk(entry.PKG_DIR):
        for f in files:
            if f.endswith(".py"):
                text = open(os.path.join(root, f)).read()
                assert "oracle" not in text.replace("no oracle", ""), f"{f} mentions the oracle"
