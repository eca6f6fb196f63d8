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
    fns.pop("hils_topk_fwd_noalloc_max_workspace")
    fns.pop("hils_sparse_attn_decode_paged_workspace")
    fns.pop("hils_decode_step_covers")
    fns.pop("hils_topk_lse16_covers")
    assert set(_cabi.SIGNATURES) == set(fns)
    for name, params in fns.items():
        argtypes = _cabi.SIGNATURES[name]
        assert len(argtypes) == len(params), name
        for p, a in zip(params, argtypes):
            if "*" in p:
                assert a is ctypes.c_void_p, (name, p)
            elif p.startswith("float"):
                assert a is ctypes.c_float, (name, p)
            elif p.startswith("size_t"):
                assert a is ctypes.c_size_t, (name, p)
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
                             0, 1, 16, 4, 1, 1, 64, 1000, 64, 1, 1, 0, 0, 0.125, None) == 1
    assert b"topk" in lib.hils_last_error()
    assert lib.hils_sparse_attn_fwd(buf, buf, buf, buf, buf, None, None, buf, None, None, 0, 0,
                                    1, 16, 64, 3, 2, 64, 64, 4, 4, 3, 1, 64, 0.125, 1, 0.0, 0, None) == 1
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


def test_topk_head_grouping_forms(pkg):
    """The accepted q / chunk-key / lse_swa forms all reduce to (B,L,h_kv,g,D) + (B,L,h_kv,g)."""
    from hils_attention_amd.ops.topk_head_softmax import _group_heads, _bias_per_group, _gumbel_rows
    B, L, N, D = 2, 8, 3, 16
    lse3 = torch.zeros(B, L, 8)
    # flat q, shared keys: groups follow the chunk keys' head count
    q, lm, lse, per = _group_heads(torch.zeros(B, L, 8, D), torch.zeros(B, N, 2, D), lse3, 1)
    assert q.shape == (B, L, 2, 4, D) and lse.shape == (B, L, 2, 4) and not per and lm.shape == (B, N, 2, D)
    # flat q, per-head keys with G given
    q, lm, lse, per = _group_heads(torch.zeros(B, L, 8, D), torch.zeros(B, N, 8, D), lse3, 4)
    assert q.shape == (B, L, 2, 4, D) and per
    # grouped q: the keys' head count decides; G > 1 regroups
    q, _, _, per = _group_heads(torch.zeros(B, L, 2, 4, D), torch.zeros(B, N, 2, D), lse3, 1)
    assert q.shape == (B, L, 2, 4, D) and not per
    q, _, _, per = _group_heads(torch.zeros(B, L, 2, 4, D), torch.zeros(B, N, 8, D), lse3, 1)
    assert q.shape == (B, L, 2, 4, D) and per
    q, _, lse, per = _group_heads(torch.zeros(B, L, 2, 4, D), torch.zeros(B, N, 8, D), lse3.view(B, L, 2, 4), 2)
    assert q.shape == (B, L, 4, 2, D) and lse.shape == (B, L, 4, 2) and per
    # chunk keys with a multiple of q's head dim are split into heads
    q, lm, _, per = _group_heads(torch.zeros(B, L, 8, D), torch.zeros(B, N, 1, 2 * D), lse3, 1)
    assert lm.shape == (B, N, 2, D) and q.shape == (B, L, 2, 4, D)
    with pytest.raises(AssertionError, match="must be h_kv"):
        _group_heads(torch.zeros(B, L, 2, 4, D), torch.zeros(B, N, 3, D), lse3, 1)
    with pytest.raises(AssertionError, match="divisible by q D"):
        _group_heads(torch.zeros(B, L, 8, D), torch.zeros(B, N, 2, D + 8), lse3, 1)
    # bias forms
    b = _bias_per_group(torch.arange(B * N * 8.0).view(B, N, 8), B, N, 2, 4, "cpu")
    assert b.shape == (B, N, 2, 4) and b.dtype == torch.float32 and b[1, 2, 1, 3] == B * N * 8 - 1
    assert _bias_per_group(None, B, N, 2, 4, "cpu") is None
    with pytest.raises(AssertionError, match="bias shape"):
        _bias_per_group(torch.zeros(B, N, 7), B, N, 2, 4, "cpu")
    with pytest.raises(AssertionError, match="bias must be"):
        _bias_per_group(torch.zeros(B, N), B, N, 2, 4, "cpu")
    # Gumbel noise: off, given, drawn; training only
    assert _gumbel_rows(False, None, True, 8, N, "cpu") is None
    g = torch.randn(1, 1, 8, N)
    assert torch.equal(_gumbel_rows(False, g, True, 8, N, "cpu"), g)
    d = _gumbel_rows(True, None, True, 8, N, "cpu")
    assert d.shape == (1, 1, 8, N) and torch.isfinite(d).all()
    with pytest.raises(AssertionError, match="training"):
        _gumbel_rows(True, None, False, 8, N, "cpu")
    with pytest.raises(AssertionError, match="gumbel_noise shape"):
        _gumbel_rows(False, torch.zeros(1, 1, 4, N), True, 8, N, "cpu")


def test_drop_in_route_imports_in_a_fresh_interpreter():
    """With only the package directory on sys.path, every module the reference's layer imports
    (`from ops.X import Y`, `from utils.hils_cache_utils import HiLSDynamicLayer`) resolves."""
    import subprocess
    import sys
    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "from ops.hils_fwd_bwd_head import HiLS_block_M_head, prepare_kv_workspace\n"
        "from ops.topk_head_softmax import online_softmax_topk_head, SoftmaxTopKMaxPooling_Fused\n"
        "from ops.chunk_attn_pool_tilelang import chunk_attn_pool_tilelang, chunk_attn_pool_tilelang_shared_k, chunk_mean_pool\n"
        "from ops.exact_chunk_log_z_tilelang import exact_chunk_log_z_tl\n"
        "from ops.hsa_triton import HSA\n"
        "from ops.flex_attn_tilelang import flex_attn_tl, flex_attn_tl_two_phase\n"
        "from ops.rope_tilelang_fp32 import rope_rotary_pos_emb, single_tensor_rope_autograd\n"
        "from ops.hils_glue import chunk_weights, topk_chunk_weights\n"
        "from utils.hils_cache_utils import HiLSDynamicLayer\n"
        "print('imports ok')\n" % entry.PKG_DIR)
    res = subprocess.run([sys.executable, "-c", code], cwd="/tmp", capture_output=True, text=True, timeout=300)
    assert res.returncode == 0 and "imports ok" in res.stdout, res.stderr


def test_short_or_foreign_kv_workspace_is_rejected(pkg):
    """A packed-K/V workspace built for a shorter call must not reach the kernel."""
    from hils_attention_amd.ops import _cabi
    from hils_attention_amd.ops.hils_fwd_bwd_head import _check_kv_workspace
    small = _cabi.sparse_attn_fwd_workspace_bytes(1, 1024, 1024, 8, 2, 128, 128, 8, 8, 1, 64, 0.0)
    large = _cabi.sparse_attn_fwd_workspace_bytes(1, 4096, 4096, 8, 2, 128, 128, 8, 8, 1, 64, 0.0)
    assert 0 < small < large
    cpu = torch.device("cpu")
    _check_kv_workspace(torch.empty(large, dtype=torch.uint8), large, cpu, "ok")
    with pytest.raises(ValueError, match="at least"):
        _check_kv_workspace(torch.empty(small, dtype=torch.uint8), large, cpu, "short")
    with pytest.raises(ValueError, match="uint8"):
        _check_kv_workspace(torch.empty(large, dtype=torch.int8), large, cpu, "dtype")
    with pytest.raises(ValueError, match="kv_workspace"):
        _check_kv_workspace(torch.empty(large, dtype=torch.uint8), large, torch.device("meta"), "device")


def test_short_workspace_is_rejected_by_the_c_abi(pkg):
    """Every entry point that takes a workspace also takes its size in bytes and rejects a buffer
    shorter than its *_workspace(...) query before anything is launched (no GPU needed: the check
    comes first; the pointers are never dereferenced on the host)."""
    from hils_attention_amd.ops import _cabi
    lib = _cabi.load()
    buf = ctypes.c_void_p(256)
    B, L, HQ, H, D, K, S = 1, 4096, 8, 2, 128, 8, 64
    need = lib.hils_sparse_attn_fwd_workspace(B, L, L, HQ, H, D, D, K, HQ, 1, S, 0.0)
    assert need > 0
    rc = lib.hils_sparse_attn_fwd(buf, buf, buf, buf, buf, None, None, buf, None, buf, need - 1, 1,
                                  B, L, L, HQ, H, D, D, K, K + 1, HQ, 1, S, 0.088, 1, 0.0, 0, None)
    assert rc == 1 and b"shorter" in lib.hils_last_error()
    rc = lib.hils_pack_kv_chunks(buf, buf, buf, 1024, B, L, H, D, D, None)
    assert rc == 1 and b"shorter" in lib.hils_last_error()
    need_b = lib.hils_sparse_attn_bwd_workspace(B, L, L, HQ, H, D, D, K, HQ, 1, S, 0.0)
    assert need_b > 0
    rc = lib.hils_sparse_attn_bwd(buf, buf, buf, buf, buf, None, buf, buf, buf, buf, buf, buf, buf, need_b - 1,
                                  B, L, L, HQ, H, D, D, K, K + 1, HQ, 1, S, 0.088, 1, 0.0, None, None, 0, 0, None)
    assert rc == 1 and b"shorter" in lib.hils_last_error()
    N, h_kv, G = L // S, H, HQ // H
    need_t = lib.hils_topk_fwd_workspace(B, L, N, h_kv, G)
    assert need_t > 0
    rc = lib.hils_topk_fwd(buf, buf, buf, None, None, None, buf, buf, None, None, buf, need_t - 1,
                           B, L, N, h_kv, G, D, K, S, 1, 1, 0, 0, 0.088, None)
    assert rc == 1 and b"shorter" in lib.hils_last_error()
    rc = lib.hils_topk_fwd_weights(buf, buf, buf, None, None, None, None, buf, buf, buf, buf, need_t - 1,
                                   B, L, N, h_kv, G, D, K, S, 1, 1, 0, 0, 0.088, None)
    assert rc == 1 and b"shorter" in lib.hils_last_error()
    need_tb = lib.hils_topk_bwd_workspace(B, L, N, h_kv, 3, D, K)   # G = 3: the inverse-index kernels
    assert need_tb > 0
    rc = lib.hils_topk_bwd(buf, buf, buf, buf, buf, buf, buf, need_tb - 1, B, L, N, h_kv, 3, D, K, 0, 0.088, None)
    assert rc == 1 and b"shorter" in lib.hils_last_error()
