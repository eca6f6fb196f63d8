"""ctypes binding of libhils_amd.so (the C ABI declared in include/hils_amd.h).

The library is the only compute path of this package: if it is missing or a call
fails, a RuntimeError is raised.  There is no Triton/TileLang/PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_float, c_int, c_void_p

import torch

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_DIR, "libhils_amd.so")

_P, _I, _F, _Z = c_void_p, c_int, c_float, ctypes.c_size_t

# name -> argument types, in the order of include/hils_amd.h
SIGNATURES = {
    "hils_mean_pool_fwd": [_P, _P, _I, _I, _I, _I, _I, _P],
    "hils_mean_pool_bwd": [_P, _P, _I, _I, _I, _I, _I, _P],
    "hils_attn_pool_fwd": [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "hils_attn_pool_bwd": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "hils_topk_fwd": [_P] * 11 + [_Z] + [_I] * 12 + [_F, _P],
    "hils_topk_fwd_noalloc": [_P] * 10 + [_I] * 12 + [_F, _P],
    "hils_topk_fwd_weights": [_P] * 11 + [_Z] + [_I] * 12 + [_F, _P],
    "hils_topk_fwd_weights_lse16": [_P] * 9 + [_Z] + [_I] * 11 + [_F, _P],
    "hils_topk_fwd_weights_paged": [_P] * 10 + [_I] * 12 + [_F, _I, _P],
    "hils_sparse_attn_decode_paged": [_P] * 8 + [_Z] + [_I] * 9 + [_F, _I, _P],
    "hils_decode_step": [_P] * 12 + [_I] * 11 + [_F, _F, _I, _I, _I, _I, _P],
    "hils_decode_step_paged": [_P] * 13 + [_I] * 12 + [_F, _F, _I, _I, _I, _I, _I, _P],
    "hils_topk_bwd": [_P] * 7 + [_Z] + [_I] * 8 + [_F, _P],
    "hils_sparse_attn_fwd": [_P] * 10 + [_Z] + [_I] * 13 + [_F, _I, _F, _I, _P],
    "hils_pack_kv_chunks": [_P, _P, _P, _Z, _I, _I, _I, _I, _I, _P],
    "hils_sparse_attn_bwd": [_P] * 13 + [_Z] + [_I] * 12 + [_F, _I, _F, _P, _P, _I, _I, _P],
    "hils_sparse_attn_fwd_f32": [_P] * 8 + [_I] * 12 + [_F, _I, _F, _P],
    "hils_sparse_attn_bwd_f32": [_P] * 12 + [_I] * 12 + [_F, _I, _F, _P],
    "hils_chunk_weights": [_P, _P, _I, _P, _P, _P] + [_I] * 7 + [_P],
    "hils_chunk_weights_bwd": [_P, _P, _I] + [_P] * 6 + [_I] * 7 + [_P],
    "hils_chunk_logz_fwd": [_P, _P, _P] + [_I] * 7 + [_F, _I, _P],
    "hils_chunk_logz_bwd_dq": [_P] * 5 + [_I] * 7 + [_F, _P],
    "hils_chunk_logz_bwd_dk": [_P] * 5 + [_I] * 7 + [_F, _P],
    "hils_rope": [_P] * 4 + [_I] * 7 + [_F, _P],
    "hils_norm_rope_pool_fwd": [_P] * 6 + [_I] * 6 + [_F, _P],
    "hils_norm_rope_pool_bwd": [_P] * 8 + [_I] * 6 + [_F, _P],
    "hils_swa_fwd": [_P] * 5 + [_I] * 12 + [_F, _P],
    "hils_swa_bwd": [_P] * 11 + [_I] * 10 + [_F, _P],
}

_lib = None


def load():
    """Load libhils_amd.so once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python __graft_entry__.py build` "
            "(hipcc --offload-arch=gfx950). This package has no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    lib.hils_last_error.restype = ctypes.c_char_p
    lib.hils_last_error.argtypes = []
    lib.hils_version.restype = c_int
    lib.hils_version.argtypes = []
    lib.hils_topk_fwd_workspace.restype = ctypes.c_size_t
    lib.hils_topk_fwd_workspace.argtypes = [_I] * 5
    lib.hils_topk_fwd_noalloc_max_workspace.restype = ctypes.c_size_t
    lib.hils_topk_fwd_noalloc_max_workspace.argtypes = []
    lib.hils_sparse_attn_decode_paged_workspace.restype = ctypes.c_size_t
    lib.hils_sparse_attn_decode_paged_workspace.argtypes = [_I] * 6
    lib.hils_topk_lse16_covers.restype = c_int
    lib.hils_topk_lse16_covers.argtypes = [_I] * 7
    lib.hils_decode_step_covers.restype = c_int
    lib.hils_decode_step_covers.argtypes = [_I] * 9
    lib.hils_sparse_attn_fwd_workspace.restype = ctypes.c_size_t
    lib.hils_sparse_attn_fwd_workspace.argtypes = [_I] * 11 + [_F]
    lib.hils_topk_bwd_workspace.restype = ctypes.c_size_t
    lib.hils_topk_bwd_workspace.argtypes = [_I] * 7
    lib.hils_sparse_attn_bwd_workspace.restype = ctypes.c_size_t
    lib.hils_sparse_attn_bwd_workspace.argtypes = [_I] * 11 + [_F]
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = c_int
        fn.argtypes = argtypes
    _lib = lib
    return lib


def ptr(t):
    """Device pointer of a tensor (None -> NULL)."""
    if t is None:
        return None
    return c_void_p(t.data_ptr())


def nbytes(t):
    """Size in bytes of the buffer behind a workspace tensor (None -> 0)."""
    return 0 if t is None else t.numel() * t.element_size()


def gpu_readable(t, device):
    """A contiguous tensor the kernels can read: ``t`` itself when it is contiguous in device memory
    or in pinned host memory; otherwise a contiguous copy in device memory (a copy of a pinned
    tensor made on the host would land in pageable memory, which the GPU cannot address)."""
    if t.is_contiguous() and (t.is_cuda or t.is_pinned()):
        return t
    if t.is_cuda:
        return t.contiguous()
    return t.to(device, non_blocking=True).contiguous()


def stream():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def call(name, *args):
    """Call an entry point on the current stream; raise RuntimeError on a non-zero status."""
    lib = load()
    rc = getattr(lib, name)(*args, stream())
    if rc != 0:
        msg = lib.hils_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{name} failed (status {rc}): {msg}")


def topk_fwd_workspace(device, B, L, N, h_kv, G):
    """Scratch tensor for hils_topk_fwd (None when the fused kernel needs none)."""
    n = load().hils_topk_fwd_workspace(B, L, N, h_kv, G)
    if n == 0:
        return None
    return torch.empty(n, dtype=torch.uint8, device=device)


def sparse_attn_fwd_workspace_bytes(B, L, Lkv, HQ, H, D, Dv, K, WH, q_block, S, sm_n):
    """Bytes of scratch hils_sparse_attn_fwd needs for this shape (0 = none)."""
    return int(load().hils_sparse_attn_fwd_workspace(B, L, Lkv, HQ, H, D, Dv, K, WH, q_block, S, sm_n))


def sparse_attn_fwd_workspace(device, B, L, Lkv, HQ, H, D, Dv, K, WH, q_block, S, sm_n):
    """Scratch tensor for hils_sparse_attn_fwd (None when the shape needs none)."""
    n = sparse_attn_fwd_workspace_bytes(B, L, Lkv, HQ, H, D, Dv, K, WH, q_block, S, sm_n)
    if n == 0:
        return None
    return torch.empty(n, dtype=torch.uint8, device=device)


def topk_bwd_workspace(device, B, L, N, h_kv, G, D, topk):
    """Scratch tensor for hils_topk_bwd (None when the shape needs none)."""
    n = load().hils_topk_bwd_workspace(B, L, N, h_kv, G, D, topk)
    if n == 0:
        return None
    return torch.empty(n, dtype=torch.uint8, device=device)


def sparse_attn_bwd_workspace(device, B, L, Lkv, HQ, H, D, Dv, K, WH, q_block, S, sm_n):
    """Scratch tensor for hils_sparse_attn_bwd (None when the shape needs none)."""
    n = load().hils_sparse_attn_bwd_workspace(B, L, Lkv, HQ, H, D, Dv, K, WH, q_block, S, sm_n)
    if n == 0:
        return None
    return torch.empty(n, dtype=torch.uint8, device=device)


def require_gpu_bf16(name, *tensors, pinned_ok=False):
    """Every tensor is bf16 and readable by the GPU: in device memory or, with ``pinned_ok`` (an
    offloaded KV cache), in pinned host memory, which the kernels read in place over the host link."""
    for t in tensors:
        if t is None:
            continue
        if not (t.is_cuda or (pinned_ok and t.is_pinned())):
            raise RuntimeError(f"{name}: tensors must live on the GPU (got {t.device}); "
                               "this package has no CPU path")
        if t.dtype != torch.bfloat16:
            raise TypeError(f"{name}: expected bfloat16 tensors, got {t.dtype}")
