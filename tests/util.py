"""Shared tolerances and helpers for the parity tests.

Parity bars (from the build's north star): chunk indices bit-exact when selected from
identical fp32 scores; bf16 outputs and gradients within 2e-2 max-abs (taken relative to
max(1, max|ref|), since one bf16 ulp of a value of magnitude m is m/128) and 1e-2
relative L2; fp32 LSE within 1e-4.
"""
import math
import sys

import torch

MAX_ABS = 2e-2
REL_L2 = 1e-2
LSE_TOL = 1e-4


def note(msg):
    """Print and flush what names the case before a GPU step."""
    print(msg, flush=True)
    sys.stdout.flush()


def errors(out, ref):
    out = out.detach().float().cpu()
    ref = ref.detach().float().cpu()
    finite = torch.isfinite(ref)
    assert torch.equal(torch.isfinite(out), finite), "non-finite pattern differs"
    # where both are non-finite they must be the same infinity
    assert torch.equal(out[~finite], ref[~finite]), "infinities differ"
    d = (out - ref)[finite]
    r = ref[finite]
    max_abs = d.abs().max().item() if d.numel() else 0.0
    scale = max(1.0, r.abs().max().item()) if r.numel() else 1.0
    rel = (d.norm() / r.norm().clamp_min(1e-20)).item() if r.numel() else 0.0
    return max_abs, scale, rel


def assert_close_bf16(out, ref, name="", max_abs=MAX_ABS, rel_l2=REL_L2):
    ma, scale, rel = errors(out, ref)
    # the unscaled figure, beside the bar it is held to (max_abs * max(1, max|ref|))
    note(f"    {name or 'tensor'}: max-abs {ma:.3e} (unscaled; max|ref| {scale:.3g}, bar {max_abs * scale:.3e}), "
         f"rel-L2 {rel:.3e}")
    assert ma <= max_abs * scale, f"{name}: max-abs {ma:.4e} > {max_abs} * {scale:.3g}"
    assert rel <= rel_l2, f"{name}: rel-L2 {rel:.4e} > {rel_l2}"
    return ma, rel


def assert_close_f32(out, ref, tol, name=""):
    ma, _, _ = errors(out, ref)
    assert ma <= tol, f"{name}: max-abs {ma:.4e} > {tol}"
    return ma


def bf16_round(x):
    return x.bfloat16().float()


def rand_indices(B, L, H, K, S, gen, causal=True, n_chunks=None, fill_prob=1.0):
    """Random ascending chunk indices, -1 padded, optionally causal (chunk < t // S)."""
    n_chunks = n_chunks if n_chunks is not None else L // S
    idx = torch.full((B, L, H, K), -1, dtype=torch.int32)
    for b in range(B):
        for t in range(L):
            nv = min(t // S, n_chunks) if causal else n_chunks
            for h in range(H):
                if nv <= 0:
                    continue
                n = min(K, nv)
                if fill_prob < 1.0:
                    n = int((torch.rand(1, generator=gen) * (n + 1)).item())
                sel = torch.randperm(nv, generator=gen)[:n].sort().values
                idx[b, t, h, :n] = sel.to(torch.int32)
    return idx


# ---------------------------------------------------------------------------------------------
# Synthetic inputs of the headline configurations.  bench.py loads these builders from this file, so
# the full-size parity tests and the benchmark run on the same tensors.
# ---------------------------------------------------------------------------------------------

def gpu_randn(shape, gen, dev, scale=None, chunk=1 << 26):
    """bf16 N(0,1) tensor generated on the GPU in slices (no fp32 copy of the whole tensor)."""
    out = torch.empty(shape, dtype=torch.bfloat16, device=dev)
    flat = out.view(-1)
    for s in range(0, flat.numel(), chunk):
        e = min(flat.numel(), s + chunk)
        flat[s:e] = torch.randn(e - s, device=dev, generator=gen).bfloat16()
    if scale is not None:
        out.mul_(scale.to(torch.bfloat16))
    return out


def swa_lse_current_chunk(q, k, S):
    """Exact lse of the local branch for window 1: keys of the query's own chunk up to the
    query, landmark (last token of the chunk) masked.  (B,L,HQ) fp32, computed with torch."""
    B, L, HQ, D = q.shape
    H = k.shape[2]
    G = HQ // H
    N = L // S
    qc = q.view(B, N, S, H, G, D).float()
    kc = k.view(B, N, S, H, D).float()
    s = torch.einsum("bnihgd,bnjhd->bnhgij", qc, kc) / math.sqrt(D)
    i = torch.arange(S, device=q.device).view(S, 1)
    j = torch.arange(S, device=q.device).view(1, S)
    s = s.masked_fill((j > i) | (j == S - 1), float("-inf"))
    lse = torch.logsumexp(s, dim=-1)  # (B,N,H,G,S)
    return lse.permute(0, 1, 4, 2, 3).reshape(B, L, HQ).contiguous()


def prefill_inputs(dev):
    """Config 3 inputs: B1 L32768, 32 query heads / 8 KV heads, D128; q, k ~ N(0,1) times a per-head
    scale U[0.5,2] (peaked chunk scores), v ~ N(0,1) (seed 1003); lse_swa = the exact lse of the
    query's own chunk, in bf16 as the layer hands it over."""
    B, L, HQ, H, D, S = 1, 32768, 32, 8, 128, 64
    G = HQ // H
    gen = torch.Generator(device=dev).manual_seed(1003)
    hs = torch.rand(HQ, device=dev, generator=gen) * 1.5 + 0.5
    q = gpu_randn((B, L, HQ, D), gen, dev, hs.view(1, 1, HQ, 1))
    k = gpu_randn((B, L, H, D), gen, dev, hs[::G].view(1, 1, H, 1))
    v = gpu_randn((B, L, H, D), gen, dev)
    return q, k, v, swa_lse_current_chunk(q, k, S).bfloat16()


def config2_inputs(dev):
    """Config 2 inputs: B4 L8192, 16 heads MHA, D64; q, k, v ~ N(0,1) (seed 1002), lse_swa = the
    exact lse of the query's own chunk, in bf16 as the layer hands it over."""
    B, L, HQ, H, D, S = 4, 8192, 16, 16, 64, 64
    gen = torch.Generator(device=dev).manual_seed(1002)
    q = gpu_randn((B, L, HQ, D), gen, dev)
    k = gpu_randn((B, L, H, D), gen, dev)
    v = gpu_randn((B, L, H, D), gen, dev)
    return q, k, v, swa_lse_current_chunk(q, k, S).bfloat16()


def train_inputs(dev):
    """Config 5 inputs: B8 L8192, 16 heads MHA, D64; q, k, v (leaves that require grad) and the
    upstream gradient d_o ~ N(0,1) (seed 1005), lse_swa = the exact fp32 lse of the own chunk."""
    B, L, HQ, H, D, S = 8, 8192, 16, 16, 64, 64
    gen = torch.Generator(device=dev).manual_seed(1005)
    q = gpu_randn((B, L, HQ, D), gen, dev).requires_grad_()
    k = gpu_randn((B, L, H, D), gen, dev).requires_grad_()
    v = gpu_randn((B, L, H, D), gen, dev).requires_grad_()
    d_o = gpu_randn((B, L, HQ, D), gen, dev)
    return q, k, v, d_o, swa_lse_current_chunk(q.detach(), k.detach(), S)


def train_forward(pkg, q, k, v, lse_swa, keep=False):
    """The training layer's remote branch: mean pool -> top-k scores -> softmax over
    [scores, lse_swa] -> sparse attention.  Returns (o, idx), plus scores and weights with keep."""
    S, K, W = 64, 32, 1
    lmk = pkg.chunk_mean_pool(k, S)
    idx, scores = pkg.online_softmax_topk_head(q, lmk, lse_swa, K, S, W, is_training=True)
    w = pkg.chunk_weights(scores, lse_swa)
    o = pkg.HiLS_block_M_head(q, k, v, w, idx, block_size=S, is_training=True)
    return (o, idx, scores, w) if keep else (o, idx)
