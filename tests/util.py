"""Shared tolerances and helpers for the parity tests.

Parity bars (from the build's north star): chunk indices bit-exact when selected from
identical fp32 scores; bf16 outputs and gradients within 2e-2 max-abs (taken relative to
max(1, max|ref|), since one bf16 ulp of a value of magnitude m is m/128) and 1e-2
relative L2; fp32 LSE within 1e-4.
"""
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
