"""CPU oracle for the HiLS-Attention operator stack (TEST INFRASTRUCTURE ONLY).

This module is a pure-PyTorch, CPU, fp32 restatement of the reference's own
torch references for the hot path.  It is the *checker*: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  Nothing in the shipped package imports it and it is never a
fallback for the HIP kernels.

Each function cites the reference text it restates (paths relative to the
reference repository root):

* ``mean_pool``            - models/FlashHiLS/hils_attention.py:398,436,446,460
* ``chunk_attn_pool``      - ops/chunk_attn_pool_tilelang.py:693-717 and
                             models/FlashHiLS/hils_attention.py:20-53
* ``topk_logits`` / ``topk_select`` / ``online_softmax_topk_head``
                           - ops/topk_head_softmax.py:15-154 (torch ref) with the
                             selection order of the kernel text :576-624 (strict
                             ``>`` while scanning chunks in ascending order, so
                             the lower chunk index wins a tie) and the ascending
                             index sort of :870-971; scores dtype from :1038
* ``sparse_attn``          - ops/hils_fwd_bwd_head.py:21-93 (block_q = 1) plus the
                             per-chunk log2 LSE of :459-471
* ``hsa``                  - ops/hsa_triton.py:881-919 (inline test reference) and
                             :171-193 (the ``sm_n`` denominator term)
* ``exact_chunk_log_z``    - models/NaiveBSA/naive_bsa_kernel.py:39-118 and the
                             mask of ops/exact_chunk_log_z_tilelang.py:89-107
* ``rope``                 - ops/rope_tilelang_fp32.py:48-62,125-134 (kernel arithmetic) and
                             :185-189 (the rotate-half torch formula its tests compare with)
* ``rms_norm`` / ``rope_hf`` / ``norm_rope_pool``
                           - models/FlashHiLS/modeling_qwen_hils.py:80-86 (rms_norm),
                             models/FlashHiLS/hils_attention.py:137-171 (rotate_half,
                             apply_rotary_pos_emb on tensors of the model dtype) and :314-321,
                             :479-483, :398 (the order norm -> rotation -> chunk mean)
* ``swa``                  - ops/flex_attn_tilelang.py:1355-1386 (mask definition) and
                             :108-121,155-171 (absolute positions with a cache offset)
* ``hils_layer_forward``   - models/FlashHiLS/hils_attention.py:536-623 (op order,
                             dtypes of the glue)
* ``dense_hils_attention`` - models/NaiveBSA/naive_bsa_ref.py:111-187 (dense
                             masked softmax the factorised form must equal)

Pinning status (what independent evidence each function is checked against
lives in tests/test_oracle_*.py):

* every function is pinned by closed forms, library routines
  (``F.scaled_dot_product_attention``, ``torch.distributions.Categorical``,
  ``torch.topk``) and brute force on tiny inputs, including the option branches
  (in-chunk slope of ``sparse_attn``, Gumbel noise of ``select_logits``, per-query-head
  chunk keys of ``topk_logits``), each against a pure-Python enumeration;
* the reference stores no golden vectors for this path, so none are used;
* the tie-break of ``topk_select`` is pinned only by the reference's kernel text.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

NEG_INF = float("-inf")
LOG2E = 1.4426950408889634


# ----------------------------------------------------------------------------
# chunk keys
# ----------------------------------------------------------------------------
def mean_pool(k: torch.Tensor, chunk_size: int) -> torch.Tensor:
    """lmk_k[b,n,h,:] = mean over the S tokens of chunk n (landmark included)."""
    B, L, H, D = k.shape
    N = L // chunk_size
    kc = k[:, : N * chunk_size].reshape(B, N, chunk_size, H, D).float()
    return kc.mean(dim=2)


def chunk_attn_pool(mu_q: torch.Tensor, k_chunked: torch.Tensor,
                    sm_scale: Optional[float] = None):
    """One prior query per (chunk, head) attends to the chunk's first S-1 keys.

    Returns (lmk_k fp32 (B,N,H,D), lmk_b fp32 (B,N,H), p fp32 (B,N,S,H)).
    """
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(mu_q.shape[-1])
    mu = mu_q.float()
    kf = k_chunked.float()
    logits = torch.einsum("bnhd,bnshd->bnsh", mu, kf) * sm_scale
    S = logits.shape[2]
    last = torch.zeros(S, dtype=torch.bool)
    last[-1] = True
    logits = logits.masked_fill(last.view(1, 1, S, 1), NEG_INF)
    p = F.softmax(logits, dim=2)
    lmk_k = torch.einsum("bnsh,bnshd->bnhd", p, kf)
    log_p = F.log_softmax(logits, dim=2)
    log_p = torch.where(torch.isfinite(log_p), log_p, torch.zeros((), dtype=log_p.dtype))
    lmk_b = -(p * log_p).sum(dim=2)
    return lmk_k, lmk_b, p


# ----------------------------------------------------------------------------
# top-k chunk selection
# ----------------------------------------------------------------------------
def causal_chunk_limit(L: int, q_offset: int, window_size: int, block_size: int) -> torch.Tensor:
    """Number of visible chunks per query: chunk c is visible iff c < limit[t]."""
    t = torch.arange(L) + q_offset
    if window_size > 0:
        return torch.div(t - window_size + 1, block_size, rounding_mode="floor")
    return torch.div(t, block_size, rounding_mode="floor")


def topk_logits(q: torch.Tensor, lmks: torch.Tensor, sm_scale: Optional[float] = None) -> torch.Tensor:
    """Raw scaled logits sm_scale * <q, lmk> in fp32, shape (B, L, h_kv, G, N).

    q is (B, L, h_kv, G, D); lmks is (B, N, h_kv, D) or per-q-head (B, N, h_kv*G, D).
    """
    B, L, h_kv, G, D = q.shape
    N = lmks.shape[1]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    if lmks.shape[2] == h_kv:
        lg = torch.einsum("blhgd,bshd->blhgs", q.float(), lmks.float())
    elif lmks.shape[2] == h_kv * G:
        lg = torch.einsum("blhgd,bshgd->blhgs", q.float(), lmks.float().view(B, N, h_kv, G, D))
    else:
        raise AssertionError("lmks head dim must be h_kv or h_kv*G")
    return lg * torch.tensor(sm_scale, dtype=torch.float32)


def select_logits(logits_scaled: torch.Tensor, bias: Optional[torch.Tensor],
                  gumbel_noise: Optional[torch.Tensor]) -> torch.Tensor:
    """Selection logits = scaled qk (+ bias[b,c,h,g]) (+ gumbel[h*G+g, c]), fp32.

    The additions are done in this order, one rounding each, which is what the
    HIP kernel does too, so that selection from identical fp32 logits is
    reproducible bit for bit.
    """
    B, L, h_kv, G, N = logits_scaled.shape
    x = logits_scaled
    if bias is not None:
        b = bias.float().reshape(B, N, h_kv, G).permute(0, 2, 3, 1).unsqueeze(1)
        x = x + b
    if gumbel_noise is not None:
        g = gumbel_noise.float().reshape(1, 1, h_kv, G, N)
        x = x + g
    return x


def topk_select(sel_logits: torch.Tensor, lse_total: torch.Tensor, limit: Optional[torch.Tensor],
                topk: int, drop_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Indices (B, L, h_kv, topk) int32, ascending, -1 padded.

    sel_logits (B,L,h_kv,G,N) fp32 selection logits (bias/gumbel already added),
    lse_total (B,L,h_kv,G) fp32.  Selection score of chunk c is
    max_g(sel_logits[...,g,c] - lse_total[...,g]) (one fp32 subtraction, then max);
    chunks with c >= limit[t], dropped chunks and chunks whose score is -inf or
    NaN are never selected.  Order: score descending, then chunk index ascending
    (the lower index wins a tie).
    """
    B, L, h_kv, G, N = sel_logits.shape
    norm = sel_logits - lse_total.unsqueeze(-1)
    norm = torch.where(sel_logits == NEG_INF, torch.full_like(norm, NEG_INF), norm)
    # max over g ignoring NaN the way a chain of fmaxf starting from -inf does
    norm = torch.where(torch.isnan(norm), torch.full_like(norm, NEG_INF), norm)
    score = norm.max(dim=3).values  # (B, L, h_kv, N)
    if limit is not None:
        c = torch.arange(N)
        invisible = c.view(1, N) >= limit.view(L, 1)
        score = score.masked_fill(invisible.view(1, L, 1, N), NEG_INF)
    if drop_mask is not None:
        score = score.masked_fill(drop_mask.bool().unsqueeze(2), NEG_INF)
    score = score + 0.0  # canonicalise -0.0
    # stable sort on descending score keeps ascending chunk index among equals
    order = torch.sort(score, dim=-1, descending=True, stable=True).indices
    kk = min(topk, N)
    top = order[..., :kk]
    top_score = torch.gather(score, -1, top)
    top = torch.where(top_score == NEG_INF, torch.full_like(top, N + 1000), top)
    if kk < topk:
        pad = torch.full((B, L, h_kv, topk - kk), N + 1000, dtype=top.dtype)
        top = torch.cat([top, pad], dim=-1)
    top = torch.sort(top, dim=-1).values
    top = torch.where(top >= N, torch.full_like(top, -1), top)
    return top.to(torch.int32)


def online_softmax_topk_head(q, lmks, lse_swa, topk, block_size, window_size,
                             is_causal=True, q_offset=0, drop_mask=None, sm_scale=None,
                             bias=None, gumbel_noise=None, return_aux=False):
    """Full top-k op.  q (B,L,h_kv,G,D).  Returns (indices int32 (B,L,h_kv,topk),
    scores fp32 (B,L,h_kv,G,topk) raw scaled qk, -inf where index < 0)."""
    B, L, h_kv, G, D = q.shape
    N = lmks.shape[1]
    logits = topk_logits(q, lmks, sm_scale)
    sel = select_logits(logits, bias, gumbel_noise)
    limit = causal_chunk_limit(L, q_offset, window_size, block_size) if is_causal else None
    if limit is not None:
        c = torch.arange(N)
        invisible = (c.view(1, N) >= limit.view(L, 1)).view(1, L, 1, 1, N)
        sel_m = sel.masked_fill(invisible, NEG_INF)
    else:
        sel_m = sel
    lse_hils = torch.logsumexp(sel_m, dim=-1)
    lse_total = torch.logaddexp(lse_swa.float().reshape(B, L, h_kv, G), lse_hils)
    idx = topk_select(sel_m, lse_total, limit, topk, drop_mask)
    safe = idx.clamp_min(0).long().unsqueeze(3).expand(-1, -1, -1, G, -1)
    scores = torch.gather(logits, -1, safe)
    scores = scores.masked_fill((idx < 0).unsqueeze(3).expand(-1, -1, -1, G, -1), NEG_INF)
    if return_aux:
        return idx, scores, {"logits": logits, "sel_logits": sel_m, "lse_hils": lse_hils,
                             "lse_total": lse_total, "limit": limit}
    return idx, scores


# ----------------------------------------------------------------------------
# sparse attention over selected chunks
# ----------------------------------------------------------------------------
def sparse_attn(q, k, v, weights, indices, *, chunk_size: int, sm_scale: Optional[float] = None,
                mask_last_token: bool = True, slope=None, sm_n: float = 0.0,
                q_block: int = 1, return_lse: bool = False):
    """o[t,h] = sum_k w[t,h,k] * softmax_{j in chunk idx[t,k]}(sm_scale*q.K_j) V_j.

    q (B,L,hq,D); k (B,Lkv,hkv,D); v (B,Lkv,hkv,Dv);
    indices (B, L//q_block, hkv, K) int; weights (B, L//q_block, hq or hkv, >=K).
    Index < 0 contributes nothing.  ``sm_n`` adds sm_n*exp(-max) to every
    per-chunk softmax denominator (the older HSA variant); ``q_block`` > 1 makes
    all queries of a block share one index/weight row.
    Returns o fp32 (B,L,hq,Dv) and, if asked, the per-chunk natural-log LSE
    (B,L,hq,K) (-inf for index < 0; without the sm_n term).
    """
    B, L, HQ, D = q.shape
    _, Lkv, H, _ = k.shape
    Dv = v.shape[-1]
    G = HQ // H
    K = indices.shape[-1]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    S = chunk_size
    N = Lkv // S
    kc = k[:, : N * S].reshape(B, N, S, H, D).float()
    vc = v[:, : N * S].reshape(B, N, S, H, Dv).float()
    if q_block > 1:
        indices = indices.repeat_interleave(q_block, dim=1)
        weights = weights.repeat_interleave(q_block, dim=1)
    if weights.shape[2] == H and G > 1:
        weights = weights.repeat_interleave(G, dim=2)
    valid = indices >= 0
    safe = indices.clamp_min(0).long()
    qf = q.float().view(B, L, H, G, D)
    o = torch.zeros(B, L, H, G, Dv, dtype=torch.float32)
    lse_out = torch.full((B, L, H, G, K), NEG_INF, dtype=torch.float32)
    bidx = torch.arange(B).view(B, 1, 1).expand(B, L, H)
    hidx = torch.arange(H).view(1, 1, H).expand(B, L, H)
    wv = weights[..., :K].float().view(B, L, H, G, K)
    if slope is not None:
        s_pos = torch.arange(S, dtype=torch.float32)
        dist = ((S - 2) - s_pos).clamp(min=0)
        slope_bias = -slope.float().view(H, G, 1) * dist.view(1, 1, S)
    for kk in range(K):
        ck = kc[bidx, safe[..., kk], :, hidx]  # (B,L,H,S,D)
        cv = vc[bidx, safe[..., kk], :, hidx]  # (B,L,H,S,Dv)
        s = torch.einsum("blhgd,blhsd->blhgs", qf, ck)
        if slope is not None:
            s = s + slope_bias.view(1, 1, H, G, S)
        s = s * sm_scale
        if mask_last_token:
            s[..., -1] = NEG_INF
        m = s.max(dim=-1, keepdim=True).values
        e = torch.exp(s - m)
        denom = e.sum(dim=-1, keepdim=True)
        lse = (m + torch.log(denom)).squeeze(-1)
        if sm_n != 0.0:
            denom = denom + sm_n * torch.exp(-m)
        p = e / denom
        ok = torch.einsum("blhgs,blhsd->blhgd", p, cv)
        vmask = valid[..., kk].view(B, L, H, 1, 1).float()
        o = o + ok * wv[..., kk].unsqueeze(-1) * vmask
        lse_out[..., kk] = torch.where(valid[..., kk].unsqueeze(-1), lse, torch.full_like(lse, NEG_INF))
    o = o.view(B, L, HQ, Dv)
    if return_lse:
        return o, lse_out.view(B, L, HQ, K)
    return o


def hsa(q, k, v, weights, indices, sm_n, chunk_size, sm_scale=None):
    """Older HSA variant: indices/weights (N, L//Q_X, h_kv, K) shared by a q-block and
    by the G heads of a KV head, no landmark mask, sm_n in the denominator."""
    L = q.shape[1]
    q_block = L // indices.shape[1]
    return sparse_attn(q, k, v, weights, indices, chunk_size=chunk_size, sm_scale=sm_scale,
                       mask_last_token=False, sm_n=float(sm_n), q_block=q_block)


# ----------------------------------------------------------------------------
# exact per-chunk log Z
# ----------------------------------------------------------------------------
def exact_chunk_log_z(q, k, *, chunk_size: int, window_size: int, sm_scale: Optional[float] = None,
                      mask_lmk: bool = False, row_block: int = 1024) -> torch.Tensor:
    """log_Z[b,t,h,c] = log sum_{j in chunk c} exp(sm_scale*<q_t,k_j>) with masks
    j > t, t < (c+1)S + W - 1 (chunk not fully remote), j >= L, and optionally the
    landmark key (j+1) % S == 0.  fp32 (B, L, h_q, ceil(L/S)); -inf where empty."""
    B, L, HQ, D = q.shape
    H = k.shape[2]
    G = HQ // H
    S, W = chunk_size, window_size
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    N = (L + S - 1) // S
    pad = N * S - L
    kf = k.float()
    if pad:
        kf = F.pad(kf, (0, 0, 0, 0, 0, pad))
    kf = kf.view(B, N, S, H, D)
    out = torch.full((B, L, HQ, N), NEG_INF, dtype=torch.float32)
    j = torch.arange(N * S).view(N, S)
    for t0 in range(0, L, row_block):
        t1 = min(L, t0 + row_block)
        qf = q[:, t0:t1].float().view(B, t1 - t0, H, G, D)
        s = torch.einsum("bthgd,bnshd->bthgns", qf, kf) * sm_scale
        t = torch.arange(t0, t1).view(-1, 1, 1)
        c = torch.arange(N).view(1, N, 1)
        masked = (j.view(1, N, S) > t) | (t < (c + 1) * S + W - 1) | (j.view(1, N, S) >= L)
        if mask_lmk:
            masked = masked | (((j.view(1, N, S) + 1) % S) == 0)
        s = s.masked_fill(masked.view(1, t1 - t0, 1, 1, N, S), NEG_INF)
        out[:, t0:t1] = torch.logsumexp(s, dim=-1).reshape(B, t1 - t0, HQ, N)
    return out


# ----------------------------------------------------------------------------
# rotary position embedding
# ----------------------------------------------------------------------------
def rope(x, cos, sin, *, lo_only: bool = False):
    """Rotate-half RoPE in fp32.  x (B,L,H,D); cos, sin (L,D), (1,L,D) or (B,L,D).
    out1 = x1*cos[d] - x2*sin[d], out2 = x2*cos[d'] + x1*sin[d'] with d' = d + D/2, or d when
    ``lo_only`` (ops/rope_tilelang_fp32.py:48-62 two-tensor kernel; :125-134 single-tensor kernel)."""
    B, L, H, D = x.shape
    half = D // 2
    cos, sin = cos.float(), sin.float()
    if cos.dim() == 2:
        cos, sin = cos.unsqueeze(0), sin.unsqueeze(0)
    cos, sin = cos.unsqueeze(2), sin.unsqueeze(2)  # (B or 1, L, 1, D)
    x1, x2 = x.float()[..., :half], x.float()[..., half:]
    c1, s1 = cos[..., :half], sin[..., :half]
    c2, s2 = (c1, s1) if lo_only else (cos[..., half:], sin[..., half:])
    return torch.cat([x1 * c1 - x2 * s1, x2 * c2 + x1 * s2], dim=-1)


def rms_norm(x, weight, eps: float = 1e-6):
    """models/FlashHiLS/modeling_qwen_hils.py:80-86: statistics in fp32, the normalised value cast
    back to the input dtype, then multiplied by the weight (in that dtype)."""
    x32 = x.to(torch.float32)
    var = x32.pow(2).mean(-1, keepdim=True)
    return weight * (x32 * torch.rsqrt(var + eps)).to(x.dtype)


def rope_hf(x, cos, sin):
    """models/FlashHiLS/hils_attention.py:137-171 for one tensor in (B,L,H,D) layout: x*cos +
    rotate_half(x)*sin, rotate_half(x) = (-x_hi, x_lo), every operation in x's dtype."""
    if cos.dim() == 2:
        cos, sin = cos.unsqueeze(0), sin.unsqueeze(0)
    cos, sin = cos.unsqueeze(2).to(x.dtype), sin.unsqueeze(2).to(x.dtype)
    half = x.shape[-1] // 2
    rot = torch.cat((-x[..., half:], x[..., :half]), dim=-1)
    return (x * cos) + (rot * sin)


def norm_rope_pool(x, weight, cos, sin, chunk_size: int, eps: float = 1e-6):
    """The layer's key preparation (hils_attention.py:314-321, :479-483, :398): optional per-head RMS
    norm, optional rotation, mean over every whole chunk.  Runs in x's dtype (pass bf16 for the
    layer's roundings, fp32 or fp64 for the exact function).  Returns (out, lmk)."""
    out = x if weight is None else rms_norm(x, weight.to(x.dtype), eps)
    if cos is not None:
        out = rope_hf(out, cos, sin)
    B, L, H, D = out.shape
    N = L // chunk_size
    lmk = out[:, :N * chunk_size].reshape(B, N, chunk_size, H, D).mean(dim=2)
    return out, lmk


# ----------------------------------------------------------------------------
# the sliding-window branch (only to synthesise a self-consistent lse_swa)
# ----------------------------------------------------------------------------
def swa(q, k, v, *, window_size: int, chunk_size: int, mask_lmk: bool = True,
        sm_scale: Optional[float] = None, q_offset: Optional[int] = None, expand_to_chunk: bool = True,
        kv_start: int = 0):
    """Causal window whose left edge is expanded to the chunk start (``expand_to_chunk``);
    landmark keys masked (``mask_lmk``).  Query t sits at the absolute position
    kv_start + q_offset + t with q_offset = Lk - Lq by default, key j at kv_start + j
    (ops/flex_attn_tilelang.py:108-121,155-171).  Returns (o fp32 (B,Lq,hq,Dv), lse fp32
    (B,Lq,hq), natural log); rows that see no key get o = 0, lse = -inf."""
    B, L, HQ, D = q.shape
    Lk, H = k.shape[1], k.shape[2]
    G = HQ // H
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    if q_offset is None:
        q_offset = Lk - L
    kf = k.float().repeat_interleave(G, dim=2)
    vf = v.float().repeat_interleave(G, dim=2)
    s = torch.einsum("bihd,bjhd->bhij", q.float(), kf) * sm_scale
    real_q = torch.arange(L).view(L, 1) + q_offset + kv_start
    kv = torch.arange(Lk).view(1, Lk) + kv_start
    start = real_q - window_size + 1
    if expand_to_chunk:
        start = torch.div(start, chunk_size, rounding_mode="floor") * chunk_size
    keep = (kv >= start) & (kv <= real_q)
    if mask_lmk:
        keep = keep & (((kv + 1) % chunk_size) != 0)
    s = s.masked_fill(~keep.view(1, 1, L, Lk), NEG_INF)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - torch.where(torch.isfinite(lse), lse, torch.zeros_like(lse)).unsqueeze(-1))
    p = torch.where(keep.view(1, 1, L, Lk), p, torch.zeros_like(p))
    o = torch.einsum("bhij,bjhd->bihd", p, vf)
    return o, lse.permute(0, 2, 1).contiguous()


# ----------------------------------------------------------------------------
# layer glue and the dense equivalent
# ----------------------------------------------------------------------------
def inter_chunk_softmax(scores, lse_swa, prior_b=None, indices=None, softmax1=False, bf16_sum=False):
    """chunk_weights = softmax([scores_1..K (+ gathered prior bias), lse_swa (, 0)]).
    scores (B,L,hq,K); returns fp32 (B,L,hq,K+1(+1)).  ``bf16_sum``: round the biased scores to bf16,
    as the layer's ``scores + gathered.to(scores.dtype)`` on bf16 tensors does
    (models/FlashHiLS/hils_attention.py:600-602); the default keeps the sum in fp32."""
    B, L, HQ, K = scores.shape
    sc = scores.float()
    if prior_b is not None:
        Hkv = indices.shape[2]
        idx = indices.repeat_interleave(HQ // Hkv, dim=2).clamp_min(0).long()
        src = prior_b.float().unsqueeze(-1).expand(-1, -1, -1, K)
        sc = sc + torch.gather(src, 1, idx)
        if bf16_sum:
            sc = sc.bfloat16().float()
    cols = [sc, lse_swa.float().unsqueeze(-1)]
    if softmax1:
        cols.append(torch.zeros(B, L, HQ, 1))
    return F.softmax(torch.cat(cols, dim=-1), dim=-1)


def hils_layer_forward(q, k, v, *, chunk_size: int, topk: int, window_size: int,
                       sm_scale: Optional[float] = None, lmk_k=None, prior_b=None):
    """One HiLS attention layer forward on already-projected q/k/v (fp32 math):
    SWA branch -> chunk keys (mean pool unless given) -> top-k -> inter-chunk
    softmax -> sparse attention -> merge.  Returns dict with every intermediate."""
    B, L, HQ, D = q.shape
    H = k.shape[2]
    G = HQ // H
    swa_o, lse_swa = swa(q, k, v, window_size=window_size, chunk_size=chunk_size,
                         mask_lmk=True, sm_scale=sm_scale)
    if lmk_k is None:
        lmk_k = mean_pool(k, chunk_size)
    idx, scores = online_softmax_topk_head(
        q.view(B, L, H, G, D), lmk_k, lse_swa, topk, chunk_size, window_size,
        is_causal=True, q_offset=0, sm_scale=sm_scale, bias=prior_b)
    scores = scores.reshape(B, L, HQ, topk)
    w = inter_chunk_softmax(scores, lse_swa, prior_b, idx)
    o_sparse, lse_chunks = sparse_attn(q, k, v, w, idx, chunk_size=chunk_size, sm_scale=sm_scale,
                                       mask_last_token=True, return_lse=True)
    o = o_sparse + swa_o * w[..., topk].unsqueeze(-1)
    return {"indices": idx, "scores": scores, "weights": w, "lse_swa": lse_swa, "swa_o": swa_o,
            "o_sparse": o_sparse, "o": o, "lse_chunks": lse_chunks, "lmk_k": lmk_k}


def dense_hils_attention(q, k, v, *, chunk_size: int, window_size: int, indices,
                         sm_scale: Optional[float] = None, mask_lmk: bool = True):
    """Ordinary softmax attention over exactly the kept tokens: the SWA window plus
    the non-landmark tokens of every selected chunk.  The factorised form equals
    this when the inter-chunk weights are softmax over the true chunk masses.
    Returns (o fp32, lse fp32 (B,L,hq))."""
    B, L, HQ, D = q.shape
    H = k.shape[2]
    G = HQ // H
    S = chunk_size
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    kf = k.float().repeat_interleave(G, dim=2)
    vf = v.float().repeat_interleave(G, dim=2)
    s = torch.einsum("bihd,bjhd->bhij", q.float(), kf) * sm_scale
    t = torch.arange(L).view(L, 1)
    j = torch.arange(L).view(1, L)
    start = torch.div(t - window_size + 1, S, rounding_mode="floor") * S
    keep = ((j >= start) & (j <= t)).view(1, 1, L, L).expand(B, HQ, L, L).clone()
    N = L // S
    sel = torch.zeros(B, L, H, N + 1, dtype=torch.bool)
    sel.scatter_(3, torch.where(indices < 0, torch.full_like(indices, N), indices).long(),
                 torch.ones_like(indices, dtype=torch.bool))
    sel = sel[..., :N]  # (B,L,H,N)
    sel_tok = sel.repeat_interleave(S, dim=3)  # (B,L,H,N*S)
    if sel_tok.shape[3] < L:
        sel_tok = F.pad(sel_tok, (0, L - sel_tok.shape[3]))
    sel_tok = sel_tok.repeat_interleave(G, dim=2).permute(0, 2, 1, 3)  # (B,HQ,L,L)
    keep = keep | sel_tok
    if mask_lmk:
        keep = keep & (((j + 1) % S) != 0).view(1, 1, 1, L)
    s = s.masked_fill(~keep, NEG_INF)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.softmax(s, dim=-1)
    p = torch.nan_to_num(p, nan=0.0)
    o = torch.einsum("bhij,bjhd->bihd", p, vf)
    return o, lse.permute(0, 2, 1).contiguous()
