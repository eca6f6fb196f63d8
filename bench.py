"""Benchmark of the HiLS attention forward hot path on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` prints ONE JSON line.

Workload at N=1 (`config.workload`): the 7B-shaped 32K-token prefill layer forward
(B1 L32768, 32 query heads / 8 KV heads, head_dim 128, chunk 64 -> 512 chunks, top-32).
One step = mean-pool chunk keys -> fused top-k -> inter-chunk softmax -> sparse
attention, inputs resident in HBM.  `value` is tokens/s of that step.  The same line
carries the 128K-context decode step (batch 32, 2048 pooled chunk keys per KV head) as
`decode_us_per_step` (K and V in pages of one chunk, the cache the configuration names; the
step on (B, Lkv, H, D) cache tensors beside it as `decode_token_major_cache_us`), a roofline
object for the dominant kernel of each, and the CPU oracle timed on a bounded query slice as
`cpu_baseline`.
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402


def _load_inputs():
    """The synthetic-input builders live with the parity tests (tests/util.py), which check the
    kernels on exactly the tensors timed here."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("hils_test_util", os.path.join(ROOT, "tests", "util.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


_inputs = _load_inputs()
gpu_randn, swa_lse_current_chunk = _inputs.gpu_randn, _inputs.swa_lse_current_chunk
prefill_inputs, config2_inputs = _inputs.prefill_inputs, _inputs.config2_inputs
train_inputs, train_forward = _inputs.train_inputs, _inputs.train_forward

MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E


def measured_traffic(key):
    """HBM bytes per launch of a kernel as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE.
    The figures live in the committed counter summary, on lines `bench.traffic <key> <bytes>`;
    None when the summary (or the key) is absent."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic_per_launch.txt")
    try:
        with open(path) as fh:
            for line in fh:
                parts = line.split()
                if len(parts) == 3 and parts[0] == "bench.traffic" and parts[1] == key:
                    return float(parts[2])
    except OSError:
        pass
    return None


def time_steps(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def bench_prefill(pkg, dev, steps, warmup):
    from hils_attention_amd.ops import hils_fwd_bwd_head as attn_mod
    B, L, HQ, H, D, S, K, W = 1, 32768, 32, 8, 128, 64, 32, 1
    G = HQ // H
    q, k, v, lse_swa = prefill_inputs(dev)  # lse_swa in bf16, as the layer hands it over
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
    state = {}
    acc = {"pool": 0.0, "topk": 0.0, "glue": 0.0, "vt": 0.0, "attn": 0.0, "n": 0}

    side = torch.cuda.Stream()

    def step(record=False):
        cur = torch.cuda.current_stream()
        if not record:
            # the K/V repacking does not depend on the selection: it runs on a second stream beside
            # the top-k kernel, which leaves most of the HBM bandwidth unused
            side.wait_stream(cur)
            with torch.cuda.stream(side):
                ws = attn_mod.prepare_kv_workspace(L, k, v, HQ, K, S)
            ws.record_stream(cur)
        if record:
            ev[0].record()
        lmk = pkg.chunk_mean_pool(k, S)
        if record:
            ev[1].record()
        idx, scores, w = pkg.topk_chunk_weights(q, lmk, lse_swa, K, S, W)  # selection + inter-chunk softmax, one call
        if record:
            ev[2].record()
            ev[3].record()
            ws = attn_mod.prepare_kv_workspace(L, k, v, HQ, K, S)  # serial here: per-kernel durations
            ev[4].record()
        else:
            cur.wait_stream(side)
        o = pkg.HiLS_block_M_head(q, k, v, w, idx, block_size=S, is_training=False, kv_workspace=ws)
        if record:
            ev[5].record()
            torch.cuda.synchronize()
            for name, a, b in (("pool", 0, 1), ("topk", 1, 2), ("glue", 2, 3), ("vt", 3, 4), ("attn", 4, 5)):
                acc[name] += ev[a].elapsed_time(ev[b])
            acc["n"] += 1
        state["idx"], state["o"] = idx, o

    sec = time_steps(step, steps, warmup)
    for _ in range(min(steps, 5)):  # per-kernel durations with events on the launch stream
        step(record=True)
    per = {kk: vv / acc["n"] for kk, vv in acc.items() if kk != "n"}
    n_sel = int((state["idx"] >= 0).sum().item())
    flops = 4.0 * D * S * G * n_sel
    attn_ms = per["attn"]
    roof = {"kernel": "sparse_attn_fwd_gather", "bound": "mfma",
            "achieved": flops / (attn_ms * 1e-3) / 1e12, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": flops / (attn_ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, "traffic": measured_traffic("prefill_attention_bytes_per_launch"),
            "flops_per_launch": flops, "ms_per_launch": attn_ms}
    cfg = {"workload": "prefill_fwd B1 L32768 hq32/hkv8 D128 chunk64 top32 causal (7B-shaped, config 3)",
           "global_batch": B, "seq_len": L, "n_sel": n_sel}
    data = {"q": q, "k": k, "v": v, "lse_swa": lse_swa}
    return sec, per, roof, cfg, data


def bench_config2(pkg, dev, iters=5):
    """Config 2: B4 L8192, 16 heads MHA, D64, top-32: the same forward step as the headline
    (mean pool -> top-k -> inter-chunk softmax -> K/V packing -> sparse attention)."""
    from hils_attention_amd.ops import hils_fwd_bwd_head as attn_mod
    B, L, HQ, H, D, S, K, W = 4, 8192, 16, 16, 64, 64, 32, 1
    q, k, v, lse_swa = config2_inputs(dev)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    t_all = t_attn = 0.0
    n_sel = 0
    for it in range(iters + 1):
        ev[0].record()
        lmk = pkg.chunk_mean_pool(k, S)
        idx, scores, w = pkg.topk_chunk_weights(q, lmk, lse_swa, K, S, W)
        ws = attn_mod.prepare_kv_workspace(L, k, v, HQ, K, S)
        ev[1].record()
        pkg.HiLS_block_M_head(q, k, v, w, idx, block_size=S, is_training=False, kv_workspace=ws)
        ev[2].record()
        torch.cuda.synchronize()
        if it:  # the first pass warms up
            t_all += ev[0].elapsed_time(ev[2])
            t_attn += ev[1].elapsed_time(ev[2])
        n_sel = int((idx >= 0).sum().item())
    t_all /= iters
    t_attn /= iters
    flops = 4.0 * D * S * (HQ // H) * n_sel
    return {"workload": "prefill_fwd B4 L8192 h16/16 D64 chunk64 top32 causal (config 2)",
            "ms_per_step": t_all, "tokens_per_s": B * L / (t_all * 1e-3), "attn_ms": t_attn,
            "attn_mfma_frac": flops / (t_attn * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS}


def bench_decode(pkg, dev, steps, warmup):
    B, Lkv, HQ, H, D, S, K, W = 32, 131072, 32, 8, 128, 64, 32, 1
    N = Lkv // S
    gen = torch.Generator(device=dev).manual_seed(1004)
    q = gpu_randn((B, 1, HQ, D), gen, dev)
    kc = gpu_randn((B, Lkv, H, D), gen, dev)
    vc = gpu_randn((B, Lkv, H, D), gen, dev)
    from hils_attention_amd.ops.hils_glue import head_major_chunk_keys
    lmk = pkg.chunk_mean_pool(kc, S)  # precomputed pooled keys (untimed)
    # the cache layers keep the pooled keys head-major, (B, H, chunks, D): a row's keys are contiguous
    lmk_hm = head_major_chunk_keys(lmk)
    # fp32, as the sliding-window attention kernel hands its log-sum-exp over
    lse_swa = torch.randn(B, 1, HQ, device=dev, generator=gen) * 5 + 10
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    acc = {"topk": 0.0, "glue": 0.0, "attn": 0.0, "n": 0}

    def step():
        # the remote branch of the step in one launch: a row's workgroup selects, then attends
        pkg.decode_step(q, lmk_hm, kc, vc, lse_swa, K, S, W, q_offset=Lkv - 1, lmk_head_major=True)

    def step_token_major():  # the chunk keys in the reference's layout (B, chunks, H, D)
        pkg.decode_step(q, lmk, kc, vc, lse_swa, K, S, W, q_offset=Lkv - 1)

    def step2(record=False):
        if record:
            ev[0].record()
        # selection and the inter-chunk softmax in one call (one kernel at this shape)
        idx, scores, w = pkg.topk_chunk_weights(q, lmk, lse_swa, K, S, W, q_offset=Lkv - 1)
        if record:
            ev[1].record()
            ev[2].record()
        pkg.HiLS_block_M_head(q, kc, vc, w, idx, block_size=S, is_training=False)
        if record:
            ev[3].record()
            torch.cuda.synchronize()
            for name, a, b in (("topk", 0, 1), ("glue", 1, 2), ("attn", 2, 3)):
                acc[name] += ev[a].elapsed_time(ev[b])
            acc["n"] += 1

    # a decode step is 80 us: the launch of the first step and the wait for the last one, a few tens
    # of microseconds together, are spread over at least 200 steps so that the figure is the steady state
    steps = max(steps, 200)
    eager_sec = time_steps(step, steps, warmup)
    token_major_sec = time_steps(step_token_major, steps, warmup)
    # the layer's default mode: a prior bias per (chunk, query head) in the selection and the softmax
    prior_hm = torch.randn(B, H, N, HQ // H, device=dev, generator=gen)
    prior_sec = time_steps(lambda: pkg.decode_step(q, lmk_hm, kc, vc, lse_swa, K, S, W, q_offset=Lkv - 1,
                                                   prior_b=prior_hm, lmk_head_major=True), steps, warmup)
    # and with one chunk key per query head beside that bias (attention-pooled keys, the layer's default
    # pooling): four times the key bytes per step
    lmk_q_hm = gpu_randn((B, HQ, N, D), gen, dev)
    perq_sec = time_steps(lambda: pkg.decode_step(q, lmk_q_hm, kc, vc, lse_swa, K, S, W, q_offset=Lkv - 1,
                                                  prior_b=prior_hm, lmk_head_major=True), steps, warmup)
    del lmk_q_hm
    two_call_sec = time_steps(step2, steps, warmup)
    for _ in range(min(steps, 5)):
        step2(record=True)
    per = {kk: vv / acc["n"] for kk, vv in acc.items() if kk != "n"}  # the two calls, each timed alone
    per["two_call_step"] = two_call_sec * 1e3
    per["token_major_keys_step"] = token_major_sec * 1e3
    per["prior_bias_step"] = prior_sec * 1e3
    per["key_per_query_head_prior_bias_step"] = perq_sec * 1e3
    # the serving loop replays the step as one HIP graph (no host work between kernels)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    sec = time_steps(graph.replay, steps, warmup)
    per["eager_step"] = eager_sec * 1e3
    best = min(sec, eager_sec)  # the figure the step is reported with
    # the same step on the paged cache (page = chunk: 16 KiB contiguous per selected chunk and tensor,
    # pages handed out in random order), the layout of a paged serving backend
    n_pages = B * N
    perm = torch.randperm(n_pages, device=dev, generator=gen)
    k_pages = torch.empty((n_pages, H, S, D), dtype=kc.dtype, device=dev)
    v_pages = torch.empty_like(k_pages)
    k_pages[perm] = kc.view(B, N, S, H, D).permute(0, 1, 3, 2, 4).reshape(n_pages, H, S, D)
    v_pages[perm] = vc.view(B, N, S, H, D).permute(0, 1, 3, 2, 4).reshape(n_pages, H, S, D)
    lmk_pages = torch.empty((n_pages, H, D), dtype=lmk.dtype, device=dev)
    lmk_pages[perm] = lmk.reshape(n_pages, H, D)
    table = perm.view(B, N).to(torch.int32).contiguous()
    paged_sec = time_steps(lambda: pkg.paged_hils_attend(q, k_pages, v_pages, None, table, lse_swa, Lkv, K, W,
                                                         lmk_dense=lmk_hm), steps, warmup)
    per["paged_step"] = paged_sec * 1e3  # K, V in pages; the pooled keys per sequence, head-major
    paged_lmk_sec = time_steps(lambda: pkg.paged_hils_attend(q, k_pages, v_pages, lmk_pages, table, lse_swa, Lkv, K, W),
                               steps, warmup)
    per["paged_keys_per_page_step"] = paged_lmk_sec * 1e3
    del k_pages, v_pages
    lmk_bytes = B * N * H * D * 2
    kv_bytes = B * H * K * S * D * 2 * 2
    small = B * HQ * D * 2 * 2
    total = lmk_bytes + kv_bytes + small
    # Reported step: the configuration's cache, K and V in pages of one chunk (16 KiB contiguous per page and KV
    # head), the pooled keys per sequence; the (B, Lkv, H, D) tensors of the reference's HiLSDynamicLayer beside it.
    roof = {"kernel": "decode_step_kernel<128, true, 4> (selection + sparse attention of a row, one launch; K, V in "
                      "pages of one chunk)", "bound": "hbm",
            "achieved": total / paged_sec / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": total / paged_sec / 1e9 / HBM_PEAK_GBS, "traffic": measured_traffic("decode_step_paged_bytes"),
            "bytes_per_step": total,
            "token_major_cache": {"kernel": "decode_step_kernel<128, false, 4> (K, V as (B, Lkv, H, D) tensors)",
                                  "us_per_step": best * 1e6, "achieved": total / best / 1e9,
                                  "frac": total / best / 1e9 / HBM_PEAK_GBS,
                                  "traffic": measured_traffic("decode_step_bytes")},
            "topk_gbs": lmk_bytes / (per["topk"] * 1e-3) / 1e9,
            "attn_gbs": kv_bytes / (per["attn"] * 1e-3) / 1e9}
    del kc, vc
    torch.cuda.empty_cache()
    # the same step at the head counts of the reference's own configurations (16 query / 2 KV heads of 64,
    # eight query heads per KV head; 256 rows, 128K context): shared chunk keys, and the layer's default mode
    HQ2, H2, D2 = 16, 2, 64
    B2 = 256 // H2
    q2 = gpu_randn((B2, 1, HQ2, D2), gen, dev)
    k2 = gpu_randn((B2, Lkv, H2, D2), gen, dev)
    v2 = gpu_randn((B2, Lkv, H2, D2), gen, dev)
    lse2 = torch.randn(B2, 1, HQ2, device=dev, generator=gen) * 5 + 10
    lmk2 = pkg.head_major_chunk_keys(pkg.chunk_mean_pool(k2, S))
    lmk2_q = gpu_randn((B2, HQ2, N, D2), gen, dev)
    prior2 = torch.randn(B2, H2, N, HQ2 // H2, device=dev, generator=gen)
    per["hq16_hkv2_d64_step"] = time_steps(lambda: pkg.decode_step(
        q2, lmk2, k2, v2, lse2, K, S, W, q_offset=Lkv - 1, lmk_head_major=True), steps, warmup) * 1e3
    per["hq16_hkv2_d64_key_per_query_head_prior_bias_step"] = time_steps(lambda: pkg.decode_step(
        q2, lmk2_q, k2, v2, lse2, K, S, W, q_offset=Lkv - 1, prior_b=prior2, lmk_head_major=True), steps, warmup) * 1e3
    del q2, k2, v2, lmk2, lmk2_q, prior2
    torch.cuda.empty_cache()
    return sec, per, roof


def bench_train(pkg, dev, iters=3):
    """Config 5: 345M-shaped training layer, forward + backward (B8 L8192, 16 heads MHA, D64, top-32):
    mean pool -> top-k scores -> softmax over [scores, lse_swa] -> sparse attention, gradients to
    q, k, v through every op."""
    B, L, HQ, H, D, S, K, W = 8, 8192, 16, 16, 64, 64, 32, 1
    q, k, v, d_o, lse_swa = train_inputs(dev)

    def fwd():
        return train_forward(pkg, q, k, v, lse_swa)

    def fwd_bwd():
        for t in (q, k, v):
            t.grad = None
        o, _ = fwd()
        o.backward(d_o)

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters

    with torch.no_grad():
        t_fwd = timed(lambda: fwd())
        n_sel = int((fwd()[1] >= 0).sum().item())
    t_all = timed(fwd_bwd)
    flops_fwd = 4.0 * D * S * (HQ // H) * n_sel
    return {"workload": "train layer fwd+bwd B8 L8192 h16/16 D64 chunk64 top32 (config 5)",
            "fwd_ms": t_fwd, "fwd_bwd_ms": t_all, "tokens_per_s_fwd_bwd": B * L / (t_all * 1e-3),
            "attn_flops_fwd": flops_fwd, "attn_flops_bwd": 2.5 * flops_fwd,
            "layer_tflops_fwd_bwd": 3.5 * flops_fwd / (t_all * 1e-3) / 1e12}


def bench_ops(pkg, dev, iters=3):
    """The operators of the path that the prefill / decode steps above do not exercise, each at a
    config-3-shaped size: attention pooling of the chunk keys, exact chunk log-Z (forward and
    forward+backward), and the older HSA operator."""
    gen = torch.Generator(device=dev).manual_seed(1006)

    def timed(fn, n=iters):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    out = {}
    # attention pool: B1, 512 chunks of 64 tokens, 32 heads, D128 (one K tile per head)
    N, S, H, D = 512, 64, 32, 128
    mu = gpu_randn((1, N, H, D), gen, dev)
    kc = gpu_randn((1, N, S, H, D), gen, dev)
    with torch.no_grad():
        t = timed(lambda: pkg.chunk_attn_pool_tilelang(mu, kc))
    out["attn_pool_fwd"] = {"workload": "B1 N512 S64 H32 D128", "us": t * 1e3,
                            "hbm_gbs": kc.numel() * 2 / (t * 1e-3) / 1e9}
    mu_g, kc_g = mu.clone().requires_grad_(), kc.clone().requires_grad_()

    def pool_fb():
        mu_g.grad = None
        kc_g.grad = None
        a, b = pkg.chunk_attn_pool_tilelang(mu_g, kc_g)
        (a.float().sum() + b.sum()).backward()

    out["attn_pool_fwd_bwd"] = {"workload": "B1 N512 S64 H32 D128 (includes the torch glue of the loss)",
                                "us": timed(pool_fb) * 1e3}
    del kc, kc_g, mu_g
    # the same prior queries over K at the model's own 8 KV heads (four query heads per K tile)
    kc8 = gpu_randn((1, N, S, 8, D), gen, dev)
    with torch.no_grad():
        t = timed(lambda: pkg.chunk_attn_pool(mu, kc8), 10)
    out["attn_pool_gqa_fwd"] = {"workload": "B1 N512 S64 hq32/hkv8 D128", "us": t * 1e3,
                                "hbm_gbs": (kc8.numel() * 2 + 2 * mu.numel() * 2 + N * S * H * 4) / (t * 1e-3) / 1e9}
    mu_g, kc_g = mu.clone().requires_grad_(), kc8.clone().requires_grad_()

    def pool_gqa_fb():
        mu_g.grad = None
        kc_g.grad = None
        a, b = pkg.chunk_attn_pool(mu_g, kc_g)
        (a.float().sum() + b.sum()).backward()

    out["attn_pool_gqa_fwd_bwd"] = {"workload": "same (includes the torch glue of the loss)",
                                    "us": timed(pool_gqa_fb, 10) * 1e3}
    del kc8, kc_g, mu, mu_g
    # key preparation in one pass (RMS norm + rotary embedding + chunk mean) on the 32K prefill's K
    Lp, Hk = 32768, 8
    kx = gpu_randn((1, Lp, Hk, D), gen, dev)
    nw = (torch.rand(D, device=dev, generator=gen) + 0.5).bfloat16()
    ang = torch.rand(Lp, D // 2, device=dev, generator=gen) * 6.0
    cos_t = torch.cat([ang.cos(), ang.cos()], -1).bfloat16()
    sin_t = torch.cat([ang.sin(), ang.sin()], -1).bfloat16()
    with torch.no_grad():
        t = timed(lambda: pkg.norm_rope_pool(kx, nw, cos_t, sin_t, 64), 10)
    out["norm_rope_pool_fwd"] = {"workload": "K of the 32K prefill: B1 L32768 H8 D128 chunk64", "us": t * 1e3,
                                 "hbm_gbs": (2 * kx.numel() + 2 * cos_t.numel()) * 2 / (t * 1e-3) / 1e9}
    del kx, nw, ang, cos_t, sin_t
    # exact chunk log-Z: B1 L8192 hq32/hkv8 D128, window 64
    L, HQ, HK = 8192, 32, 8
    q = gpu_randn((1, L, HQ, D), gen, dev)
    k = gpu_randn((1, L, HK, D), gen, dev)
    with torch.no_grad():
        t = timed(lambda: pkg.exact_chunk_log_z_tl(q, k, chunk_size=64, window_size=64))
    flops = 2.0 * D * HQ * L * (L / 2)
    out["log_z_fwd"] = {"workload": "B1 L8192 hq32/hkv8 D128 chunk64 window64", "ms": t,
                        "mfma_tflops": flops / (t * 1e-3) / 1e12}
    qg, kg = q.clone().requires_grad_(), k.clone().requires_grad_()

    def lz_fb():
        qg.grad = None
        kg.grad = None
        z = pkg.exact_chunk_log_z_tl(qg, kg, chunk_size=64, window_size=64)
        torch.where(torch.isfinite(z), z, torch.zeros_like(z)).sum().backward()

    t = timed(lz_fb)
    out["log_z_fwd_bwd"] = {"workload": "same (includes the torch glue of the loss)", "ms": t,
                            "mfma_tflops": 5.0 * flops / (t * 1e-3) / 1e12}
    del q, k, qg, kg
    # sliding-window attention of the local branch: B1 L32768 hq32/hkv8 D128, window 64, chunk 64
    L, HQ, HK, D = 32768, 32, 8, 128
    q = gpu_randn((1, L, HQ, D), gen, dev)
    k = gpu_randn((1, L, HK, D), gen, dev)
    v = gpu_randn((1, L, HK, D), gen, dev)
    with torch.no_grad():
        t = timed(lambda: pkg.flex_attn_tl(q, k, v, 64, 64))
        _, lse_w = pkg.flex_attn_tl(q, k, v, 64, 64)
    # visible keys per query: from the chunk start of (t - 63) to t, landmarks excluded
    tt = torch.arange(L, device=dev)
    start = torch.div(tt - 63, 64, rounding_mode="floor").clamp_min(0) * 64
    n_vis = float((tt - start + 1 - (tt // 64 - start // 64) - ((tt + 1) % 64 == 0).long()).sum().item())
    out["swa_fwd"] = {"workload": "B1 L32768 hq32/hkv8 D128 window64 chunk64", "us": t * 1e3,
                      "visible_tflops": 4.0 * D * HQ * n_vis / (t * 1e-3) / 1e12,
                      "hbm_gbs": (2 * q.numel() + k.numel() + v.numel()) * 2 / (t * 1e-3) / 1e9}
    qg, kg, vg = (x.clone().requires_grad_() for x in (q, k, v))
    d_o = gpu_randn((1, L, HQ, D), gen, dev)

    def swa_fb():
        for x in (qg, kg, vg):
            x.grad = None
        o, lse = pkg.flex_attn_tl(qg, kg, vg, 64, 64)
        torch.autograd.backward([o, lse], [d_o, torch.ones_like(lse)])

    out["swa_fwd_bwd"] = {"workload": "same", "us": timed(swa_fb) * 1e3}
    del q, k, v, qg, kg, vg, d_o
    # the local branch at the window the reference times it at (scripts/bench/bench_flex_attn_bwd_clamp.py:66-72:
    # window 512, chunk 64, L16384; 16/2 heads of 64 with the window expanded to its chunk start, 32/32 heads
    # of 128 without)
    for name, HQ, HK, D, expand in (("w512_hq16_hkv2_d64", 16, 2, 64, True), ("w512_hq32_hkv32_d128", 32, 32, 128, False)):
        L, Wn = 16384, 512
        q = gpu_randn((1, L, HQ, D), gen, dev)
        k = gpu_randn((1, L, HK, D), gen, dev)
        v = gpu_randn((1, L, HK, D), gen, dev)
        with torch.no_grad():
            t = timed(lambda: pkg.flex_attn_tl(q, k, v, Wn, 64, expand_to_chunk=expand))
        tt = torch.arange(L, device=dev)
        lo = (tt - Wn + 1).clamp_min(0)
        if expand:
            lo = torch.div(lo, 64, rounding_mode="floor") * 64
        # keys lo .. t, landmarks (positions 63 mod 64) excluded
        n_lmk = torch.div(tt + 1, 64, rounding_mode="floor") - torch.div(lo, 64, rounding_mode="floor")
        n_vis = float((tt - lo + 1 - n_lmk).sum().item())
        flops = 4.0 * D * HQ * n_vis
        out["swa_fwd_" + name] = {"workload": f"B1 L{L} hq{HQ}/hkv{HK} D{D} window{Wn} chunk64 expand_to_chunk={expand}",
                                  "us": t * 1e3, "visible_tflops": flops / (t * 1e-3) / 1e12,
                                  "hbm_gbs": (2 * q.numel() + k.numel() + v.numel()) * 2 / (t * 1e-3) / 1e9}
        qg, kg, vg = (x.clone().requires_grad_() for x in (q, k, v))
        d_o = gpu_randn((1, L, HQ, D), gen, dev)

        def swa_fb512():
            for x in (qg, kg, vg):
                x.grad = None
            o, lse = pkg.flex_attn_tl(qg, kg, vg, Wn, 64, expand_to_chunk=expand)
            torch.autograd.backward([o, lse], [d_o, torch.ones_like(lse)])

        t = timed(swa_fb512)
        # the forward's two products (S, P V) and the backward's five (S again, dV, dP, dQ, dK)
        out["swa_fwd_bwd_" + name] = {"workload": "same", "us": t * 1e3,
                                      "visible_tflops": 3.5 * flops / (t * 1e-3) / 1e12,
                                      "hbm_gbs": (4 * q.numel() + 2 * (k.numel() + v.numel())) * 2 / (t * 1e-3) / 1e9}
        del q, k, v, qg, kg, vg, d_o
    # chunk selection + inter-chunk weights of the 32K prefill, without and with the layer's prior bias
    # (models/FlashHiLS/hils_attention.py:568-602: the bias of the selection and of the softmax)
    q, k, v, lse_p = prefill_inputs(dev)
    del v
    lmk = pkg.chunk_mean_pool(k, 64)
    prior = (torch.randn(1, lmk.shape[1], q.shape[2], device=dev, generator=gen) * 0.5).bfloat16()
    with torch.no_grad():
        t0 = timed(lambda: pkg.topk_chunk_weights(q, lmk, lse_p, 32, 64, 1), 5)
        t1 = timed(lambda: pkg.topk_chunk_weights(q, lmk, lse_p, 32, 64, 1, prior_b=prior), 5)
    out["topk_prefill"] = {"workload": "B1 L32768 hq32/hkv8 D128 N512 top32 (selection + weights)", "us": t0 * 1e3}
    out["topk_prefill_bias"] = {"workload": "same, with a prior bias (B,N,h_q)", "us": t1 * 1e3}
    del q, k, lse_p, lmk, prior
    # the same operator at the head counts of the reference's own model configurations (eight query heads per
    # KV head; configs/hils_attention: 16/2 heads of 64, 32/4 heads of 128) and on a 128K prefill (2048 chunks),
    # with shared chunk keys and in the layer's default mode (a key per query head + the prior bias)
    for name, L, HQ, HK, D in (("hq16_hkv2_d64", 32768, 16, 2, 64), ("hq32_hkv4_d128", 32768, 32, 4, 128),
                               ("128k_hq32_hkv8_d128", 131072, 32, 8, 128), ("128k_hq16_hkv2_d64", 131072, 16, 2, 64)):
        N = L // 64
        q = gpu_randn((1, L, HQ, D), gen, dev)
        lmk = gpu_randn((1, N, HK, D), gen, dev)
        lmk_q = gpu_randn((1, N, HQ, D), gen, dev)
        lse_p = torch.randn(1, L, HQ, device=dev, generator=gen) * 3 + 5
        prior = torch.randn(1, N, HQ, device=dev, generator=gen) * 0.5
        with torch.no_grad():
            t0 = timed(lambda: pkg.topk_chunk_weights(q, lmk, lse_p, 32, 64, 1), 3)
            t1 = timed(lambda: pkg.topk_chunk_weights(q, lmk_q, lse_p, 32, 64, 1, prior_b=prior, num_kv_heads=HK), 3)
        out["topk_prefill_" + name] = {"workload": f"B1 L{L} hq{HQ}/hkv{HK} D{D} N{N} top32 (selection + weights)",
                                       "us": t0 * 1e3, "key_per_query_head_prior_bias_us": t1 * 1e3}
        del q, lmk, lmk_q, lse_p, prior
    # rotary embedding of q and k: B1 L32768 hq32/hkv8 D128
    L, HQ, HK, D = 32768, 32, 8, 128
    q = gpu_randn((1, L, HQ, D), gen, dev)
    k = gpu_randn((1, L, HK, D), gen, dev)
    ang = torch.rand(1, L, D // 2, device=dev, generator=gen) * 6.283
    cos = torch.cat([ang.cos(), ang.cos()], -1).bfloat16()
    sin = torch.cat([ang.sin(), ang.sin()], -1).bfloat16()
    with torch.no_grad():
        t = timed(lambda: pkg.rope_rotary_pos_emb(q, k, cos, sin))
    out["rope_qk"] = {"workload": "B1 L32768 hq32/hkv8 D128", "us": t * 1e3,
                      "hbm_gbs": 2 * (q.numel() + k.numel()) * 2 / (t * 1e-3) / 1e9}
    del q, k, cos, sin, ang
    # HSA: N2 L4096 hq16/hkv4 D64, 16 chunks per block of 16 queries
    Nb, L, HQ, HK, D, K, QX = 2, 4096, 16, 4, 64, 16, 16
    q = gpu_randn((Nb, L, HQ, D), gen, dev)
    k = gpu_randn((Nb, L, HK, D), gen, dev)
    v = gpu_randn((Nb, L, HK, D), gen, dev)
    idx = torch.rand(Nb, L // QX, HK, L // 64, device=dev, generator=gen).topk(K, dim=-1).indices
    idx = idx.sort(-1).values.to(torch.int32)
    w = torch.softmax(torch.randn(Nb, L // QX, HK, K, device=dev, generator=gen), -1).bfloat16()
    with torch.no_grad():
        t = timed(lambda: pkg.HSA(q, k, v, w, idx, 1.0, 64, 1 / 8.0))
    out["hsa_fwd"] = {"workload": "N2 L4096 hq16/hkv4 D64 top16 q_block16", "ms": t,
                      "tflops": 4.0 * D * 64 * HQ * Nb * L * K / (t * 1e-3) / 1e12}
    qg, kg, vg, wg = (x.clone().requires_grad_() for x in (q, k, v, w))
    d_o = gpu_randn((Nb, L, HQ, D), gen, dev)

    def hsa_fb():
        for x in (qg, kg, vg, wg):
            x.grad = None
        pkg.HSA(qg, kg, vg, wg, idx, 1.0, 64, 1 / 8.0).backward(d_o)

    out["hsa_fwd_bwd"] = {"workload": "same", "ms": timed(hsa_fb)}
    return out


def cpu_baseline(data, n_queries=4096):
    """The CPU oracle on a bounded slice of the prefill workload: n_queries consecutive
    queries around the middle of the sequence (top-k + inter-chunk softmax + sparse attention)."""
    orc = entry.load_oracle()
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    S, K, W = 64, 32, 1
    q, k, v, lse = (data[n].cpu() for n in ("q", "k", "v", "lse_swa"))
    B, L, HQ, D = q.shape
    H = k.shape[2]
    t0q = L // 2 - n_queries // 2
    qs = q[:, t0q:t0q + n_queries]
    ls = lse[:, t0q:t0q + n_queries].float()
    t0 = time.perf_counter()
    lmk = orc.mean_pool(k, S)
    idx, scores = orc.online_softmax_topk_head(qs.view(B, n_queries, H, HQ // H, D), lmk.bfloat16(), ls, K, S,
                                               W, q_offset=t0q)
    w = orc.inter_chunk_softmax(scores.reshape(B, n_queries, HQ, K), ls)
    orc.sparse_attn(qs, k, v, w, idx, chunk_size=S)
    dt = time.perf_counter() - t0
    return {"value": n_queries * B / dt, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{n_queries} consecutive queries at t={t0q} of the same 32K prefill inputs "
                      f"(pure-torch fp32 oracle: mean pool of all K, top-k, softmax, sparse attention), "
                      f"{dt:.2f} s", "seconds": dt}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-train", action="store_true", help="skip the config-5 forward+backward timing")
    ap.add_argument("--no-ops", action="store_true", help="skip the timings of the secondary operators")
    ap.add_argument("--no-prefill", action="store_true", help="profiling aid: decode step only")
    ap.add_argument("--train-only", action="store_true",
                    help="profiling aid: only the config-5 training layer forward+backward")
    ap.add_argument("--ops-only", action="store_true",
                    help="profiling aid: only the secondary operators (pooling, log-Z, sliding window, RoPE, HSA)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="profiling aid: run only a 512 MiB device copy (reference reading for the "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (no collectives are part of the hot "
                 "path); run with --gpus 1")
    entry.ensure_built()
    pkg = entry.load_package()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.copy_calibration:
        src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes": int(src.numel())}))
        return
    if args.train_only:
        print(json.dumps({"train_fwd_bwd": bench_train(pkg, dev)}))
        return
    if args.ops_only:
        print(json.dumps({"ops": bench_ops(pkg, dev)}))
        return
    if args.no_prefill:
        dsec, dper, droof = bench_decode(pkg, dev, max(args.steps, 20), args.warmup)
        print(json.dumps({"decode_us_per_step": dper["paged_step"] * 1e3,
                          "decode_token_major_cache_us": min(dsec * 1e6, dper["eager_step"] * 1e3),
                          "decode_graph_us": dsec * 1e6, "decode_kernel_ms": dper, "roofline_decode": droof}))
        return
    sec, per, roof, cfg, data = bench_prefill(pkg, dev, args.steps, args.warmup)
    tokens = cfg["global_batch"] * cfg["seq_len"]
    line = {
        "metric": "hils_attn_fwd_tokens_per_s_32k_prefill", "value": tokens / sec, "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (seeded N(0,1), per-head scale U[0.5,2] on q/k; lse_swa of the local chunk)",
        "config": cfg, "kernel_ms": per, "roofline": roof,
    }
    cpu = None if args.no_cpu else cpu_baseline(data)
    del data
    torch.cuda.empty_cache()
    if not args.no_decode:
        dsec, dper, droof = bench_decode(pkg, dev, max(args.steps, 20), args.warmup)
        # config 4 names a paged-contiguous K/V cache: the step on K, V pages of one chunk (pages handed out in
        # random order, the pooled keys per sequence: what HiLSPagedLayer keeps), eager launches on one stream.
        # The same step on the reference's (B, Lkv, H, D) cache tensors, eager and as one HIP-graph replay
        # (the faster of the two), is reported beside it.
        line["decode_us_per_step"] = dper["paged_step"] * 1e3
        line["decode_token_major_cache_us"] = min(dsec * 1e6, dper["eager_step"] * 1e3)
        line["decode_graph_us"] = dsec * 1e6
        line["decode_eager_us"] = dper["eager_step"] * 1e3
        line["decode_config"] = {"workload": "decode step B32 Lq1 Lkv131072 (2048 pooled keys) hq32/hkv8 D128 top32 "
                                             "(config 4), K and V in pages of one 64-token chunk",
                                 "timed_steps": max(args.steps, 200)}
        line["decode_kernel_ms"] = dper
        line["roofline_decode"] = droof
    if not args.no_train:
        line["config2_fwd"] = bench_config2(pkg, dev)
        line["train_fwd_bwd"] = bench_train(pkg, dev)
    if not args.no_ops:
        line["ops"] = bench_ops(pkg, dev)
    if cpu is not None:
        line["cpu_baseline"] = cpu
    print(json.dumps(line))


if __name__ == "__main__":
    main()
