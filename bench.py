#!/usr/bin/env python3
"""Benchmark of the GPT-OSS decode hot path on one MI355X.

One "step" = one pass of the MoE block (router GEMM, top-4 gating, stable grouping, grouped expert
GEMMs with clamped SwiGLU, weighted combine) over a batch of 1024 synthetic tokens at the
GPT-OSS-20B layer shape (hidden 2880, 32 experts, top-4, intermediate 2880), inputs and weights
resident in HBM.  Successive steps alternate between two independent sets of layer weights
(2 x 1.6 GB) so no cache level can keep them.

Prints ONE JSON line: the headline MoE-layer tokens/s with its roofline (dominant kernel = the
fused gather + GEMM1 + SwiGLU kernel, timed with HIP events on its launch stream) and the CPU
baseline (the CPU oracle restatement of the reference run.cpp MoE loop on a token slice), plus,
under "extra", the decode-attention HBM rates and the per-kernel breakdown.
"""
from __future__ import annotations

import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0         # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
GEMM1_KERNEL = "grouped_gemm_kernel<5, true, 1, false>"
GEMM1_TRAFFIC_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                                  "gemm1_bf16_20b_1024tok_hbm_traffic.txt")


def measured_traffic(workload):
    """HBM bytes of one launch of the roofline kernel, as two rocprofv3 --pmc runs of this command
    counted them (FETCH_SIZE and WRITE_SIZE, each scaled by what it reads for the 1 GiB copy
    below).  The figure is read from the committed counter summary and returned only if that
    summary is for this kernel on this workload; otherwise None."""
    try:
        kv = {}
        with open(GEMM1_TRAFFIC_FILE) as f:
            for line in f:
                if line.startswith("#") or ":" not in line:
                    continue
                k, v = line.split(":", 1)
                kv[k.strip()] = v.strip()
        if kv.get("kernel") != GEMM1_KERNEL:
            return None
        for k, v in workload.items():
            if int(kv[k]) != int(v):
                return None
        return int(kv["traffic_bytes"])
    except (OSError, KeyError, ValueError):
        return None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--tokens", type=int, default=1024)
    ap.add_argument("--cpu-tokens", type=int, default=1024,
                    help="token slice timed on the CPU baseline (0 = skip)")
    ap.add_argument("--no-attn", action="store_true", help="skip the decode-attention figures")
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end decode figure")
    ap.add_argument("--no-mxfp4", action="store_true", help="skip the 120B-shape MXFP4 MoE figure")
    ap.add_argument("--no-zipf", action="store_true",
                    help="skip the skewed-routing figure of the headline layer (profile runs: every "
                         "launch of the roofline kernel is then the headline workload)")
    ap.add_argument("--mfma-rates", action="store_true",
                    help="only measure the register-fed issue rate of the bf16 and the scaled f8f6f4 MFMA "
                         "(gptoss_diag_mfma_rate) and print one JSON line of its own")
    ap.add_argument("--no-sched", action="store_true", help="skip the scheduler leg of the end-to-end figure")
    return ap.parse_args()


def bench_moe(ops, torch, args):
    B, E, H, I, k = args.tokens, 32, 2880, 2880, 4
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(1234)

    def n(*shape, std=0.02):
        return (torch.randn(*shape, device=dev, generator=g) * std).to(torch.bfloat16)

    raw, layers = [], []
    for _ in range(2):
        w = dict(w_router=n(E, H), b_router=n(E), w1=n(E, 2 * I, H), b1=n(E, 2 * I),
                 w2=n(E, H, I), b2=n(E, H))
        layers.append(ops.MoeLayer(w["w_router"], w["b_router"], w["w1"], w["b1"], w["w2"],
                                   w["b2"], top_k=k, swiglu_limit=7.0, max_tokens=B))
        raw.append(w if not raw else None)      # keep one unpacked copy for the CPU baseline
        if raw[-1] is None:
            del w
    t = n(B, H, std=1.0)
    out = torch.empty(B, H, dtype=torch.float32, device=dev)

    for i in range(args.warmup):
        layers[i % 2].forward(t, out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        layers[i % 2].forward(t, out)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # same steps again with per-kernel HIP events on the launch stream
    trace = ops.KernelTrace(capacity=8 * args.steps + 8)
    with trace:
        for i in range(args.steps):
            layers[i % 2].forward(t, out)
    kern = trace.summary()

    zipf_res = None
    if not args.no_zipf:
        # the same layer under a skewed routing (what trained routers produce): a Zipf(1.1) bias over a
        # fixed permutation of the experts replaces the router bias, then the original bias is restored
        import numpy as np
        ranks = np.random.default_rng(5).permutation(E) + 1
        zipf = torch.from_numpy(np.log(1.0 / ranks ** 1.1).astype(np.float32)).to(dev)
        saved = [l.b_router.clone() for l in layers]
        for l in layers:
            l.b_router.copy_(zipf)
        for i in range(args.warmup):
            layers[i % 2].forward(t, out)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            layers[i % 2].forward(t, out)
        torch.cuda.synchronize()
        ms_zipf = (time.perf_counter() - t0) * 1e3 / args.steps
        counts = np.diff(layers[0].routing_views()[3].cpu().numpy())
        for l, b in zip(layers, saved):
            l.b_router.copy_(b)
        torch.cuda.synchronize()
        zipf_res = {"ms_per_step": round(ms_zipf, 5), "tokens_per_s": round(B / ms_zipf * 1e3, 1),
                    "rows_per_expert": {"min": int(counts.min()), "max": int(counts.max()),
                                        "above_160": int((counts > 160).sum())},
                    "config": "same layer and tokens, router bias replaced by log(rank^-1.1)"}

    flops = 2.0 * B * k * H * 3 * I + 2.0 * B * H * E
    w1_bytes = E * 2 * I * H * 2
    w2_bytes = E * H * I * 2
    # algorithmic bytes of one GEMM1 launch: W1 once + the B token rows once + the SwiGLU output
    gemm1_bytes = w1_bytes + B * H * 2 + B * k * I * 2
    gemm1_ms = kern["gemm1_gather_swiglu"][1]
    res = {
        "ms_per_step": ms,
        "tokens_per_s": B / ms * 1e3,
        "tflops": flops / ms / 1e9,
        "weight_gbs": (w1_bytes + w2_bytes) / ms / 1e6,
        "kernels_us": {name: round(v[1] * 1e3, 2) for name, v in kern.items()},
        "gemm1_ms": gemm1_ms,
        "gemm1_bytes": gemm1_bytes,
        "gemm1_flops": 2.0 * B * k * H * 2 * I,
        "zipf": zipf_res,
    }
    return res, (raw[0], t, layers[0], out)


def cpu_baseline_moe(torch, state, n_tok):
    """The oracle's restatement of run.cpp:625-704 on the first n_tok tokens, all host threads."""
    from oracle import oracle as orc
    raw, t, layer, _ = state
    f = lambda x: x.float().cpu().numpy()
    args = [f(raw[nm]) for nm in ("w_router", "b_router", "w1", "b1", "w2", "b2")]
    tt = f(t[:n_tok])
    t0 = time.perf_counter()
    want = orc.moe_layer(tt, *args, k=4, limit=7.0, stage=orc.STAGE_SWIGLU)
    dt = time.perf_counter() - t0
    # the timed sample doubles as a parity check of the benchmarked tensors
    got = layer.forward(t[:n_tok].contiguous()).cpu().numpy()
    import numpy as np
    d = np.abs(got - want)
    rel_max = float(d.max() / np.abs(want).max())
    rel_mean = float(d.mean() / np.abs(want).mean())
    return {"value": n_tok / dt, "unit": "tokens/s", "cores": orc.num_threads(), "kind": "port",
            "sample": f"first {n_tok} of the {t.shape[0]} tokens, same tensors, {dt:.1f} s",
            "parity_vs_gpu": {"max_rel": rel_max, "mean_rel": rel_mean}}


def _dequant_mxfp4(torch, blocks, scales):
    """e2m1 codes (low nibble = even element) times 2^(scale-127), one scale per 32 inputs -> fp32 on
    the host, expert by expert (export_model_bin/gpt-oss-20b/export_model_bin.py:66-123)."""
    lut = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6],
                       device=blocks.device)
    out = []
    for e in range(blocks.shape[0]):
        b = blocks[e]
        vals = torch.stack([lut[(b & 15).long()], lut[(b >> 4).long()]], -1).reshape(b.shape[0], -1)
        sc = torch.exp2(scales[e].float() - 127.0).repeat_interleave(32, dim=-1)
        out.append((vals * sc).cpu())
    return torch.stack(out).numpy()


def bench_moe_mxfp4_120b(ops, torch, steps, warmup, cpu_tokens=0):
    """configs[4]: MoE layer at the GPT-OSS-120B shape with MXFP4 expert weights: 4096 tokens, 128
    experts, top-4; FP4 codes uniform over the 16 values, one e8m0 scale per 32 inputs with exponent
    U{-8..0}; router bias Zipf(1.1) over a fixed permutation of the experts."""
    import numpy as np
    B, E, H, I, k = 4096, 128, 2880, 2880, 4
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(99)

    def n(*shape, std=0.02):
        return (torch.randn(*shape, device=dev, generator=g) * std).to(torch.bfloat16)

    def codes(*shape):
        return torch.randint(0, 256, shape, device=dev, generator=g, dtype=torch.uint8)

    def scales(*shape):
        return (127 - torch.randint(0, 9, shape, device=dev, generator=g)).to(torch.uint8)

    ranks = np.random.default_rng(5).permutation(E) + 1
    br = torch.from_numpy(np.log(1.0 / ranks ** 1.1).astype(np.float32)).to(dev)
    layers, raw = [], None
    for _ in range(2):
        w = (n(E, H), br, codes(E, 2 * I, H // 2), scales(E, 2 * I, H // 32), n(E, 2 * I),
             codes(E, H, I // 2), scales(E, H, I // 32), n(E, H))
        layers.append(ops.MoeLayerMxfp4(*w, top_k=k, swiglu_limit=7.0, max_tokens=B))
        if raw is None and cpu_tokens > 0:
            raw = w
        del w
    t = n(B, H, std=1.0)
    out = torch.empty(B, H, dtype=torch.float32, device=dev)
    for i in range(warmup):
        layers[i % 2].forward(t, out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        layers[i % 2].forward(t, out)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    trace = ops.KernelTrace(capacity=8 * steps + 8)
    with trace:
        for i in range(steps):
            layers[i % 2].forward(t, out)
    kern = trace.summary()
    counts = np.diff(layers[0].routing_views()[3].cpu().numpy())
    flops = 2.0 * B * k * H * 3 * I + 2.0 * B * H * E
    w_bytes = E * 3 * I * H * (0.5 + 1.0 / 32)
    cpu = None
    if raw is not None:
        # the oracle's MoE loop on the dequantised fp32 weights, first cpu_tokens tokens
        from oracle import oracle as orc
        f = lambda x: x.float().cpu().numpy()
        w1d, w2d = _dequant_mxfp4(torch, raw[2], raw[3]), _dequant_mxfp4(torch, raw[5], raw[6])
        tt = f(t[:cpu_tokens])
        t0 = time.perf_counter()
        want = orc.moe_layer(tt, f(raw[0]), f(raw[1]), w1d, f(raw[4]), w2d, f(raw[7]), k=k, limit=7.0,
                             stage=orc.STAGE_SWIGLU)
        dt = time.perf_counter() - t0
        got = layers[0].forward(t[:cpu_tokens].contiguous()).cpu().numpy()
        d = np.abs(got - want)
        cpu = {"value": round(cpu_tokens / dt, 2), "unit": "tokens/s", "cores": orc.num_threads(), "kind": "port",
               "sample": f"first {cpu_tokens} tokens on the dequantised fp32 weights, {dt:.1f} s",
               "parity_vs_gpu": {"max_rel": float(d.max() / np.abs(want).max()),
                                 "mean_rel": float(d.mean() / np.abs(want).mean())}}
        del w1d, w2d, raw
    del layers
    return {"cpu_baseline": cpu, "ms_per_step": round(ms, 4), "tokens_per_s": round(B / ms * 1e3, 1),
            "tflops": round(flops / ms / 1e9, 1),
            "mfma_bf16_frac": round(flops / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
            "weight_mb": round(w_bytes / 1e6, 1), "weight_gbs": round(w_bytes / ms / 1e6, 1),
            "weight_hbm_frac": round(w_bytes / ms / 1e6 / HBM_PEAK_GBS, 4),
            "rows_per_expert": {"min": int(counts.min()), "mean": float(counts.mean()), "max": int(counts.max())},
            "kernels_us": {name: round(v[1] * 1e3, 2) for name, v in kern.items()},
            "config": "4096 tokens, 128 experts top-4, hidden 2880, intermediate 2880, MXFP4 experts "
                      "(codes uniform, scale exponent U{-8..0}), Zipf(1.1) router bias, two weight sets alternated"}


def bench_attn(ops, torch, steps, warmup):
    import numpy as np
    B, n_q, n_kv, D, S = 256, 64, 8, 64, 4096
    rng = np.random.default_rng(0)
    lens_np = rng.integers(512, 4097, size=B).astype(np.int32)
    lens = torch.from_numpy(lens_np).cuda()
    caches = []
    for _ in range(2):
        c = ops.KVCache(B, n_kv, D, S)
        c.kv.normal_()
        caches.append(c)
    q = torch.randn(B, n_q, D, device="cuda")
    sinks = torch.randn(n_q, device="cuda")
    attn = ops.AttnDecode(B, n_q, n_kv, D, S)
    out = torch.empty(B, n_q, D, dtype=torch.bfloat16, device="cuda")
    res = {}
    for name, window in (("full", 0), ("window128", 128)):
        for i in range(warmup):
            attn.forward(q, caches[i % 2], lens, sinks, window=window, out=out)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            attn.forward(q, caches[i % 2], lens, sinks, window=window, out=out)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        act = np.minimum(lens_np, window) if window else lens_np
        kv_bytes = int(act.sum()) * n_kv * D * 2 * 2
        res[name] = {"us": round(ms * 1e3, 1), "kv_mb": round(kv_bytes / 1e6, 1),
                     "gbs": round(kv_bytes / ms / 1e6, 1),
                     "hbm_frac": round(kv_bytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    del caches, attn
    res["engine_shapes_position_383"] = bench_attn_engine_shapes(ops, torch, steps, warmup)
    res["prompt_attention"] = bench_attn_prompt(ops, torch)
    return res


def bench_attn_engine_shapes(ops, torch, steps, warmup):
    """The two attention calls of a layer pair of the whole-model decode step at its last position
    (configs[3]: 1024 sequences, position 383): a full layer (384 cached positions, one length for
    the batch) and a sliding-window layer (128-slot ring that has wrapped, every slot active)."""
    B, n_q, n_kv, D, pos = 1024, 64, 8, 64, 383
    q = torch.randn(B, n_q, D, device="cuda")
    sinks = torch.randn(n_q, device="cuda")
    out = torch.empty(B, n_q, D, dtype=torch.bfloat16, device="cuda")
    res = {}
    for name, cap, window in (("full_384", 384, 0), ("window_ring_128", 128, 128)):
        caches = []
        for _ in range(2):
            c = ops.KVCache(B, n_kv, D, cap)
            c.kv.normal_()
            caches.append(c)
        attn = ops.AttnDecode(B, n_q, n_kv, D, pos + 1)
        for i in range(warmup):
            attn.forward(q, caches[i % 2], None, sinks, window=window, out=out, max_len=pos + 1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            attn.forward(q, caches[i % 2], None, sinks, window=window, out=out, max_len=pos + 1)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        kv_bytes = B * min(pos + 1, cap) * n_kv * D * 2 * 2
        res[name] = {"us": round(ms * 1e3, 1), "kv_mb": round(kv_bytes / 1e6, 1),
                     "gbs": round(kv_bytes / ms / 1e6, 1),
                     "hbm_frac": round(kv_bytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
        del caches, attn
    return res


def bench_attn_prompt(ops, torch):
    """Prompt attention of one layer for 8192 rows: 64 prompts of 128 positions against 8 prompts of
    1024 positions (the reference's cap), full and with the 128-position window."""
    n_q, n_kv, D = 64, 8, 64
    res = {}
    for B, T in ((64, 128), (8, 1024)):
        q = torch.randn(B, T, n_q, D, device="cuda")
        cache = ops.KVCache(B, n_kv, D, T)
        cache.kv.normal_()
        sinks = torch.randn(n_q, device="cuda")
        pre = ops.AttnPrefill(B, T, n_q, n_kv, D, T)
        for name, window in (("full", 0), ("window128", 128)):
            for _ in range(3):
                pre.forward(q, cache, pos0=0, sinks=sinks, window=window)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                pre.forward(q, cache, pos0=0, sinks=sinks, window=window)
            e1.record()
            torch.cuda.synchronize()
            res[f"{B}x{T}_{name}_us"] = round(e0.elapsed_time(e1) * 100, 1)
        del q, cache, pre
    return res


def cpu_baseline_attn(ops, torch, n_seq=32):
    """configs[2] on the host: the oracle's restatement of run.cpp:562-607 (OpenMP over sequence and
    head) on n_seq sequences of the same shape, with the GPU result of the same tensors beside it."""
    import numpy as np
    from oracle import oracle as orc
    n_q, n_kv, D, S = 64, 8, 64, 4096
    rng = np.random.default_rng(1)
    lens_np = rng.integers(512, S + 1, size=n_seq).astype(np.int32)
    g = torch.Generator(device="cuda").manual_seed(7)
    k_rows = torch.randn(n_seq, S, n_kv, D, device="cuda", generator=g).to(torch.bfloat16)
    v_rows = torch.randn(n_seq, S, n_kv, D, device="cuda", generator=g).to(torch.bfloat16)
    q = torch.randn(n_seq, n_q, D, device="cuda", generator=g)
    sinks = torch.randn(n_q, device="cuda", generator=g)
    cache = ops.KVCache(n_seq, n_kv, D, S)
    cache.write(k_rows, v_rows, 0)
    attn = ops.AttnDecode(n_seq, n_q, n_kv, D, S)
    lens = torch.from_numpy(lens_np).cuda()
    kf, vf = k_rows.float().cpu().numpy(), v_rows.float().cpu().numpy()
    qf, sf = q.cpu().numpy(), sinks.cpu().numpy()
    res = {}
    for name, window in (("full", 0), ("window128", 128)):
        got = attn.forward(q, cache, lens, sinks, window=window).float().cpu().numpy()
        t0 = time.perf_counter()
        want = orc.attn_decode(qf, kf, vf, lens_np, sf, window=window)
        dt = time.perf_counter() - t0
        act = np.minimum(lens_np, window) if window else lens_np
        kv_bytes = int(act.sum()) * n_kv * D * 2 * 2
        d = np.abs(got - want)
        res[name] = {"gbs": round(kv_bytes / dt / 1e9, 2), "seconds": round(dt, 3),
                     "parity_vs_gpu": {"max_rel": float(d.max() / np.abs(want).max()),
                                       "mean_rel": float(d.mean() / np.abs(want).mean())}}
    res["cores"] = orc.num_threads()
    res["kind"] = "port"
    res["sample"] = f"{n_seq} sequences of the same shape (lengths U[512,4096]), bf16 KV bytes per second"
    return res


def bench_e2e(ops, torch, n_req=1024, n_prompt=128, n_decode=256, scheduler=True):
    """configs[3]: full GPT-OSS-20B shape, random-init bf16 weights generated on the device,
    1024 prompts of 128 random ids, then 256 greedy decode steps, all sequences in lock step (the
    reference's getp scheduling).  The prompt phase is timed both ways: forced token by token, as
    the reference does, and through the engine's prompt pass (128 positions per sequence at once);
    the decode figure is taken after the prompt pass."""
    import numpy as np
    synth = importlib.import_module("gpt-oss-team01_amd.synth")
    cfg = synth.gptoss20b_config(max_seq_len=n_prompt + n_decode)
    t0 = time.perf_counter()
    eng = ops.Engine(cfg, None, max_batch=n_req, max_seq=n_prompt + n_decode, synthetic=True, seed=1,
                     keep_logits=False)
    t_create = time.perf_counter() - t0
    rng = np.random.default_rng(3)
    prompts = rng.integers(0, cfg.vocab_size, size=(n_req, n_prompt), dtype=np.int32)
    tok = prompts[:, 0].copy()
    eng.step(tok, 0)                                   # warm-up of every kernel
    t0 = time.perf_counter()
    for pos in range(n_prompt - 1):                    # forced prompt positions, one step each
        eng.step(prompts[:, pos], pos)
    t_prompt = time.perf_counter() - t0
    eng.prefill(prompts[:64])                          # warm-up of the pass
    t0 = time.perf_counter()
    tok = eng.prefill(prompts)                         # all 128 positions of all 1024 prompts
    t_prefill = time.perf_counter() - t0
    t0 = time.perf_counter()
    for pos in range(n_prompt, n_prompt + n_decode):
        tok = eng.step(tok, pos)
    t_decode = time.perf_counter() - t0
    trace = ops.KernelTrace(capacity=2048)
    with trace:
        eng.step(tok, n_prompt + n_decode - 1)
    kern = trace.summary()
    trace = ops.KernelTrace(capacity=8192)
    with trace:
        eng.prefill(prompts[:64])                      # one pass of 64 x 128 = 8192 rows
    pkern = trace.summary()
    dev_gb = eng.device_bytes() / 1e9
    # Scheduler: 4096 requests (32-token prompts, length limits U[64, 384]) over the 1024 slots.
    # Continuous schedule (a finished sequence's slot takes the next request at once) against the
    # reference's batches of 1024 in lock step until the longest sequence of the batch ends.
    n_sched = 4 * n_req if scheduler else 0
    sp = rng.integers(0, cfg.vocab_size, size=(n_sched, 32), dtype=np.int32)
    limits = rng.integers(64, n_prompt + n_decode + 1, size=n_sched).astype(np.int32)
    useful = int((limits - 1).sum())
    t0 = time.perf_counter()
    if scheduler:
        eng.generate(sp, n_prompt + n_decode, max_len=limits)
    t_cont = time.perf_counter() - t0
    t0 = time.perf_counter()
    for b0 in range(0, n_sched, n_req):
        tok = sp[b0:b0 + n_req, 0].copy()
        for pos in range(int(limits[b0:b0 + n_req].max()) - 1):
            tok = eng.step(tok, pos)
    t_lock = time.perf_counter() - t0
    sched = {"requests": n_sched, "slots": n_req, "positions": useful,
             "continuous_tok_s": round(useful / t_cont, 1), "lockstep_batches_tok_s": round(useful / t_lock, 1),
             "workload": "32-token prompts, total length limits U[64,384]"} if scheduler else None
    eng.close()
    # The same model with the experts kept in MXFP4, as GPT-OSS checkpoints hold them (random codes
    # and scales here): same kernels' bf16 operands, a quarter of the expert bytes per step.
    eng = ops.Engine(cfg, None, max_batch=n_req, max_seq=n_prompt + n_decode, synthetic=True, seed=1,
                     keep_logits=False, mxfp4_experts=True)
    dev_gb_q = eng.device_bytes() / 1e9
    eng.prefill(prompts[:64])
    t0 = time.perf_counter()
    tok = eng.prefill(prompts)
    t_prefill_q = time.perf_counter() - t0
    t0 = time.perf_counter()
    for pos in range(n_prompt, n_prompt + n_decode):
        tok = eng.step(tok, pos)
    t_decode_q = time.perf_counter() - t0
    trace = ops.KernelTrace(capacity=2048)
    with trace:
        eng.step(tok, n_prompt + n_decode - 1)
    qkern = trace.summary()
    eng.close()
    mxfp4 = {"decode_tok_s": round(n_req * n_decode / t_decode_q, 1),
             "decode_ms_per_step": round(t_decode_q / n_decode * 1e3, 3),
             "prompt_tok_s_prefill": round(n_req * n_prompt / t_prefill_q, 1), "device_gb": round(dev_gb_q, 1),
             "last_step_kernels_us": {k: [c, round(ms * c * 1e3, 1)] for k, (c, ms) in qkern.items()},
             "weights": "experts MXFP4 (codes uniform, scale exponents U{-13..-5}), everything else as above"}
    return {"decode_tok_s": round(n_req * n_decode / t_decode, 1),
            "decode_ms_per_step": round(t_decode / n_decode * 1e3, 3),
            "prompt_tok_s_lockstep": round(n_req * (n_prompt - 1) / t_prompt, 1),
            "prompt_tok_s_prefill": round(n_req * n_prompt / t_prefill, 1),
            "prefill_ms": round(t_prefill * 1e3, 1),
            "total_tok_s": round(n_req * (n_prompt + n_decode) / (t_prefill + t_decode), 1),
            "engine_create_s": round(t_create, 1), "device_gb": round(dev_gb, 1),
            "last_step_kernels_us": {k: [c, round(ms * c * 1e3, 1)] for k, (c, ms) in kern.items()},
            "prefill_pass_8192_rows_kernels_us": {k: [c, round(ms * c * 1e3, 1)] for k, (c, ms) in pkern.items()},
            "scheduler": sched,
            "mxfp4_experts": mxfp4,
            "config": "24 blocks, hidden 2880, 64q/8kv heads x 64, 32 experts top-4, vocab 201088, "
                      "window 128 on even layers; 1024 seqs x (128 prompt + 256 decoded)"}


def bench_loader(ops, torch):
    """Loader: an fp32 payload in .bin tensor order with the GPT-OSS-20B dimensions and two blocks
    (11.2 GB in host memory) through gptoss_engine_create's pinned, double-buffered staging into the
    kernels' bf16 layouts; GB/s of fp32 payload, second of two runs."""
    import dataclasses
    import numpy as np
    synth = importlib.import_module("gpt-oss-team01_amd.synth")
    binfmt = importlib.import_module("gpt-oss-team01_amd.binfmt")
    cfg = dataclasses.replace(synth.gptoss20b_config(max_seq_len=64), n_layers=2)
    flat = np.empty(binfmt.n_weight_floats(cfg), np.float32)
    g = torch.Generator(device="cuda").manual_seed(5)
    off = 0
    for name, shape in binfmt.tensor_shapes(cfg).items():
        n = int(np.prod(shape))
        lead = shape[0] if len(shape) > 2 else 1
        per = n // lead
        for i in range(lead):
            x = torch.randn(per, device="cuda", generator=g) * 0.02
            flat[off + i * per: off + (i + 1) * per] = x.to(torch.bfloat16).float().cpu().numpy()
        off += n
    times = []
    for _ in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng = ops.Engine(cfg, flat, max_batch=1, max_seq=16, prefill=False, keep_logits=False)
        times.append(time.perf_counter() - t0)
        eng.close()
    return {"payload_gb": round(flat.nbytes / 1e9, 2), "seconds": round(times[-1], 3),
            "gbs": round(flat.nbytes / times[-1] / 1e9, 1),
            "what": "fp32 host payload (20B dimensions, 2 blocks) -> packed bf16 device weights, PCIe included"}


def bench_mfma_rates(torch):
    """Register-fed rate of the matrix instructions (no loads, no LDS): 256 workgroups of 8 waves."""
    import ctypes as C
    L = importlib.import_module("gpt-oss-team01_amd.lib")
    lib = L.load()
    sink = torch.zeros(16, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    names = ("bf16_32x32x16", "scaled_fp8_x_fp4_32x32x64", "scaled_fp4_x_fp4_32x32x64", "scaled_fp8_x_fp8_32x32x64")
    out = {}
    for kind, name in enumerate(names):
        flop = C.c_double(0)
        for timed in (False, True):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            L.check(lib.gptoss_diag_mfma_rate(kind, 256, 20000, sink.data_ptr(), C.byref(flop), stream))
            e1.record()
            torch.cuda.synchronize()
        ms = e0.elapsed_time(e1)
        out[name] = {"ms": round(ms, 3), "tflops": round(flop.value / ms / 1e9, 1)}
    return out


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.stderr.write("bench.py: this build runs on ONE GPU (all experts on one MI355X); "
                         "--gpus N with N > 1 is not supported\n")
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        sys.stderr.write("bench.py: no GPU visible; there is no CPU path to benchmark\n")
        sys.exit(3)
    importlib.import_module("gpt-oss-team01_amd.lib").load()
    ops = importlib.import_module("gpt-oss-team01_amd.ops")
    if args.mfma_rates:
        print(json.dumps({"what": "register-fed MFMA issue rates, 256 workgroups x 8 waves x 4 accumulators",
                          "rates": bench_mfma_rates(torch)}))
        return

    # a plain device copy of known size (2 x 1 GiB moved), so counter runs of this same command can
    # be scaled by what the counters read for it
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    # src and dst stay allocated until the end: see the note on memory handed back to the driver below

    moe, state = bench_moe(ops, torch, args)
    # The attention caches are allocated while the MoE tensors are still alive: memory handed back
    # to the driver and allocated again is laid out differently, which was measured to cost a
    # streaming kernel 3-4 % (an engine allocates its caches once, on fresh memory).
    attn = None
    if not args.no_attn:
        # a launch is ~0.2 ms: enough of them that the timed region is tens of milliseconds
        attn = bench_attn(ops, torch, max(100, 2 * args.steps), max(20, args.warmup))
    cpu = cpu_baseline_moe(torch, state, args.cpu_tokens) if args.cpu_tokens > 0 else None
    del state
    torch.cuda.empty_cache()
    extra = {"moe_tflops": round(moe["tflops"], 1),
             "moe_mfma_frac": round(moe["tflops"] / MFMA_BF16_PEAK_TFLOPS, 4),
             "moe_weight_gbs": round(moe["weight_gbs"], 1),
             "moe_weight_hbm_frac": round(moe["weight_gbs"] / HBM_PEAK_GBS, 4),
             "moe_kernels_us": moe["kernels_us"],
             "gemm1_tflops": round(moe["gemm1_flops"] / moe["gemm1_ms"] / 1e9, 1),
             "moe_zipf_routing": moe["zipf"]}
    if attn is not None:
        extra["decode_attn"] = attn
        if args.cpu_tokens > 0:
            extra["decode_attn"]["cpu_baseline"] = cpu_baseline_attn(ops, torch)

    if not args.no_mxfp4:
        torch.cuda.empty_cache()
        extra["moe_120b_mxfp4"] = bench_moe_mxfp4_120b(ops, torch, max(10, args.steps // 2), args.warmup,
                                                       cpu_tokens=min(64, args.cpu_tokens))
    if not args.no_e2e:
        torch.cuda.empty_cache()
        extra["e2e_20b"] = bench_e2e(ops, torch, scheduler=not args.no_sched)
        torch.cuda.empty_cache()
        extra["loader"] = bench_loader(ops, torch)

    if cpu is not None and "e2e_20b" in extra:
        # whole-model CPU figure: not run (84 GB of fp32 weights, minutes per token); scaled from the
        # measured CPU MoE-layer rate by FLOPs per token (24 blocks of MoE 199 + projections 53 MFLOP,
        # plus the 1158 MFLOP unembedding)
        per_tok_s = (1.0 / cpu["value"]) * (24 * (199.1 + 53.1) + 1158.3) / 199.1
        extra["e2e_20b"]["cpu_baseline"] = {"value": round(1.0 / per_tok_s, 2), "unit": "tokens/s",
                                            "cores": cpu["cores"], "kind": "port",
                                            "sample": "extrapolated from the measured CPU MoE-layer rate by FLOPs per token"}
    achieved = moe["gemm1_bytes"] / moe["gemm1_ms"] / 1e6
    line = {
        "metric": "MoE-layer tokens/s (GPT-OSS-20B layer shape, 1024 tokens, 1 GPU)",
        "value": round(moe["tokens_per_s"], 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(moe["ms_per_step"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "configs[1]: single GPT-OSS-20B MoE layer, isolated",
                   "tokens": args.tokens, "hidden": 2880, "experts": 32, "top_k": 4,
                   "intermediate": 2880, "weights": "bf16 N(0,0.02), two sets alternated",
                   "activations": "bf16 N(0,1)"},
        "roofline": {"kernel": GEMM1_KERNEL + " (gather + GEMM1 + SwiGLU)",
                     "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic({"tokens": args.tokens, "hidden": 2880,
                                                  "intermediate": 2880, "experts": 32,
                                                  "top_k": 4}),
                     "bytes_per_launch": moe["gemm1_bytes"],
                     "avg_launch_us": round(moe["gemm1_ms"] * 1e3, 2)},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
