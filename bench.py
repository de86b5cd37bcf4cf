#!/usr/bin/env python3
"""Benchmark of the quantized-MoE decode hot path on one MI355X.

A step is one MoE-layer decode step (router -> top-8 -> routed experts gate/up SwiGLU and down,
shared expert with sigmoid gate, weighted combine) over one batch of synthetic tokens, through the
C ABI (nvmai_hip_moe_decode_layer).  The workload is BASELINE.json configs[1]: 8-bit group-64
weights, hidden 2048, 256 experts top-8, intermediate 512, all experts resident in HBM.  Steps
rotate over `--layers` independent layers and over different token batches so that expert reads
come from HBM, not from L2 or the 256 MB Infinity Cache.

Prints ONE JSON line.  `value` is algorithmic bytes / wall time of the timed region; the roofline
object prices the dominant kernel (routed gate/up SwiGLU) by HIP events recorded on its stream.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

D, F, E, K = 2048, 512, 256, 8
HBM_PEAK_GBPS = 8000.0
METRIC = "4/8-bit MoE expert GEMV GB/s (% HBM peak); prefill grouped-GEMM TFLOPS"
RAMP_STEPS = 200       # untimed steps ahead of the --warmup steps of the decode workload: a fresh device takes a few
                       # milliseconds of work to reach its clock, and --steps 20 of this workload are under 3 ms


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--batch", type=int, default=32, help="tokens per decode step (1..32)")
    ap.add_argument("--bits", type=int, default=None, choices=[4, 8], help="default 8 (4 for --workload prefill)")
    ap.add_argument("--layers", type=int, default=40)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--sweep", action="store_true", help="also print batch/bits sweep lines to stderr")
    ap.add_argument("--no-extra", action="store_true", help="skip the `extra` object (the other cells of the metric) "
                    "that the default invocation appends")
    ap.add_argument("--workload", default="decode", choices=["decode", "prefill", "attention", "prefill_attention", "sampler", "greedy", "step", "prefill_step", "copy", "read"],
                    help="decode = configs[1] (the headline line); prefill = configs[2] grouped GEMM; "
                         "attention = configs[3] quantized-KV decode attention; prefill_attention = causal attention of --tokens queries "
                         "at the end of a --context cache; sampler = the end of configs[4]: "
                         "quantized LM head GEMV over 248,320 rows, tiled softmax, top-k sampler; greedy = the fused greedy LM head "
                         "(RMSNorm + logits in a fixed order + argmax) over the same head; step = configs[4], the full 40-layer decode "
                         "step (tok/s at --batch 1..16, KV at --context); prefill_step = --tokens prompt tokens of one sequence through the "
                         "same 40 layers with the prefill kernels, in chunks of --chunk; copy = a plain 1 GiB device copy, "
                         "the known-size kernel the FETCH_SIZE / WRITE_SIZE counters are calibrated on")
    ap.add_argument("--context", type=int, default=None, help="attention: tokens in the KV cache (default 32768; "
                    "prefill_attention: the chunk itself)")
    ap.add_argument("--tokens", type=int, default=4096, help="prefill: tokens per step")
    ap.add_argument("--chunk", type=int, default=4096, help="prefill_step: tokens per chunk")
    a = ap.parse_args()
    if a.bits is None:
        a.bits = 4 if a.workload == "prefill" else 8
    a.context_given = a.context is not None
    if a.context is None:
        a.context = 32768
    return a


def build_layers(nv, ctx, torch, bits, n_layers, seed=1234):
    """Random-init layers: bf16 N(0, 0.02) weights quantized on the device into expert blobs."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    off, stride = nv.expert_offsets(D, F, bits)
    layers = []
    for _ in range(n_layers):
        pool = torch.empty((E + 1, stride), dtype=torch.uint8, device="cuda")
        # one big matrix per role, quantized in one launch, then scattered into the blobs
        for (rows, n, wo, so, bo) in ((F, D, off.gate_w, off.gate_s, off.gate_b),
                                      (F, D, off.up_w, off.up_s, off.up_b),
                                      (D, F, off.down_w, off.down_s, off.down_b)):
            w = torch.empty(((E + 1) * rows, n), dtype=torch.bfloat16, device="cuda")
            w.normal_(0.0, 0.02, generator=gen)
            p, s, b = nv.quantize_affine(ctx, w, bits)
            wb, mb = rows * n * bits // 8, rows * n // 32
            pool[:, wo:wo + wb] = p.view(E + 1, wb)
            pool[:, so:so + mb] = s.view(torch.uint8).view(E + 1, mb)
            pool[:, bo:bo + mb] = b.view(torch.uint8).view(E + 1, mb)
            del w, p, s, b
        router = torch.empty((E, D), dtype=torch.bfloat16, device="cuda").normal_(0.0, 0.02, generator=gen)
        gate_w = torch.empty((1, D), dtype=torch.bfloat16, device="cuda").normal_(0.0, 0.02, generator=gen)
        gq = nv.quantize_affine(ctx, gate_w, 8)
        desc = nv.moe_layer_desc(D, F, E, K, bits, nv.rows_desc(16, router), pool[:E], pool[E],
                                 nv.rows_desc(8, *gq))
        layers.append(dict(desc=desc, pool=pool, router=router, gate=gq))
    return layers, stride


def step_bytes(distinct, batch, stride):
    """Algorithmic bytes of one step: each distinct routed expert once, the shared expert, the
    dense bf16 router, the 8-bit gate row, activations in and out."""
    return distinct * stride + stride + E * D * 2 + (D + 2 * (D // 64) * 2) + batch * (D * 2 + D * 2)


def run_config(nv, ctx, torch, layers, stride, bits, batch, steps, warmup, profile):
    moe = nv.MoE(ctx, bits)
    n_x = 64
    gen = torch.Generator(device="cuda").manual_seed(99 + batch)
    xs = torch.empty((n_x, batch, D), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
    y = torch.empty((batch, D), dtype=torch.bfloat16, device="cuda")
    stats = torch.zeros((steps, 2), dtype=torch.int32, device="cuda")
    for i in range(RAMP_STEPS + warmup):                    # untimed: the clock ramp, then the warm-up steps asked for
        moe.decode_layer(layers[i % len(layers)]["desc"], xs[i % n_x], y)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        moe.decode_layer(layers[i % len(layers)]["desc"], xs[i % n_x], y, stats=stats[i])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    distinct = stats[:, 1].cpu().numpy().astype(np.int64)
    total = float(sum(step_bytes(int(u), batch, stride) for u in distinct))
    out = dict(seconds=dt, bytes=total, gbps=total / dt / 1e9, ms_per_step=dt / steps * 1e3,
               mean_distinct=float(distinct.mean()))
    if profile:
        # second pass with per-kernel events on the launch stream
        ctx.profile_enable(True)
        for i in range(steps):
            moe.decode_layer(layers[i % len(layers)]["desc"], xs[i % n_x], y)
        torch.cuda.synchronize()
        ctx.profile_enable(False)
        names = ["router", "select", "group", "phase1", "phase2", "combine"]
        kern = {}
        for tag, name in enumerate(names):
            ms, n = ctx.profile_read(tag)
            kern[name] = ms / max(n, 1) * 1e3      # microseconds per launch
        out["kernel_us"] = kern
        # phase 1 streams gate+up of every distinct routed expert and of the shared expert
        gate_up = 2 * (F * D * bits // 8 + 2 * F * (D // 64) * 2)
        p1_bytes = float(np.mean((distinct + 1) * gate_up + batch * D * 2 + (distinct + 1) * F * 4))
        out["phase1_bytes"] = p1_bytes
        out["phase1_gbps"] = p1_bytes / (kern["phase1"] * 1e-6) / 1e9
    return out


def cpu_baseline(layers, stride, bits, batch, torch):
    """The CPU oracle (a C port of the reference's CPU path, rebuilt here at -O3 -march=native) on a
    bounded sample of the same workload: one decode step of layer 0, timed inside the C library
    (median of the repetitions), on one thread over the first 8 tokens and on all host cores over
    the whole batch (tokens shared out over the threads: the reference kernel has no threads of
    its own)."""
    import oracle as O
    L = layers[0]
    pool = L["pool"].cpu().numpy()
    router = L["router"].view(torch.int16).cpu().numpy().view(np.uint16)
    gq = [t.cpu().numpy() for t in L["gate"]]
    gate = (8, gq[0], gq[1].view(np.uint16), gq[2].view(np.uint16))
    rng = np.random.default_rng(7)
    model, cores = O.host_cpu()
    _, flags = O.timing_lib()
    x = O.round_bf16(rng.standard_normal((max(batch, cores), D)).astype(np.float32))
    rows = {}
    for name, n, threads, reps in (("one_thread", min(batch, 8), 1, 21), ("all_cores", max(batch, cores), cores, 41)):
        dt, idx = O.time_moe_layer(x[:n], D, F, K, bits, (16, router, None, None), pool[:E], pool[E], gate,
                                   threads, warmup=1, reps=reps)
        algo = step_bytes(len(np.unique(idx)), n, stride)
        rows[name] = dict(value=round(algo / dt / 1e9, 3), unit="GB/s", cores=threads,
                          sample="%d tokens, one %d-bit layer, median of %d x %.3f s; %.0f MB algorithmic, %.0f MB touched per pair"
                                 % (n, bits, reps, dt, algo / 1e6, (n * (K + 1) * stride + n * E * D * 2) / 1e6))
    out = dict(rows["all_cores"])
    out.update(kind="port", cpu_model=model, build="oracle/nvmai_oracle.c, gcc " + flags,
               one_thread_value=rows["one_thread"]["value"], one_thread_sample=rows["one_thread"]["sample"])
    out["sample"] = "orc_moe_layer_forward, " + out["sample"]
    return out


MFMA_BF16_PEAK_TFLOPS = 2500.0

# HBM bytes per launch of the roofline kernel: RECORDED figures from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE runs of this file (KiB per dispatch, FETCH_SIZE scaled x2.00 and WRITE_SIZE x1.00 after
# calibration on `--workload copy`), not something this run measures; each comes with the summary
# under profiles/ it was read from and goes stale when its kernel changes.  Keyed by (workload,
# bits, batch or tokens); other configurations report null.
MEASURED_TRAFFIC_BYTES = {
    ("decode", 8, 32): ((181300 * 2.00 + 1229 * 1.00) * 1024, "profiles/expert_rows_fast_decode_configs1_8bit_batch32.txt"),
    ("prefill", 4, 4096): ((246530 * 2.00 + 36144 * 1.00) * 1024, "profiles/prefill_gemm_kernel_configs2_4bit_4096tokens.txt"),
    ("attention", 8, 8, 131072): ((557830 * 2.00 + 2176 * 1.00) * 1024, "profiles/attn_partial_mfma_kernel_configs3_8bit_128k_batch8.txt"),
    ("attention", 4, 8, 131072): ((295590 * 2.00 + 4362 * 1.00) * 1024, "profiles/attn_partial_mfma_kernel_configs3_4bit_128k_batch8.txt"),
}


def recorded_traffic(key):
    """(bytes or None, source or None) for a roofline object."""
    return MEASURED_TRAFFIC_BYTES.get(key, (None, None))


def run_prefill(nv, ctx, torch, a):
    """configs[2]: 4096 tokens, top-8 of 256 experts with Zipf(1.1) popularity, 4-bit experts.
    A step = grouping by expert + gate/up SwiGLU GEMM + down GEMM + rank-order reduce."""
    bits, T = a.bits, a.tokens
    layers, stride = build_layers(nv, ctx, torch, bits, 1)
    pool = layers[0]["pool"][:E]
    off, _ = nv.expert_offsets(D, F, bits)
    gen = torch.Generator(device="cuda").manual_seed(4242)
    n_x = 4
    xs = torch.empty((n_x, T, D), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
    # router logits = log popularity + Gumbel noise: top-8 then samples experts without
    # replacement with probability proportional to a Zipf(1.1) law over a random expert order
    pop = 1.0 / torch.arange(1, E + 1, device="cuda", dtype=torch.float32) ** 1.1
    pop = pop[torch.randperm(E, device="cuda", generator=gen)]
    u = torch.rand((n_x, T, E), device="cuda", generator=gen).clamp_(1e-9, 1.0)
    logits = torch.log(pop)[None, None, :] - torch.log(-torch.log(u))
    top = torch.topk(logits, K, dim=-1)
    idx = top.indices.to(torch.int32).contiguous()
    w = torch.softmax(top.values, dim=-1).to(torch.float16).contiguous()
    grouping, moe, red = nv.PrefillMoEGrouping(ctx), nv.PrefillGroupedRoutedMoE(ctx, bits), nv.PrefillMoE(ctx)
    act = torch.empty((T * K, F), dtype=torch.bfloat16, device="cuda")
    partials = torch.empty((T * K, D), dtype=torch.bfloat16, device="cuda")
    h2 = torch.empty((T, D), dtype=torch.bfloat16, device="cuda")

    def step(i):
        j = i % n_x
        routes = grouping.group_routes(idx[j], w[j], E)
        moe.encode(pool, off, xs[j], D, F, routes, act, partials)
        red.encode_reduce_token_major(partials, w[j], T, K, D, h2)
        return routes

    for i in range(a.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(i)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / a.steps
    ctx.profile_enable(True)
    for i in range(a.steps):
        step(i)
    torch.cuda.synchronize()
    ctx.profile_enable(False)
    kern = {}
    for tag, name in ((nv.PROF_PREFILL_GROUP, "group"), (nv.PROF_PREFILL_GEMM1, "gemm_gate_up"),
                      (nv.PROF_PREFILL_GEMM2, "gemm_down"), (nv.PROF_PREFILL_COMBINE, "reduce")):
        ms, n = ctx.profile_read(tag)
        kern[name] = ms / max(n, 1) * 1e3
    flops = T * K * 6.0 * D * F
    g1 = T * K * 4.0 * D * F / (kern["gemm_gate_up"] * 1e-6) / 1e12
    counts = step(0).per_expert_counts.cpu().numpy()
    # the router + top-k that precedes the step in a layer (not part of the step or of `value`:
    # the step's routes follow the Zipf law above): bf16 router matrix over the same hidden rows
    rw = torch.empty((E, D), dtype=torch.bfloat16, device="cuda").normal_(0.0, 0.02, generator=gen)
    rdesc, rmoe = nv.rows_desc(16, rw.view(torch.int16)), nv.MoE(ctx, bits)
    for _ in range(3):
        rmoe.encode_router(rdesc, xs[0], E, D, K)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(10):
        rmoe.encode_router(rdesc, xs[i % n_x], E, D, K)
    torch.cuda.synchronize()
    router_us = (time.perf_counter() - t0) / 10 * 1e6
    # what a plain dense bf16 GEMM of the library that ships with torch reaches on this device
    A = torch.empty((8192, 8192), dtype=torch.bfloat16, device="cuda").normal_(0, 1, generator=gen)
    B = torch.empty((8192, 8192), dtype=torch.bfloat16, device="cuda").normal_(0, 1, generator=gen)
    for _ in range(3):
        A @ B
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(10):
        A @ B
    torch.cuda.synchronize()
    dense = 10 * 2.0 * 8192 ** 3 / (time.perf_counter() - t0) / 1e12
    del A, B
    cpu = None
    if not a.no_cpu:
        import oracle as O
        model, cores = O.host_cpu()
        _, flags = O.timing_lib()
        blobs = pool.cpu().numpy()
        rows = {}
        for name, n, threads, reps in (("one_thread", 4, 1, 5), ("all_cores", 4 * cores, cores, 5)):
            x0 = xs[0, :n].float().cpu().numpy()     # the first tokens of the same step on the CPU oracle
            i0 = idx[0, :n].cpu().numpy().astype(np.uint32)
            w0 = w[0, :n].view(torch.int16).cpu().numpy().view(np.uint16)
            dtc = O.time_prefill_moe(blobs, bits, x0, D, F, i0, w0, threads, warmup=1, reps=reps)
            rows[name] = dict(value=n * K * 6.0 * D * F / dtc / 1e12, unit="TFLOP/s", cores=threads,
                              sample="%d tokens x top-%d of the same step, median of %d repetitions of %.3f s"
                                     % (n, K, reps, dtc))
        cpu = dict(rows["all_cores"])
        cpu.update(kind="port", cpu_model=model, build="oracle/nvmai_oracle.c, gcc " + flags, one_thread=rows["one_thread"])
        cpu["sample"] = "oracle orc_prefill_moe, " + cpu["sample"]
    return {
        "metric": METRIC, "value": round(flops / dt / 1e12, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u%d codes -> bf16 MFMA, f32 accumulate" % bits, "data": "synthetic",
        "config": {"workload": "configs[2]: MoE prefill grouped GEMM, %d tokens x hidden 2048, top-8 of 256 experts "
                               "(Zipf 1.1 popularity), %d-bit group-64 experts, intermediate 512" % (T, bits),
                   "tokens_per_s": round(T / dt), "largest_expert_pairs": int(counts.max()),
                   "experts_hit": int((counts > 0).sum()),
                   "dense_bf16_gemm_8192_tflops": round(dense, 1),
                   "kernel_us": {k: round(v, 2) for k, v in kern.items()},
                   "router_topk_us_outside_the_step": round(router_us, 1)},
        "roofline": {"kernel": "prefill_gemm_kernel<DUAL> (gate/up + SwiGLU)", "bound": "mfma",
                     "achieved": round(g1, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(g1 / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": recorded_traffic(("prefill", bits, T))[0],
                     "traffic_source": recorded_traffic(("prefill", bits, T))[1],
                     "flops_per_launch": T * K * 4.0 * D * F, "avg_launch_us": round(kern["gemm_gate_up"], 2)},
        "cpu_baseline": cpu,
    }


def run_attention(nv, ctx, torch, a):
    """configs[3]: 16 query heads, 2 KV heads, head_dim 256, KV quantized on write; a step = one
    decode attention call over `--context` cached tokens for `--batch` sequences."""
    bits, B, ctx_len = a.bits, min(a.batch, 8), a.context
    HQ, HKV, HD = 16, 2, 256
    gen = torch.Generator(device="cuda").manual_seed(31)
    n_sets = max(1, min(8, int(1.5e9 // (2 * B * ctx_len * 600))))      # rotate caches past L2 / MALL
    quant, att = nv.KVCacheQuantizer(ctx), nv.Attention(ctx)
    caches = []
    for _ in range(n_sets):
        kc, vc = nv.KVCache(B, ctx_len, HKV * HD, bits), nv.KVCache(B, ctx_len, HKV * HD, bits)
        for b in range(B):
            for start in range(0, ctx_len, 8192):
                n = min(8192, ctx_len - start)
                for c in (kc, vc):
                    src = torch.empty((n, HKV * HD), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
                    quant.encode(src, HKV * HD, c.view(b, start), n, HKV * HD)
        caches.append((kc, vc))
    q = torch.empty((B, HQ, HD), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
    out = torch.empty_like(q)
    for i in range(a.warmup):
        att.encode_full(q, *caches[i % n_sets], HD, HQ, HKV, ctx_len, out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        att.encode_full(q, *caches[i % n_sets], HD, HQ, HKV, ctx_len, out=out)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / a.steps
    ctx.profile_enable(True)
    for i in range(a.steps):
        att.encode_full(q, *caches[i % n_sets], HD, HQ, HKV, ctx_len, out=out)
    torch.cuda.synchronize()
    ctx.profile_enable(False)
    kern = {}
    for tag, name in ((nv.PROF_ATTN_PARTIAL, "partial"), (nv.PROF_ATTN_COMBINE, "combine")):
        ms, n = ctx.profile_read(tag)
        kern[name] = ms / max(n, 1) * 1e3
    # quantize-on-write of 8192-token blocks (the prefill-side use), K and V
    srcq = torch.empty((8192, HKV * HD), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
    nq = min(8192, ctx_len)
    ctx.profile_enable(True)
    for i in range(20):
        quant.encode(srcq, HKV * HD, caches[0][i % 2].view(0, 0), nq, HKV * HD)
    torch.cuda.synchronize()
    ctx.profile_enable(False)
    ms, n = ctx.profile_read(nv.PROF_KV_QUANT)
    kern["kv_quantize_%d_tokens" % nq] = ms / max(n, 1) * 1e3
    stride = caches[0][0].stride
    cpu = None
    parity = None
    if True:
        import oracle as O
        # the numbers above are only worth printing if the kernel is right at this size: the last
        # 4096 positions of sequence 0 (a start offset deep in the cache) against the oracle
        start = max(0, ctx_len - 4096)
        got = att.encode_full(q[:1], caches[0][0], caches[0][1], HD, HQ, HKV, ctx_len, kv_start=start)
        torch.cuda.synchronize()
        kr = caches[0][0].rows[0].cpu().numpy()
        vr = caches[0][1].rows[0].cpu().numpy()
        want = O.attention_decode(q[0].float().cpu().numpy(), kr, vr, bits, HQ, HKV, HD, ctx_len, 1.0 / 16.0, start)
        rel = float(O.rel_error(got[0].float().cpu().numpy(), want))
        assert rel < 1e-2, "attention differs from the oracle at context %d: max-rel %g" % (ctx_len, rel)
        parity = {"max_rel": round(rel, 6), "against": "oracle attention_decode, sequence 0, positions %d..%d" % (start, ctx_len)}
    if not a.no_cpu:
        model, cores = O.host_cpu()
        _, flags = O.timing_lib()
        n = min(ctx_len, 8192)                          # first rows of the sequences on the CPU oracle
        nb = max(1, min(B, cores))
        krs = np.stack([caches[0][0].rows[b, :n].cpu().numpy() for b in range(nb)])
        vrs = np.stack([caches[0][1].rows[b, :n].cpu().numpy() for b in range(nb)])
        qs = q[:nb].float().cpu().numpy()
        rows = {}
        for name, seqs, threads in (("one_thread", 1, 1), ("all_cores", nb, nb)):
            dtc = O.time_attention(qs[:seqs], krs[:seqs], vrs[:seqs], bits, HQ, HKV, HD, n, 1.0 / 16.0, threads,
                                   warmup=1, reps=5)
            rows[name] = dict(value=2.0 * seqs * n * stride / dtc / 1e9, unit="GB/s", cores=threads,
                              sample="%d sequence(s) of %d cached tokens, one thread per sequence, median of 5 "
                                     "repetitions of %.3f s" % (seqs, n, dtc))
        cpu = dict(rows["all_cores"])
        cpu.update(kind="port", cpu_model=model, build="oracle/nvmai_oracle.c, gcc " + flags, one_thread=rows["one_thread"])
        cpu["sample"] = "oracle orc_attention_decode, " + cpu["sample"]
    kv_bytes = 2.0 * B * ctx_len * stride
    step_b = kv_bytes + 2 * B * HQ * HD * 2
    part = kv_bytes / (kern["partial"] * 1e-6) / 1e9
    return {
        "metric": METRIC, "value": round(step_b / dt / 1e9, 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(dt * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u%d KV codes, f16 MFMA, f32 softmax" % bits, "data": "synthetic",
        "config": {"workload": "configs[3]: GQA decode attention, 16 query / 2 KV heads, head_dim 256, %d-bit KV "
                               "(group 64, fp16 scale/bias), context %d, batch %d" % (bits, ctx_len, B),
                   "frac_of_hbm_peak": round(step_b / dt / 1e9 / HBM_PEAK_GBPS, 4), "cache_sets_rotated": n_sets,
                   "kv_quantize_gbps": round(nq * (HKV * HD * 2 + caches[0][0].stride) /
                                             (kern["kv_quantize_%d_tokens" % nq] * 1e-6) / 1e9, 1),
                   "kernel_us": {k: round(v, 2) for k, v in kern.items()}},
        "roofline": {"kernel": "attn_partial_mfma_kernel", "bound": "hbm", "achieved": round(part, 2),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(part / HBM_PEAK_GBPS, 4),
                     "traffic": recorded_traffic(("attention", bits, B, ctx_len))[0],
                     "traffic_source": recorded_traffic(("attention", bits, B, ctx_len))[1],
                     "bytes_per_launch": kv_bytes, "avg_launch_us": round(kern["partial"], 2)},
        "cpu_baseline": cpu, "parity_check": parity,
    }


def run_prefill_attention(nv, ctx, torch, a):
    """The attention half of a configs[2] prefill step: `--tokens` query tokens (16 query / 2 KV
    heads, head_dim 256) at the end of a quantized KV cache of `--context` tokens (at least the
    chunk itself), causal.  A step = one PrefillAttention.encodeCausal call."""
    bits, T = a.bits, a.tokens
    HQ, HKV, HD = 16, 2, 256
    kv_valid = max(a.context, T) if a.context_given else T
    start = kv_valid - T
    gen = torch.Generator(device="cuda").manual_seed(37)
    quant, pa = nv.KVCacheQuantizer(ctx), nv.PrefillAttention(ctx)
    kc, vc = nv.KVCache(1, kv_valid, HKV * HD, bits), nv.KVCache(1, kv_valid, HKV * HD, bits)
    for at in range(0, kv_valid, 8192):
        n = min(8192, kv_valid - at)
        for c in (kc, vc):
            src = torch.empty((n, HKV * HD), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
            quant.encode(src, HKV * HD, c.view(0, at), n, HKV * HD)
    q = torch.empty((T, HQ, HD), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
    out = torch.empty_like(q)
    call = lambda: pa.encode_causal(q, kc.view(), vc.view(), out, start, T, HD, HQ, HKV, kv_valid)
    for _ in range(a.warmup):
        call()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        call()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / a.steps
    ctx.profile_enable(True)
    for _ in range(a.steps):
        call()
    torch.cuda.synchronize()
    ctx.profile_enable(False)
    ms, n = ctx.profile_read(nv.PROF_ATTN_PARTIAL)
    kern_us = ms / max(n, 1) * 1e3
    import oracle as O
    kr, vr = kc.rows[0].cpu().numpy(), vc.rows[0].cpu().numpy()
    rows = sorted({0, 1, T // 2, T - 1}) if kv_valid <= 16384 else [0, T - 1]
    worst = 0.0
    for t in rows:                                     # the oracle walks one query's keys in about a second at 128K
        want = O.attention_prefill_causal(q[t].float().cpu().numpy().reshape(1, -1), kr, vr, bits, HQ, HKV, HD,
                                          start + t, start + t + 1, 1.0 / 16.0)
        worst = max(worst, float(O.rel_error(out[t].float().cpu().numpy(), want)))
    assert worst < 1e-2, "prefill attention differs from the oracle: max-rel %g" % worst
    pairs = float(sum(min(kv_valid, start + t + 1) for t in range(T)))
    flops = 4.0 * pairs * HD * HQ                      # q.k and p.v, one multiply-add each per (query, key, head, dim)
    tf = flops / (kern_us * 1e-6) / 1e12
    return {
        "metric": METRIC, "value": round(flops / dt / 1e12, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u%d KV codes, f16 MFMA, f32 softmax" % bits, "data": "synthetic",
        "config": {"workload": "attention of a configs[2] prefill step: causal, %d query tokens at positions %d..%d, "
                               "16 query / 2 KV heads, head_dim 256, %d-bit KV" % (T, start, kv_valid - 1, bits),
                   "tokens_per_s": round(T / dt), "query_key_pairs": pairs},
        "roofline": {"kernel": ("attn_prefill_dequant_kernel + attn_prefill_fa_kernel (the key range dequantized once into "
                                "fp16 scratch, then flash attention)" if T * HQ >= 16384 else
                                "attn_partial_mfma_kernel (causal, %d queries per block)" % (16 // (HQ // HKV))),
                     "bound": "mfma", "achieved": round(tf, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "flops_per_launch": flops, "avg_launch_us": round(kern_us, 2)},
        "cpu_baseline": None,
        "parity_check": {"max_rel": round(worst, 6), "against": "oracle attention_prefill_causal, query rows %s" % rows},
    }


def run_sampler(nv, ctx, torch, a):
    """The end of configs[4]: logits = LM head (4/8-bit affine [248320, 2048]) x hidden, softcap +
    tiled softmax, tiled top-k sampler (k 20, top-p 0.95, T 0.6, fixed seed) for `--batch` rows."""
    V, bits, rows = 248320, a.bits, min(a.batch, 32)
    gen = torch.Generator(device="cuda").manual_seed(77)
    n_heads = 4                                            # rotate copies of the head past the caches
    heads = []
    for _ in range(n_heads):
        wt = torch.empty((V, D), dtype=torch.bfloat16, device="cuda").normal_(0.0, 0.02, generator=gen)
        heads.append(nv.quantize_affine(ctx, wt, bits))
        del wt
    xs = torch.empty((8, rows, D), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
    sm, tk = nv.LogitSoftcapSoftmaxTiled(ctx, V), nv.SampleTopK64(ctx, V)
    probs = torch.empty((rows, V), dtype=torch.float16, device="cuda")
    seeds = [nv.sampler_seed_for(1234, r) for r in range(rows)]

    logits_buf = torch.empty((rows, V), dtype=torch.bfloat16, device="cuda")

    def head(i):
        # the GEMV entry point: the row engine for 1-4 rows; for more rows it hands a matrix of this
        # size to the dense matrix-core product (weights read and dequantized once for all rows)
        p_, s_, b_ = heads[i % n_heads]
        if rows <= 4:
            return nv.affine_gemv(ctx, p_, s_, b_, bits, xs[i % 8], V, D)
        return nv.affine_gemv(ctx, p_, s_, b_, bits, xs[i % 8], V, D, y=logits_buf)[0]

    def step(i):
        logits = head(i)
        sm.encode(logits, probs, softcap=30.0)
        return tk.encode(probs, 0.6, 0.95, seeds, 20)

    for i in range(a.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(i)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / a.steps
    # the GEMV alone, by events
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    ev[0].record()
    for i in range(a.steps):
        head(i)
    ev[1].record()
    torch.cuda.synchronize()
    gemv_us = ev[0].elapsed_time(ev[1]) / a.steps * 1e3
    # the fused greedy head (RMSNorm + one logit per row + argmax) over the same matrices, by events
    chain = nv.LMHeadChain(ctx, bits)
    norm_w = torch.full((D,), 0x3F80, dtype=torch.int16, device="cuda")
    toks = torch.empty(rows, dtype=torch.int32, device="cuda")
    for i in range(a.warmup):
        chain.encode_greedy_decode(xs[i % 8], norm_w, *heads[i % n_heads], D, V, out=toks)
    ev[0].record()
    for i in range(a.steps):
        chain.encode_greedy_decode(xs[i % 8], norm_w, *heads[i % n_heads], D, V, out=toks)
    ev[1].record()
    torch.cuda.synchronize()
    greedy_us = ev[0].elapsed_time(ev[1]) / a.steps * 1e3
    ctx.profile_enable(True)
    for i in range(a.steps):
        step(i)
    torch.cuda.synchronize()
    ctx.profile_enable(False)
    kern = {"lm_head_gemv": gemv_us, "lm_head_greedy_fused": greedy_us}
    for tag, name in ((nv.PROF_SOFTMAX, "softmax"), (nv.PROF_SAMPLE, "sample_topk64")):
        ms, n = ctx.profile_read(tag)
        kern[name] = ms / max(n, 1) * 1e3
    cpu = None
    if not a.no_cpu:
        # the same stage on the CPU oracle, one row, one thread: LM head GEMV, softmax, sampler
        import oracle as O
        p_, s_, b_ = (t_.cpu().numpy() for t_ in heads[0])
        x0 = xs[0, 0].float().cpu().numpy()
        t0 = time.perf_counter()
        reps = 0
        while True:
            lg = O.affine_gemv(p_, s_.view(np.uint16), b_.view(np.uint16), x0, bits)
            pr = O.softmax_f16(O.round_bf16(lg), softcap=30.0, tiled=True)
            O.sample_topk64(pr, 0.6, 0.95, seeds[0], top_k=20)
            reps += 1
            if time.perf_counter() - t0 > 10.0 or reps >= 20:
                break
        dtc = (time.perf_counter() - t0) / reps
        cpu = dict(value=1.0 / dtc, unit="tok/s", cores=1, kind="port",
                   sample="oracle affine_gemv over the %d-bit LM head + softmax_f16 (tiled) + sample_topk64, "
                          "one row, %d reps, %.3f s each" % (bits, reps, dtc))
    head_bytes = V * D * bits / 8 + 2 * V * (D // 64) * 2
    step_bytes_ = head_bytes + rows * (D * 2 + V * 2 * 2 + V * 2)   # x, logits w+r, probs w (+ r by the sampler)
    gbps = head_bytes / (gemv_us * 1e-6) / 1e9
    return {
        "metric": METRIC, "value": round(rows / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(dt * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u%d codes, f32 accumulate; fp16 probabilities" % bits, "data": "synthetic",
        "config": {"workload": "end of configs[4]: %d-bit LM head GEMV over 248,320 x 2048, softcap + tiled softmax, "
                               "tiled top-k sampler (k 20, top-p 0.95, T 0.6), %d rows per step" % (bits, rows),
                   "step_gbps": round(step_bytes_ / dt / 1e9, 1),
                   "kernel_us": {k: round(v, 2) for k, v in kern.items()}},
        "roofline": {"kernel": "LM head: expert_rows GEMV (<= 4 rows) or prefill_gemm_kernel (more)", "bound": "hbm", "achieved": round(gbps, 2),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None,
                     "bytes_per_launch": head_bytes, "avg_launch_us": round(gemv_us, 2)},
        "cpu_baseline": cpu,
    }


def run_greedy(nv, ctx, torch, a):
    """LMHeadChain.encode_greedy_decode over a 4/8-bit head [248320, 2048]: one token per hidden row."""
    V, bits, rows = 248320, a.bits, min(a.batch, 4)
    gen = torch.Generator(device="cuda").manual_seed(78)
    n_heads = 4                                            # rotate copies of the head past the caches
    heads = []
    for _ in range(n_heads):
        wt = torch.empty((V, D), dtype=torch.bfloat16, device="cuda").normal_(0.0, 0.02, generator=gen)
        heads.append(nv.quantize_affine(ctx, wt, bits))
        del wt
    xs = torch.empty((8, rows, D), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
    norm_w = torch.empty(D, dtype=torch.bfloat16, device="cuda").uniform_(0.5, 1.5, generator=gen).view(torch.int16)
    chain = nv.LMHeadChain(ctx, bits)
    toks = torch.empty(rows, dtype=torch.int32, device="cuda")

    def step(i):
        chain.encode_greedy_decode(xs[i % 8], norm_w, *heads[i % n_heads], D, V, out=toks)

    for i in range(a.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        step(i)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / a.steps
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]     # the launch stream is torch's current stream
    ev[0].record()
    for i in range(a.steps):
        step(i)
    ev[1].record()
    torch.cuda.synchronize()
    us = ev[0].elapsed_time(ev[1]) / a.steps * 1e3
    cpu = None
    if not a.no_cpu:
        import oracle as O
        p_, s_, b_ = (t_.cpu().numpy() for t_ in heads[0])
        h0 = xs[0, 0].float().cpu().numpy()
        nw = norm_w.cpu().numpy().view(np.uint16)
        t0 = time.perf_counter()
        reps = 0
        while True:
            tok = O.lm_head_greedy(h0, nw, p_, s_.view(np.uint16), b_.view(np.uint16), bits, act=0)
            reps += 1
            if time.perf_counter() - t0 > 10.0 or reps >= 20:
                break
        dtc = (time.perf_counter() - t0) / reps
        step(0)
        torch.cuda.synchronize()
        assert int(toks[0]) == tok, "greedy token differs from the oracle"
        cpu = dict(value=1.0 / dtc, unit="tok/s", cores=1, kind="port",
                   sample="oracle lm_head_greedy over the %d-bit head, one row, %d reps, %.3f s each (same token as "
                          "the GPU)" % (bits, reps, dtc))
    head_bytes = V * D * bits / 8 + 2 * V * (D // 64) * 2
    gbps = rows * head_bytes / (us * 1e-6) / 1e9
    return {
        "metric": METRIC, "value": round(rows / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(dt * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u%d codes, f32 fma chain in a fixed order" % bits, "data": "synthetic",
        "config": {"workload": "end of configs[4], greedy: RMSNorm + %d-bit LM head 248,320 x 2048 + argmax in one "
                               "call, %d hidden rows per step (the head is read once per row)" % (bits, rows)},
        "roofline": {"kernel": "lm_head_greedy_kernel (+ its reduce launch)", "bound": "hbm", "achieved": round(gbps, 2),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4),
                     # rocprofv3 --pmc FETCH_SIZE: 264,100 KiB x 2.00 (copy-kernel calibration) at 8 bit, one row
                     "traffic": 264100 * 2.0 * 1024 if (bits == 8 and rows == 1) else None,
                     "bytes_per_launch": rows * head_bytes, "avg_launch_us": round(us, 2)},
        "cpu_baseline": cpu,
    }


def run_step(nv, ctx, torch, a):
    """configs[4]: the full synthetic decode step of the 40-layer hybrid model (30 gated-DeltaNet layers with
    a BF16 recurrent state, 10 full-attention layers over an 8-bit KV cache at `--context`, 4-bit experts and
    projections, BF16 LM head over 248,320, tiled top-k sampler), captured once into a HIP graph and replayed:
    tok/s for `--batch` sequences and the fraction of the bytes-per-token roofline."""
    from nvmai_amd.decoder import HybridConfig, HybridDecoder, HybridWeights
    B, context = min(a.batch, 16), a.context
    cfg = HybridConfig(layers=40, expert_bits=4, attn_bits=4, kv_bits=8, head_bits=16, gdn_state_bf16=True)
    w = HybridWeights(ctx, cfg, seed=2024)
    dec = HybridDecoder(ctx, cfg, w, batch=B, max_context=context)
    gen = torch.Generator(device="cuda").manual_seed(5)
    quant = nv.KVCacheQuantizer(ctx)
    for L, (kc, vc) in dec.kv.items():                      # a cache full of quantized N(0, 1) rows
        for c in (kc, vc):
            for b in range(B):
                for start in range(0, context, 8192):
                    n = min(8192, context - start)
                    src = torch.empty((n, cfg.kv_dim), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
                    quant.encode(src, cfg.kv_dim, c.view(b, start), n, cfg.kv_dim)
    dec.tokens.copy_(torch.randint(0, cfg.vocab, (B,), generator=gen, device="cuda", dtype=torch.int32))
    position = context - 1
    seeds = [nv.sampler_seed_for(1234, position + b) for b in range(B)]
    dec.step(position, seeds)                               # warm-up: sizes the workspace
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            dec.step(position, seeds)
    torch.cuda.synchronize()
    for _ in range(a.warmup):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        graph.replay()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / a.steps
    # the same step launched eagerly (every call through the C ABI from Python), for comparison
    t0 = time.perf_counter()
    for _ in range(5):
        dec.step(position, seeds)
    torch.cuda.synchronize()
    dt_eager = (time.perf_counter() - t0) / 5
    bpt = cfg.bytes_per_token(B, context)
    gbps = bpt * B / dt / 1e9
    assert bool(((dec.next_tokens >= 0) & (dec.next_tokens < cfg.vocab)).all()) and bool(torch.isfinite(dec.logits.float()).all())
    return {
        "metric": METRIC, "value": round(B / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u4 codes, f32 accumulate; bf16 activations, recurrent state and LM head; u8 KV", "data": "synthetic",
        "config": {"workload": "configs[4]: full decode step of the 40-layer hybrid MoE model (30 gated-DeltaNet + 10 "
                               "full-attention layers, 256 experts top-8 + shared, 4-bit), 8-bit KV at context %d, bf16 LM "
                               "head over 248,320, tiled top-k sampler; batch %d, one HIP graph per step" % (context, B),
                   "batch": B, "context": context, "bytes_per_token_MB": round(bpt / 1e6, 1),
                   "roofline_tok_per_s_at_8TBps": round(HBM_PEAK_GBPS * 1e9 / bpt, 1),
                   "eager_ms_per_step": round(dt_eager * 1e3, 3)},
        "roofline": {"kernel": "whole step (all kernels of one graph replay)", "bound": "hbm", "achieved": round(gbps, 2),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None,
                     "traffic_source": None, "bytes_per_launch": round(bpt * B), "avg_launch_us": round(dt * 1e6, 2)},
        "cpu_baseline": None,
    }


def run_prefill_step(nv, ctx, torch, a):
    """The prompt side of configs[4]: `--tokens` tokens of one sequence through all 40 layers of the same
    hybrid model with the prefill kernels (HybridDecoder.prefill_chunked, chunks of `--chunk` tokens): dense
    matrix-core projections, gated-DeltaNet over the rows of a chunk, causal attention over the 8-bit
    cache, tiled router + permutation + grouped GEMM + reduce, shared expert.  Prompt tokens per second;
    the flops counted are the matrix products of the model (2 flop per weight and token)."""
    from nvmai_amd.decoder import HybridConfig, HybridDecoder, HybridWeights
    cfg = HybridConfig(layers=40, expert_bits=4, attn_bits=4, kv_bits=8, head_bits=16, gdn_state_bf16=True)
    w = HybridWeights(ctx, cfg, seed=2024)
    T, chunk = a.tokens, a.chunk
    dec = HybridDecoder(ctx, cfg, w, batch=1, max_context=T)
    gen = torch.Generator(device="cuda").manual_seed(9)
    tokens = torch.randint(0, cfg.vocab, (T,), generator=gen, device="cuda", dtype=torch.int32)

    def once():
        for L in dec.gdn_states:
            for buf in dec.gdn_states[L]:
                buf.zero_()
        return dec.prefill_chunked(tokens, 0, 0, chunk)
    ctx.profile_enable(False)
    for _ in range(max(1, a.warmup)):
        last = once()
    torch.cuda.synchronize()
    assert bool(torch.isfinite(last.float()).all())
    steps = max(1, a.steps)
    t0 = time.perf_counter()
    for _ in range(steps):
        once()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    D, F, K = cfg.hidden, cfg.moe_intermediate, cfg.top_k
    kh, vh, dk, dv, taps = cfg.gdn
    n_lin = sum(cfg.is_linear(L) for L in range(cfg.layers))
    n_full = cfg.layers - n_lin
    lin_w = (cfg.gdn_qkv_dim + cfg.gdn_value_dim + 2 * vh) * D + D * cfg.gdn_value_dim
    full_w = (2 * cfg.q_dim + 2 * cfg.kv_dim) * D + D * cfg.q_dim
    moe_w = (K + 1) * 3 * D * F + cfg.num_experts * D
    attn_flops = n_full * 4.0 * cfg.num_heads * cfg.head_dim * (T * (T + 1) / 2)
    flops = 2.0 * T * (n_lin * lin_w + n_full * full_w + cfg.layers * moe_w) + attn_flops
    tf = flops / dt / 1e12
    return {
        "metric": METRIC, "value": round(T / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": a.warmup,
        "ms_per_step": round(dt * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u4 codes dequantized to bf16 MFMA operands, f32 accumulate; bf16 recurrent state; u8 KV", "data": "synthetic",
        "config": {"workload": "prompt side of configs[4]: %d tokens of one sequence through the 40-layer hybrid MoE model "
                               "in chunks of %d (prefill kernels; launched eagerly through the C ABI)" % (T, chunk),
                   "tokens": T, "chunk": chunk, "model_gflop_per_token": round(flops / T / 1e9, 2)},
        "roofline": {"kernel": "whole prompt (all kernels)", "bound": "mfma", "achieved": round(tf, 2), "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None, "traffic_source": None,
                     "flops_per_launch": flops, "avg_launch_us": round(dt * 1e6, 1)},
        "cpu_baseline": None,
    }


def run_copy(torch, a):
    """A plain copy kernel of known size: 1 GiB read + 1 GiB written per launch."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 256)
    dst = torch.empty_like(src)
    for _ in range(a.warmup):
        dst.copy_(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        dst.copy_(src)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / a.steps
    return {"metric": "plain device copy", "value": round(2 * n / dt / 1e9, 2), "unit": "GB/s", "n_gpus": 1,
            "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": "copy: 1 GiB read + 1 GiB written per launch", "bytes_read": n, "bytes_written": n}}


def run_read(nv, ctx, torch, a, window_mib=512):
    """What a kernel that only reads reaches on this device: windows of 512 MiB out of 8 GiB in turn (twice the
    memory-side cache apart, so every launch comes from HBM), one launch per step, HIP events around the timed steps."""
    window = window_mib << 20
    pool = torch.empty(8 << 30, dtype=torch.uint8, device="cuda")
    pool.view(torch.int32).random_(0, 1 << 31)
    n_win = pool.numel() // window
    views = [pool[i * window:(i + 1) * window] for i in range(n_win)]
    for i in range(max(a.warmup, 4)):
        ctx.read_probe(views[i % n_win])
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    steps = max(a.steps, 16)
    e0.record()
    for i in range(steps):
        ctx.read_probe(views[i % n_win])
    e1.record()
    torch.cuda.synchronize()
    dt = e0.elapsed_time(e1) * 1e-3 / steps
    gbps = window / dt / 1e9
    return {"metric": "plain device read", "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps,
            "warmup": max(a.warmup, 4), "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": "read: %d MiB per launch, nothing else (nvmai_hip_read_probe)" % window_mib,
                       "bytes_read": window, "frac_of_hbm_peak": round(gbps / 8000.0, 4)}}


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import torch
    import nvmai_amd as nv
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    ctx = nv.Context(0, nv.ACT_BF16)
    if a.workload != "decode":
        line = (run_prefill(nv, ctx, torch, a) if a.workload == "prefill" else
                run_attention(nv, ctx, torch, a) if a.workload == "attention" else
                run_prefill_attention(nv, ctx, torch, a) if a.workload == "prefill_attention" else
                run_sampler(nv, ctx, torch, a) if a.workload == "sampler" else
                run_greedy(nv, ctx, torch, a) if a.workload == "greedy" else
                run_step(nv, ctx, torch, a) if a.workload == "step" else
                run_prefill_step(nv, ctx, torch, a) if a.workload == "prefill_step" else
                run_read(nv, ctx, torch, a) if a.workload == "read" else run_copy(torch, a))
        print(json.dumps(line), flush=True)
        return
    layers, stride = build_layers(nv, ctx, torch, a.bits, a.layers)
    torch.cuda.synchronize()
    r = run_config(nv, ctx, torch, layers, stride, a.bits, a.batch, a.steps, a.warmup, profile=True)
    line = decode_line(a, r, a.bits, a.batch, a.steps, a.warmup)
    if a.sweep:
        for bits in (8, 4):
            ls, st = (layers, stride) if bits == a.bits else build_layers(nv, ctx, torch, bits, a.layers)
            for b in (1, 2, 4, 8, 16, 32):
                s = run_config(nv, ctx, torch, ls, st, bits, b, a.steps, a.warmup, profile=True)
                print("sweep bits=%d batch=%d: %.1f GB/s (%.1f%% of HBM peak) %.2f us/step distinct=%.1f "
                      "phase1 %.1f GB/s kernels(us)=%s"
                      % (bits, b, s["gbps"], 100 * s["gbps"] / HBM_PEAK_GBPS, s["ms_per_step"] * 1e3,
                         s["mean_distinct"], s["phase1_gbps"],
                         {k: round(v, 1) for k, v in s["kernel_us"].items()}), file=sys.stderr, flush=True)
            if bits != a.bits:
                del ls
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(layers, stride, a.bits, a.batch, torch)
    else:
        line["cpu_baseline"] = None
    if not a.no_extra and a.bits == 8 and a.batch == 32:
        line["extra"] = extra_cells(nv, ctx, torch, a, layers, stride)
    print(json.dumps(line), flush=True)


def compact(line, **more):
    """One cell of the `extra` object: value, unit, ms per step, and the roofline kernel's launch time, rate and
    fraction of its peak (GB/s against 8 TB/s, or TFLOP/s against 2.5 PFLOP/s); the key names the cell."""
    r = line["roofline"]
    out = {"v": line["value"], "u": line["unit"], "ms": line["ms_per_step"], "kern_us": r["avg_launch_us"],
           "kern": r["achieved"], "frac": r["frac"]}
    for k in ("mean_distinct_experts", "frac_of_hbm_peak"):
        if k in line["config"]:
            out[k] = line["config"][k]
    out.update(more)
    return out


def decode_line(a, r, bits, batch, steps, warmup):
    return {
        "metric": METRIC, "value": round(r["gbps"], 2), "unit": "GB/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": round(r["ms_per_step"], 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u%d codes, f32 accumulate" % bits, "data": "synthetic",
        "config": {"workload": "configs[1]: MoE-layer decode step, %d-bit g64 experts, 256 top-8 + gated shared, D 2048, F 512, "
                               "all in HBM" % bits,
                   "batch_tokens": batch, "layers_rotated": a.layers, "untimed_clock_ramp_steps": RAMP_STEPS,
                   "mean_distinct_experts": round(r["mean_distinct"], 2),
                   "frac_of_hbm_peak": round(r["gbps"] / HBM_PEAK_GBPS, 4),
                   "kernel_us": {k: round(v, 2) for k, v in r["kernel_us"].items()}},
        "roofline": {"kernel": "expert_rows_fast (routed + shared gate/up SwiGLU, phase 1)" if batch > 4 else
                               "expert_rows_routed / expert_rows_fast (gate/up SwiGLU, phase 1)", "bound": "hbm",
                     "achieved": round(r["phase1_gbps"], 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(r["phase1_gbps"] / HBM_PEAK_GBPS, 4),
                     "traffic": recorded_traffic(("decode", bits, batch))[0],
                     "traffic_source": recorded_traffic(("decode", bits, batch))[1],
                     "bytes_per_launch": round(r["phase1_bytes"]),
                     "avg_launch_us": round(r["kernel_us"]["phase1"], 2)},
    }


def run_config0(nv, ctx, torch, layers4, stride4, a):
    """BASELINE configs[0]: ONE 4-bit expert (SwiGLU MLP, 512 x 2048 gate and up, 2048 x 512 down), one token,
    through the shared-expert operator without a gate (the single-expert FFN of CPUExpertFFN.accumulate).  Every
    call takes another expert of the 40 x 257 resident ones, so the 1.78 MB come from HBM.  At 8 TB/s the bytes
    of one call are 0.22 us of traffic, less than a launch: the figure is a latency, stated as such."""
    import oracle as O
    off, _ = nv.expert_offsets(D, F, 4)
    run = nv.SharedExpertRuntime(ctx, 4)
    gen = torch.Generator(device="cuda").manual_seed(404)
    xs = torch.empty((64, 1, D), dtype=torch.bfloat16, device="cuda").normal_(0.0, 1.0, generator=gen)
    y = torch.empty((1, D), dtype=torch.bfloat16, device="cuda")
    blob_of = lambda i: layers4[i % len(layers4)]["pool"][(i * 37) % (E + 1)]
    call = lambda i: run.encode(blob_of(i), off, xs[i % 64], D, F, shared_gate=None, y=y)
    steps, warm = 400, 20
    for i in range(warm):
        call(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        call(warm + i)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    ev[0].record()
    for i in range(steps):
        call(i)
    ev[1].record()
    torch.cuda.synchronize()
    ev_us = ev[0].elapsed_time(ev[1]) / steps * 1e3
    lat = []
    for i in range(20):                                     # one call alone: submit to completion, host clock
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        call(1000 + i)
        torch.cuda.synchronize()
        lat.append(time.perf_counter() - t0)
    i = 1019
    want = np.zeros(D, np.float32)
    O.expert_ffn_accumulate(blob_of(i).cpu().numpy(), 4, xs[i % 64, 0].float().cpu().numpy(), D, F, 1.0, want)
    rel = float(O.rel_error(y[0].float().cpu().numpy(), want))
    assert rel < 1e-2, "configs[0] expert differs from the oracle: max-rel %g" % rel
    nbytes = stride4 + 2 * D * 2
    out = {"v": round(nbytes / dt / 1e9, 1), "u": "GB/s", "ms": round(dt * 1e3, 5), "kern_us": round(ev_us, 2),
           "frac": round(nbytes / dt / 1e9 / HBM_PEAK_GBPS, 4), "bytes_per_call": nbytes,
           "single_call_latency_us": round(float(np.median(lat)) * 1e6, 1), "launches_per_call": 2, "max_rel": round(rel, 6)}
    if not a.no_cpu:
        blobs = layers4[0]["pool"][:64].cpu().numpy()
        x0 = xs[0, 0].float().cpu().numpy()
        t_ref, _ = O.time_expert_ffn(blobs, D, F, x0, reps=41, reference=True)
        t_port, _ = O.time_expert_ffn(blobs, D, F, x0, reps=41, reference=False)
        row = lambda t, kind, what: {"value": round(nbytes / t / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": kind,
                                     "ms_per_expert": round(t * 1e3, 4), "sample": what}
        out["cpu_baseline"] = [
            row(t_ref, "reference", "the reference's nvmai_int4_affine_gemv (oracle/_ref, gcc -O2) x3 + silu in numpy, "
                                    "41 experts, median") if t_ref else None,
            row(t_port, "port", "oracle orc_expert_ffn_accumulate (gcc -O3 -march=native), 41 experts, median")]
    return out


def extra_cells(nv, ctx, torch, a, layers8, stride8):
    """The other cells of the metric, each measured like its own --workload line but shorter and printed in
    compact form (the key names the cell; v = value, u = unit, ms = per step, kern_us / kern / frac = the
    roofline kernel's launch time, rate and fraction of its peak).  First what a kernel that only reads reaches on
    this device in this run, the measuring stick for the HBM fractions; then the twelve cells of configs[3] as
    one table, the metric's own cells last: configs[0], the configs[2] prefill grouped GEMM, 4-bit decode at batch
    32, 8-bit decode at one token, configs[4] at batch 1 and 16."""
    import argparse
    out = {}
    sub = argparse.Namespace(**vars(a))
    sub.steps, sub.warmup = 32, 8
    c = run_read(nv, ctx, torch, sub)
    out["plain_read_512MiB"] = {"v": c["value"], "u": "GB/s", "frac": c["config"]["frac_of_hbm_peak"]}
    torch.cuda.empty_cache()
    rows = []
    for bits in (8, 4):
        for context, batch in ((131072, 8), (131072, 1), (32768, 8), (32768, 1), (4096, 8), (4096, 1)):
            sub = argparse.Namespace(**vars(a))
            sub.no_cpu, sub.steps, sub.warmup, sub.bits, sub.context, sub.batch = True, 30, 5, bits, context, batch
            c = run_attention(nv, ctx, torch, sub)
            r = c["roofline"]
            rows.append([bits, context // 1024, batch, c["value"], c["config"]["frac_of_hbm_peak"], r["avg_launch_us"],
                         r["frac"], c["parity_check"]["max_rel"]])
            torch.cuda.empty_cache()
    out["attention_configs3"] = {"cols": ["kv_bits", "ctx_k", "batch", "GB/s", "frac", "kern_us", "kern_frac", "max_rel_vs_oracle"],
                                 "rows": rows}
    for bits in (8, 4):
        sub = argparse.Namespace(**vars(a))
        sub.no_cpu, sub.steps, sub.warmup, sub.bits, sub.tokens, sub.context_given = True, 20, 3, bits, 4096, False
        c = run_prefill_attention(nv, ctx, torch, sub)
        out["prefill_attention_%dbit_4096tokens" % bits] = compact(c, max_rel=c["parity_check"]["max_rel"])
        torch.cuda.empty_cache()
    sub = argparse.Namespace(**vars(a))
    sub.no_cpu, sub.steps, sub.warmup, sub.tokens, sub.chunk = True, 2, 1, 4096, 4096
    cell = run_prefill_step(nv, ctx, torch, sub)
    out["prefill_step_configs4_4096tokens"] = compact(cell, model_gflop_per_token=cell["config"]["model_gflop_per_token"])
    torch.cuda.empty_cache()
    layers4, stride4 = build_layers(nv, ctx, torch, 4, a.layers)
    torch.cuda.synchronize()
    out["configs0_4bit_one_expert_one_token"] = run_config0(nv, ctx, torch, layers4, stride4, a)
    sub = argparse.Namespace(**vars(a))
    sub.no_cpu, sub.steps, sub.warmup, sub.bits, sub.tokens = True, 30, 5, 4, 4096
    c = run_prefill(nv, ctx, torch, sub)
    out["prefill_4bit_4096tokens"] = compact(c, kernel_us=c["config"]["kernel_us"], tokens_per_s=c["config"]["tokens_per_s"])
    torch.cuda.empty_cache()
    r = run_config(nv, ctx, torch, layers4, stride4, 4, 32, 200, 20, profile=True)
    c = decode_line(a, r, 4, 32, 200, 20)
    out["decode_4bit_batch32"] = compact(c, kernel_us=c["config"]["kernel_us"])
    del layers4
    torch.cuda.empty_cache()
    r = run_config(nv, ctx, torch, layers8, stride8, 8, 1, 200, 20, profile=True)
    c = decode_line(a, r, 8, 1, 200, 20)
    out["decode_8bit_batch1"] = compact(c, kernel_us=c["config"]["kernel_us"])
    for batch in (1, 16):
        sub = argparse.Namespace(**vars(a))
        sub.no_cpu, sub.steps, sub.warmup, sub.batch, sub.context = True, 30, 3, batch, 32768
        cell = run_step(nv, ctx, torch, sub)
        out["decode_step_configs4_batch%d" % batch] = compact(
            cell, bytes_per_token_MB=cell["config"]["bytes_per_token_MB"],
            roofline_tok_per_s_at_8TBps=cell["config"]["roofline_tok_per_s_at_8TBps"])
        torch.cuda.empty_cache()
    return out


if __name__ == "__main__":
    main()
