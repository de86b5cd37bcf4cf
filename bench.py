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


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--batch", type=int, default=32, help="tokens per decode step (1..32)")
    ap.add_argument("--bits", type=int, default=8, choices=[4, 8])
    ap.add_argument("--layers", type=int, default=40)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--sweep", action="store_true", help="also print batch/bits sweep lines to stderr")
    return ap.parse_args()


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
    for i in range(warmup):
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
    """The CPU oracle (a scalar C port of the reference's CPU path) on a bounded sample: the
    first tokens of one step of layer 0, one thread."""
    import oracle as O
    L = layers[0]
    pool = L["pool"].cpu().numpy()
    router = L["router"].view(torch.int16).cpu().numpy().view(np.uint16)
    gq = [t.cpu().numpy() for t in L["gate"]]
    gate = (8, gq[0], gq[1].view(np.uint16), gq[2].view(np.uint16))
    rng = np.random.default_rng(7)
    n = min(batch, 8)
    x = O.round_bf16(rng.standard_normal((n, D)).astype(np.float32))
    t0 = time.perf_counter()
    reps = 0
    while True:
        idx, _, _ = O.moe_layer_forward(x, D, F, K, bits, (16, router, None, None), pool[:E], pool[E], gate)
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 20:
            break
    dt = (time.perf_counter() - t0) / reps
    # the scalar port evaluates every (token, slot) pair separately: its bytes are per pair
    bytes_ = n * (K + 1) * stride + n * (E * D * 2) + n * D * 8
    algo = step_bytes(len(np.unique(idx)), n, stride)
    return dict(value=algo / dt / 1e9, unit="GB/s", cores=1, kind="port",
                sample="oracle moe_layer_forward, %d tokens of one %d-bit layer, %d reps, %.2f s each; "
                       "%.1f MB algorithmic (%.1f MB touched by the scalar path)"
                       % (n, bits, reps, dt, algo / 1e6, bytes_ / 1e6))


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
    layers, stride = build_layers(nv, ctx, torch, a.bits, a.layers)
    torch.cuda.synchronize()
    r = run_config(nv, ctx, torch, layers, stride, a.bits, a.batch, a.steps, a.warmup, profile=True)
    line = {
        "metric": METRIC, "value": round(r["gbps"], 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(r["ms_per_step"], 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u%d codes, f32 accumulate" % a.bits,
        "data": "synthetic",
        "config": {"workload": "configs[1]: one MoE-layer decode step, %d-bit group-64 experts, hidden 2048, "
                               "256 experts top-8 + gated shared expert, intermediate 512, bf16 activations, "
                               "all experts resident in HBM" % a.bits,
                   "batch_tokens": a.batch, "layers_rotated": a.layers,
                   "mean_distinct_experts": round(r["mean_distinct"], 2),
                   "frac_of_hbm_peak": round(r["gbps"] / HBM_PEAK_GBPS, 4),
                   "kernel_us": {k: round(v, 2) for k, v in r["kernel_us"].items()}},
        "roofline": {"kernel": "expert_rows_fast (routed + shared gate/up SwiGLU, phase 1)", "bound": "hbm",
                     "achieved": round(r["phase1_gbps"], 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(r["phase1_gbps"] / HBM_PEAK_GBPS, 4), "traffic": None,
                     "bytes_per_launch": round(r["phase1_bytes"]),
                     "avg_launch_us": round(r["kernel_us"]["phase1"], 2)},
    }
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
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
