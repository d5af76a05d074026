#!/usr/bin/env python3
"""Headline benchmark: RWKV-7 7.2B-shape W8A16 greedy decode at batch 1 on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--preset 7.2B] [--fmt w8] [--batch 1]

One "step" is one decode step of the whole model: embedding row -> 32 layers -> lm_head -> argmax, with the
argmax fed back on the device (no host round trip).  Weights are random-init N(0, 0.02) generated and
quantised on the GPU; inputs are resident in HBM before the timed region.  Prints ONE JSON line with the
whole-job tokens/s plus
  roofline     -- the weight-streaming GEMV kernel against the 8 TB/s HBM peak: algorithmic bytes per
                  launch / average launch duration from HIP events on the session stream
  cpu_baseline -- the scalar C++ oracle timed on the host cores on a bounded slice of the same workload.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--preset", default="7.2B")
    ap.add_argument("--fmt", default="w8", choices=["f16", "w8", "w4"])
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--prefill", type=int, default=64, help="tokens prefilled (chunk 128) before the decode loop")
    ap.add_argument("--no-graph", action="store_true", help="launch decode steps eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    return ap.parse_args()


def gemv_bytes_per_step(dims, fmt):
    """Algorithmic bytes the weight-streaming linear launches move per decode step: every code of the seven
    big matrices once + their scales (+ zero points), the fp16 LoRA rank-in matrices that share the r/k/v launch,
    + x in and y out (fp16).  Returns (bytes, launches)."""
    C, F, V, L = dims.C, dims.F, dims.V, dims.L

    def mat(N, K):
        if fmt == "w8":
            w = N * K + 2 * N
        elif fmt == "w4":
            w = N * K // 2 + 3 * N * (K // 128)
        else:
            w = 2 * N * K
        return w + 2 * K + 2 * N

    def lora_in(l):
        ranks = dims.Rw + dims.Ra + dims.Rg + (dims.Rv if l > 0 else 0)
        return 2 * C * ranks + 2 * ranks + (3 if l > 0 else 3) * 2 * C  # fp16 [R,C] rows, hidden out, x_w/x_a/x_g in

    total = mat(V, C)
    for l in range(L):
        # launch 1: r/k/v + the LoRA rank-ins (one launch); 2: output; 3: ffn.key; 4: ffn.value
        total += 3 * mat(C, C) + lora_in(l) + mat(C, C) + mat(F, C) + mat(C, F)
    launches = 4 * L + 1
    return total, launches


def cpu_baseline(dims, fmt_name):
    """Times the CPU oracle on one decode step of 1- and 2-layer slices of the same shape (full width, full
    vocabulary) and extrapolates linearly in the layer count to the full depth."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle
    from rwkv_lightning_cuda_amd.model import ModelDims, synth_weights
    threads = min(os.cpu_count() or 1, 16)
    oracle.set_threads(threads)
    fmt = {"f16": 0, "w8": 1, "w4": 2}[fmt_name]
    times = {}
    d2 = ModelDims(L=2, C=dims.C, H=dims.H, F=dims.F, V=dims.V, Rw=dims.Rw, Ra=dims.Ra, Rg=dims.Rg, Rv=dims.Rv)
    weights = synth_weights(d2, seed=7)
    for layers in (1, 2):
        d = ModelDims(L=layers, C=dims.C, H=dims.H, F=dims.F, V=dims.V, Rw=dims.Rw, Ra=dims.Ra, Rg=dims.Rg, Rv=dims.Rv)
        om = oracle.Model(d, dict(weights, layers=weights["layers"][:layers]), fmt)
        st = om.new_state(1)
        tok = np.array([[17]], np.int64)
        om.forward(tok, st)  # touch everything once
        reps = 3
        t0 = time.perf_counter()
        for _ in range(reps):
            om.forward(tok, st)
        times[layers] = (time.perf_counter() - t0) / reps
        del om
    per_layer = max(times[2] - times[1], 1e-9)
    fixed = max(times[1] - per_layer, 0.0)
    step_s = fixed + per_layer * dims.L
    return {
        "value": 1.0 / step_s,
        "unit": "tok/s",
        "cores": threads,
        "kind": "port",
        "sample": "one batch-1 decode step of 1- and 2-layer slices at full width/vocab (%s), "
                  "extrapolated linearly to %d layers: %.3f s/layer + %.3f s fixed" % (fmt_name, dims.L, per_layer, fixed),
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (got --gpus %d); nothing was run" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from rwkv_lightning_cuda_amd import hip
    from rwkv_lightning_cuda_amd.model import PRESETS, HipModel, Session, State

    hip.load()
    if hip.device_count() < 1:
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dims = PRESETS[args.preset]
    fmt = {"f16": hip.FMT_F16, "w8": hip.FMT_W8, "w4": hip.FMT_W4}[args.fmt]
    B = args.batch

    model = HipModel.random_on_device(dims, fmt, seed=1)
    sess = Session(model)
    if args.no_graph:
        sess.set_graph(False)
    state = State(dims, B)
    logits = hip.DeviceArray((B, dims.V), np.float32)
    rng = np.random.default_rng(0)
    if args.prefill > 0:
        for t0 in range(0, args.prefill, 128):
            tn = min(128, args.prefill - t0)
            sess.forward(rng.integers(0, dims.V, (B, tn)), state, logits)
    first = rng.integers(0, dims.V, (B,))

    if args.warmup > 0:
        sess.decode_greedy(first, args.warmup, state, logits)
    hip.device_sync()
    t0 = time.perf_counter()
    toks = sess.decode_greedy(first, args.steps, state, logits)
    hip.device_sync()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    value = args.steps * B / elapsed

    weight_bytes = model.weight_bytes()
    state_bytes = B * (2 * dims.L * dims.H * 64 * 64 * 4 + 2 * dims.L * 2 * dims.C * 2)
    out = {
        "metric": "decode tok/s @%s W%sA16 bs%d" % (args.preset, {"f16": "16", "w8": "8", "w4": "4"}[args.fmt], B),
        "value": value,
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 activations, fp32 accumulate, %s weights" % args.fmt,
        "data": "synthetic (random-init N(0,0.02) weights quantised on load, random token ids)",
        "config": {"workload": "RWKV-7 %s-shape greedy decode, batch %d, %d-token prefill, lm_head+argmax on device"
                               % (args.preset, B, args.prefill),
                   "L": dims.L, "C": dims.C, "H": dims.H, "F": dims.F, "V": dims.V,
                   "weight_format": args.fmt, "hip_graph": not args.no_graph, "weight_bytes_per_step": weight_bytes,
                   "state_bytes_per_step": state_bytes,
                   "step_hbm_fraction": (weight_bytes + state_bytes) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                   "distinct_tokens": int(len(np.unique(toks)))},
    }

    if not args.no_roofline:
        # the same steps again, eagerly, with every weight-streaming linear launch bracketed by HIP events
        sess.set_profile(True)
        sess.read_profile()
        tok = toks[-1].reshape(B, 1).astype(np.int64)
        n_prof = min(args.steps, 32)
        for _ in range(n_prof):
            sess.forward(tok, state, logits, sync=False)
        launches, total_ms = sess.read_profile()
        sess.set_profile(False)
        gemv_bytes, per_step = gemv_bytes_per_step(dims, args.fmt)
        assert launches == per_step * n_prof, (launches, per_step, n_prof)
        bytes_per_launch = gemv_bytes / per_step
        avg_ms = total_ms / launches
        achieved = bytes_per_launch / (avg_ms * 1e-3) / 1e9
        out["roofline"] = {
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS, "traffic": None,
            "kernel": "linear_gemv_kernel (W8A16 weight-streaming GEMV; r/k/v fused, output, ffn.key, ffn.value, lm_head)",
            "bytes_per_launch": bytes_per_launch, "avg_launch_us": avg_ms * 1e3, "launches_per_step": per_step,
        }

    sess.close()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(dims, args.fmt)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
