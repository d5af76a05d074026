#!/usr/bin/env python3
"""Headline benchmark: RWKV-7 7.2B-shape W8A16 greedy decode at batch 1 on one MI355X, after a 4096-token
prefill in chunks of 128.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--preset 7.2B] [--fmt w8] [--batch 1] [--prefill 4096]

One "step" is one decode step of the whole model: embedding row -> 32 layers -> lm_head -> argmax, with the
argmax fed back on the device (no host round trip).  Weights are random-init N(0, 0.02) generated and
quantised on the GPU; inputs are resident in HBM before the timed region.  Prints ONE JSON line with the
whole-job tokens/s plus
  roofline     -- the weight-streaming GEMV kernel against the 8 TB/s HBM peak: algorithmic bytes per
                  launch / average launch duration from HIP events on the session stream
  cpu_baseline -- the scalar C++ oracle timed on the host cores on a bounded slice of the same workload
  also         -- the other figures the metric names, measured in the same run: prefill tokens/s of the
                  4096-token prompt (and the MFMA fraction of its GEMM launches), batch-8, -16 and -64 decode tokens/s,
                  batch-1 decode with int4 weights,
                  and the WKV7 op alone on a long sequence.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published peak
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 matrix peak, published
# HBM bytes per launch of the GEMV kernel from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE (two runs), each scaled
# by what the same counter reads for a 1 GiB device-to-device copy (FETCH_SIZE reads half the bytes copied,
# WRITE_SIZE all of them).  Keyed by (preset, format, batch); each record names the summary under profiles/ it was
# taken from and the SHA-256 of the kernel source it was measured on: when csrc/linear.hip no longer matches, the
# figure is stale and `traffic` is reported as null until the counters are collected again.
MEASURED_TRAFFIC = {
    ("7.2B", "w8", 1): {
        "bytes_per_launch": 49977226,
        "profile": "profiles/linear_gemv_row1_decode_7p2b_w8_bs1_pmc_traffic.md",
        "kernel_source": "rwkv_lightning_cuda_amd/csrc/linear.hip",
        "kernel_source_sha256": "80f6b9afc28f817c5b9ae5e25654c011378935dd2cceed2a2299f90b05f38d9e",
    },
}


def measured_traffic(key):
    """(bytes per launch or None, record) - None when there is no record or the kernel source has changed since."""
    import hashlib
    rec = MEASURED_TRAFFIC.get(key)
    if rec is None or rec["bytes_per_launch"] is None:
        return None, rec
    with open(os.path.join(ROOT, rec["kernel_source"]), "rb") as f:
        sha = hashlib.sha256(f.read()).hexdigest()
    if sha != rec["kernel_source_sha256"]:
        return None, dict(rec, stale=True)
    return rec["bytes_per_launch"], rec


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--preset", default="7.2B")
    ap.add_argument("--fmt", default="w8", choices=["f16", "w8", "w4"])
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--prefill", type=int, default=4096, help="tokens prefilled (chunk 128) before the decode loop")
    ap.add_argument("--no-also", action="store_true", help="skip the secondary measurements (prefill MFMA fraction, "
                    "batch-8/16/64 decode, W4 decode, WKV7 op)")
    ap.add_argument("--no-graph", action="store_true", help="launch decode steps eagerly instead of replaying a HIP graph")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="BYTES",
                    help="only run a device-to-device copy of BYTES (twice) and exit: the known-size kernel that "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings are scaled by")
    ap.add_argument("--wkv7-op-only", action="store_true", help="only run the WKV7 op at the long-context configuration "
                    "(B 16, T 16384, 64 heads; two calls) and exit: the target of rocprofv3 counter runs")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--fused-ln", type=int, default=-1, help="tuning hook: 1 / 0 force LayerNorm inside / outside the linear "
                    "launches of decode steps (default: by row count)")
    ap.add_argument("--no-parity", action="store_true", help="skip the oracle comparison of the measured configurations "
                    "(the `parity` objects; about a minute of CPU work outside the timed regions)")
    ap.add_argument("--wkv-fp16", action="store_true", help="keep the WKV state in fp16 (the reference server's default, "
                    "use_wkv32 == false) in the main measurement; the headline figure is the fp32 state")
    return ap.parse_args()


def gemv_bytes_per_step(dims, fmt, sparse_value):
    """Algorithmic bytes the weight-streaming GEMV launches move per decode step: every code of the big
    matrices once + their scales (+ zero points), the fp16 LoRA rank-in matrices that share the r/k/v launch,
    + x in and y out (fp16).  With `sparse_value` the ffn.value product is not a GEMV launch (a one-sequence
    step reads only the rows with a non-zero activation through another kernel) and is left out.
    Returns (bytes, launches)."""
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
        total += 3 * mat(C, C) + lora_in(l) + mat(C, C) + mat(F, C) + (0 if sparse_value else mat(C, F))
    launches = (3 if sparse_value else 4) * L + 1
    return total, launches


def cpu_baseline(dims, fmt_name):
    """Times the CPU oracle on one decode step of 1- and 2-layer slices of the same shape (full width, full
    vocabulary) and extrapolates linearly in the layer count to the full depth: with all host threads (the headline
    `value`) and with one thread."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle
    from rwkv_lightning_cuda_amd.model import ModelDims, synth_weights
    threads = min(os.cpu_count() or 1, 16)
    fmt = {"f16": 0, "w8": 1, "w4": 2}[fmt_name]
    d2 = ModelDims(L=2, C=dims.C, H=dims.H, F=dims.F, V=dims.V, Rw=dims.Rw, Ra=dims.Ra, Rg=dims.Rg, Rv=dims.Rv)
    weights = synth_weights(d2, seed=7)
    models = {}
    for layers in (1, 2):
        d = ModelDims(L=layers, C=dims.C, H=dims.H, F=dims.F, V=dims.V, Rw=dims.Rw, Ra=dims.Ra, Rg=dims.Rg, Rv=dims.Rv)
        models[layers] = oracle.Model(d, dict(weights, layers=weights["layers"][:layers]), fmt)
    tok = np.array([[17]], np.int64)

    def step_seconds(n_threads, reps):
        oracle.set_threads(n_threads)
        times = {}
        for layers, om in models.items():
            st = om.new_state(1)
            om.forward(tok, st)  # touch everything once
            t0 = time.perf_counter()
            for _ in range(reps):
                om.forward(tok, st)
            times[layers] = (time.perf_counter() - t0) / reps
        per_layer = max(times[2] - times[1], 1e-9)
        fixed = max(times[1] - per_layer, 0.0)
        return fixed + per_layer * dims.L, per_layer, fixed

    step_n, per_layer_n, fixed_n = step_seconds(threads, 3)
    step_1, per_layer_1, fixed_1 = step_seconds(1, 1)
    oracle.set_threads(1)
    return {
        "value": 1.0 / step_n,
        "unit": "tok/s",
        "cores": threads,
        "kind": "port",
        "sample": "one batch-1 decode step of 1- and 2-layer slices at full width/vocab (%s), "
                  "extrapolated linearly to %d layers: %.3f s/layer + %.3f s fixed with %d threads; "
                  "%.3f s/layer + %.3f s fixed with 1 thread" % (fmt_name, dims.L, per_layer_n, fixed_n, threads,
                                                                per_layer_1, fixed_1),
        "value_1_thread": 1.0 / step_1,
    }


def parity_legs(hip, fmt_name, with_others):
    """Oracle comparison of what the benchmark times, outside every timed region: the same layer graph with weights
    generated on the host, so that the CPU oracle (the checker) and the GPU hold the same model.  Teacher-forced
    greedy steps (both sides fed the oracle's tokens), every step's logits compared; a differing top-1 counts as a
    tie when the oracle's own best two are within two fp16 ulps.  Returns (headline parity, {name: parity})."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle
    from parity import greedy_parity
    from rwkv_lightning_cuda_amd.model import PRESETS, ModelDims, synth_weights
    fmts = {"f16": hip.FMT_F16, "w8": hip.FMT_W8, "w4": hip.FMT_W4}

    def sliced(preset, layers):
        d = PRESETS[preset]
        return ModelDims(L=layers, C=d.C, H=d.H, F=d.F, V=d.V, Rw=d.Rw, Ra=d.Ra, Rg=d.Rg, Rv=d.Rv)

    def leg(dims, weights, fmt_key, prompt_len, steps, what, rows=1):
        prompt = np.random.default_rng(89).integers(0, dims.V, (rows, prompt_len))
        res = greedy_parity(hip, oracle, dims, weights, fmts[fmt_key], prompt, steps, control=True)
        res["workload"] = "%s, %s weights: %d-token prompt, then %d greedy steps at batch %d, all %d logits of every step " \
                          "and row against the CPU oracle" % (what, fmt_key, prompt_len, steps, rows, dims.V)
        return res

    d8 = sliced("7.2B", 8)
    w8 = synth_weights(d8, 88)
    what = "7.2B shape at a quarter of the depth (8 of 32 layers, C 4096, full 65536-row head)"
    headline = leg(d8, w8, fmt_name, 8, 32, what)
    others = {}
    if with_others:
        if fmt_name == "w8":
            others["w4_parity"] = leg(d8, w8, "w4", 8, 16, what)
            # the few-row launches of 5 to 16 rows (products on the matrix core, LN2 folded into ffn.key, ffn.value in
            # column slices) and of 2 to 4 rows (the GEMV with several rows of x, one walk of ffn.value)
            d2l = sliced("7.2B", 2)
            w2l = synth_weights(d2l, 90)
            two = "7.2B shape, 2 of 32 layers (C 4096, full 65536-row head)"
            others["bs8_parity"] = leg(d2l, w2l, "w8", 4, 6, two, rows=8)
            others["bs3_parity"] = leg(d2l, w2l, "w8", 4, 6, two, rows=3)
            del w2l
        del w8
        d1 = PRESETS["0.1B"]
        others["cfg1_0p1b_f16_parity"] = leg(d1, synth_weights(d1, 12), "f16", 128, 32, "0.1B shape, all 12 layers")
        d2 = sliced("1.5B", 8)
        others["cfg2_1p5b_w8_parity"] = leg(d2, synth_weights(d2, 13), "w8", 8, 16,
                                            "1.5B shape at a third of the depth (8 of 24 layers, C 2048, full head)")
    return headline, others


def sampled_decode(hip, sess, dims, state, logits, B, first, steps=64):
    """The decode loop a server runs: forward, then the device sampler (repetition penalties, temperature, top-k,
    top-p) on the session stream, then the picked token ids back to the host, every step."""
    penalties = hip.DeviceArray.zeros((B, dims.V), np.float32)
    probs = hip.DeviceArray((B, dims.V), np.float32)
    picked = hip.DeviceArray((B,), np.int32)
    stream = sess.stream
    lib = hip.load()
    kw = dict(presence=0.5, frequency=0.1, decay=0.99, temperature=1.0, top_k=50, top_p=0.6, seed=3, stream=stream)
    tok = np.asarray(first, np.int64).reshape(B, 1)
    for phase_steps in (4, steps):
        hip.device_sync()
        t0 = time.perf_counter()
        for i in range(phase_steps):
            sess.forward(tok, state, logits, sync=False)
            hip.sample(B, dims.V, logits, penalties, probs, picked, step=i, **kw)
            hip.check(lib.rwkv_hip_stream_sync(ctypes.c_void_p(stream)))
            tok = picked.numpy().astype(np.int64).reshape(B, 1)
        dt = time.perf_counter() - t0
    return {"decode_sampled_bs%d_tok_s" % B: steps * B / dt, "decode_sampled_bs%d_ms_per_step" % B: dt * 1e3 / steps}


def sampler_call_us(hip, V, calls=200):
    """Microseconds per call of the device sampler alone (one launch; rows of V logits ~ N(0, 9), penalties on): without
    filters, with top-k 50 + top-p 0.6, and with top-p 0.9 alone, at 1 and 64 rows."""
    res = {}
    for B in (1, 64):
        g = np.random.default_rng(B)
        logits = hip.DeviceArray.from_numpy((g.standard_normal((B, V)) * 3).astype(np.float32))
        pen = hip.DeviceArray.zeros((B, V), np.float32)
        probs = hip.DeviceArray((B, V), np.float32)
        picked = hip.DeviceArray((B,), np.int32)
        for name, kw in (("plain", dict(top_k=0, top_p=1.0)), ("top_k50_top_p0.6", dict(top_k=50, top_p=0.6)),
                         ("top_p0.9", dict(top_k=0, top_p=0.9))):
            for phase in (5, calls):
                hip.device_sync()
                t0 = time.perf_counter()
                for i in range(phase):
                    hip.sample(B, V, logits, pen, probs, picked, presence=0.5, frequency=0.1, decay=0.99, temperature=1.0,
                               seed=3, step=i, **kw)
                hip.device_sync()
                dt = time.perf_counter() - t0
            res["bs%d_%s" % (B, name)] = dt * 1e6 / calls
    return res


def wkv7_op_long_context(hip, H, reps=3):
    """The WKV7 op alone at the long-context configuration: fp16 r,w,k,v,a,b [16,16384,64 H], fp32 state, raw-logit
    decay, one call.  Rows are 4096-token windows of one host-generated sequence (r,k,v ~ N(0,1); decay =
    exp(-exp(U(-6,-0.5))) given as its raw logit; kk = k/|k| per head, a = -kk, b = kk * sigmoid(U(-3,3)))."""
    res = {}
    Bw, Tw, seg = 16, 16384, 4096
    C = H * 64
    n = Bw * Tw * C
    n_win = Bw * (Tw // seg)
    base_T = seg + 64 * (n_win - 1)
    g = np.random.default_rng(11)
    kf = g.standard_normal((base_T, H, 64)).astype(np.float32)
    kk = kf / np.linalg.norm(kf, axis=-1, keepdims=True)
    sg = np.exp(g.uniform(-6.0, -0.5, (base_T, C)).astype(np.float32) + np.float32(0.5))
    host = [g.standard_normal((base_T, C)).astype(np.float16), np.log(sg / (1.0 - sg)).astype(np.float16),
            kf.reshape(base_T, C).astype(np.float16), g.standard_normal((base_T, C)).astype(np.float16),
            (-kk).reshape(base_T, C).astype(np.float16),
            (kk.reshape(base_T, C) / (1.0 + np.exp(-g.uniform(-3.0, 3.0, (base_T, C)).astype(np.float32)))).astype(np.float16)]
    del kf, kk, sg
    bufs = []
    for h in host:
        src = hip.DeviceArray.from_numpy(h)
        d = hip.DeviceArray((Bw, Tw, C), np.float16)
        for w_i in range(n_win):
            d.view(w_i * seg * C, (seg, C)).copy_from(src.view(64 * w_i * C, (seg, C)))
        src.free()
        bufs.append(d)
    del host
    bufs.append(hip.DeviceArray((Bw, Tw, C), np.float16))
    wstate = hip.DeviceArray.zeros((Bw, H, 64, 64), np.float32)
    r, w, k, v, a, b, y = bufs
    hip.wkv7(Bw, Tw, C, H, hip.W_RAW_LOGIT, hip.IO_F16, wstate, r, w, k, v, a, b, y)
    hip.device_sync()
    e0, e1 = hip.Event(), hip.Event()
    e0.record()
    for _ in range(reps):
        hip.wkv7(Bw, Tw, C, H, hip.W_RAW_LOGIT, hip.IO_F16, wstate, r, w, k, v, a, b, y)
    e1.record()
    hip.device_sync()
    ms = e0.elapsed_ms(e1) / reps
    res["wkv7_op"] = {"workload": "B=%d T=%d H=%d N=64, fp16 io, fp32 state, one call (average of %d)" % (Bw, Tw, H, reps),
                      "tok_s": Bw * Tw / (ms * 1e-3), "ms": ms,
                      "fp32_tflops": Bw * Tw * H * 10.0 * 64 * 64 / (ms * 1e-3) / 1e12,
                      "io_gb_s": n * 7 * 2 / (ms * 1e-3) / 1e9, "us_per_token_step": ms * 1e3 / Tw,
                      "outputs_finite": bool(np.isfinite(y.view(0, (Tw, C)).numpy().astype(np.float32)).all())}
    for d in bufs:
        d.free()

    return res["wkv7_op"]


def secondary_measurements(hip, model, dims, rng):
    """Batch-1, -2, -4, -8, -16 and -64 decode of the same model (128-token prefill per row, 64 timed steps) and the WKV7
    op alone."""
    from rwkv_lightning_cuda_amd.model import Session, State
    res = {}
    for B in (1, 2, 4, 8, 16, 64):
        sess = Session(model)
        state = State(dims, B)
        logits = hip.DeviceArray((B, dims.V), np.float32)
        sess.forward(rng.integers(0, dims.V, (B, 128)), state, logits)
        first = rng.integers(0, dims.V, (B,))
        sess.decode_greedy(first, 8, state, logits)
        hip.device_sync()
        t0 = time.perf_counter()
        steps = 64
        sess.decode_greedy(first, steps, state, logits)
        hip.device_sync()
        dt = time.perf_counter() - t0
        state_bytes = B * (2 * dims.L * dims.H * 64 * 64 * 4 + 2 * dims.L * 2 * dims.C * 2)
        res["decode_bs%d_tok_s" % B] = steps * B / dt
        res["decode_bs%d_ms_per_step" % B] = dt * 1e3 / steps
        res["decode_bs%d_hbm_fraction" % B] = (model.weight_bytes() + state_bytes) / (dt / steps) / 1e9 / HBM_PEAK_GBPS
        if B not in (2, 4):
            res.update(sampled_decode(hip, sess, dims, state, logits, B, first))
        sess.close()
        del state, logits

    # The same decode with the WKV state kept in fp16 (the reference server's default, use_wkv32 == false): half the
    # state bytes per step.  Reported beside the fp32-state figures above, never instead of them.
    for B in (16, 64):
        sess = Session(model)
        sess.set_wkv_fp16(True)
        state = State(dims, B, wkv_fp16=True)
        logits = hip.DeviceArray((B, dims.V), np.float32)
        sess.forward(rng.integers(0, dims.V, (B, 128)), state, logits)
        first = rng.integers(0, dims.V, (B,))
        sess.decode_greedy(first, 8, state, logits)
        hip.device_sync()
        t0 = time.perf_counter()
        steps = 64
        sess.decode_greedy(first, steps, state, logits)
        hip.device_sync()
        dt = time.perf_counter() - t0
        res["decode_fp16_state_bs%d_tok_s" % B] = steps * B / dt
        res["decode_fp16_state_bs%d_ms_per_step" % B] = dt * 1e3 / steps
        sess.close()
        del state, logits

    res["wkv7_op"] = wkv7_op_long_context(hip, dims.H)
    e0, e1 = hip.Event(), hip.Event()

    # the reference's own small operator case: B = 1, T = 64, H = 12, fp32 io (average over 20 calls)
    B0, T0, H0 = 1, 64, 12
    C0 = H0 * 64
    rng = np.random.default_rng(7)
    small = [hip.DeviceArray.from_numpy((rng.standard_normal((B0, T0, C0)) * 0.5).astype(np.float32)) for _ in range(6)]
    y0 = hip.DeviceArray((B0, T0, C0), np.float32)
    s0 = hip.DeviceArray.zeros((B0, H0, 64, 64), np.float32)
    r, w, k, v, a, b = small
    for _ in range(3):
        hip.wkv7(B0, T0, C0, H0, hip.W_RAW_LOGIT, hip.IO_F32, s0, r, w, k, v, a, b, y0)
    hip.device_sync()
    e0.record()
    for _ in range(20):
        hip.wkv7(B0, T0, C0, H0, hip.W_RAW_LOGIT, hip.IO_F32, s0, r, w, k, v, a, b, y0)
    e1.record()
    hip.device_sync()
    us = e0.elapsed_ms(e1) * 1e3 / 20
    res["wkv7_op_small"] = {"workload": "B=1 T=64 H=12 N=64, fp32 io, fp32 state", "us_per_call": us,
                            "tok_s": B0 * T0 / (us * 1e-6)}
    return res


def engine_boundary_rates(preset, fmt_name):
    """tok/s through the drop-in boundary: the C++ host API (InferenceEngine::batch_generate_stream over ModelBackend,
    one fresh GenerationState and logits buffer per request, device sampler + picked ids back to the host every step)
    as its own GenerationStats report them - the reference server's decode_speed / prefill_speed counters.  Runs the
    tool tests/cpp/bin/engine_rate_bench as a child process (its own model of the same shape and format)."""
    import subprocess
    exe = os.path.join(ROOT, "tests", "cpp", "bin", "engine_rate_bench")
    if not os.path.exists(exe):
        return {"error": "tests/cpp/bin/engine_rate_bench is not built"}
    out = {}
    for name, batch, tokens, sampled in (("greedy_bs1", 1, 128, 0), ("sampled_bs1", 1, 128, 1), ("greedy_bs16", 16, 64, 0),
                                         ("sampled_bs16", 16, 64, 1)):
        cmd = [exe, ROOT, "synthetic:%s:%s" % (preset, fmt_name), str(batch), str(tokens), "3", str(sampled), "1"]
        proc = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        if proc.returncode != 0:
            out[name] = {"error": proc.stderr.strip()[-300:]}
            continue
        reqs = [json.loads(line) for line in proc.stdout.splitlines() if line.startswith("{")]
        out[name] = {
            "first_request_decode_tok_s": reqs[0]["decode_tok_s"],
            "steady_decode_tok_s": reqs[-1]["decode_tok_s"],
            "steady_decode_ms_per_step": reqs[-1]["decode_ms_per_step"],
            "steady_prefill_tok_s": reqs[-1]["prefill_tok_s"],
            "prompt_tokens": reqs[-1]["prompt_tokens"], "generated_tokens": reqs[-1]["generated_tokens"],
            "graph_captures_per_request": [r["graph_captures"] for r in reqs],
        }
    out["what"] = ("InferenceEngine::batch_generate_stream over ModelBackend(synthetic:%s:%s, fp32 WKV state), 3 requests "
                   "of identical prompts each; rates from GenerationStats" % (preset, fmt_name))
    return out


def other_configs(hip, rng):
    """Benchmark configurations 1 and 2 on the same GPU: the 0.1B shape with fp16 weights (512-token prompt in chunks
    of 128, then 128 greedy steps at batch 1) and the 1.5B shape W8A16 (256-token prefill per sequence, then decode at
    batch 1, 8 and 64)."""
    from rwkv_lightning_cuda_amd.model import PRESETS, HipModel, Session, State
    res = {}
    dims = PRESETS["0.1B"]
    model = HipModel.random_on_device(dims, hip.FMT_F16, seed=2)
    sess = Session(model)
    lg = hip.DeviceArray((1, dims.V), np.float32)
    prompt = rng.integers(0, dims.V, (1, 512))
    warm = State(dims, 1)
    sess.forward(prompt[:, :128], warm, lg)
    st = State(dims, 1)
    hip.device_sync()
    t0 = time.perf_counter()
    for c0 in range(0, 512, 128):
        sess.forward(prompt[:, c0:c0 + 128], st, lg, sync=False)
    hip.device_sync()
    res["cfg1_0p1b_f16_prefill512_tok_s"] = 512 / (time.perf_counter() - t0)
    first = rng.integers(0, dims.V, (1,))
    sess.decode_greedy(first, 8, st, lg)
    hip.device_sync()
    t0 = time.perf_counter()
    sess.decode_greedy(first, 128, st, lg)
    hip.device_sync()
    dt = time.perf_counter() - t0
    res["cfg1_0p1b_f16_decode_bs1_tok_s"] = 128 / dt
    res["cfg1_0p1b_f16_decode_bs1_ms_per_step"] = dt * 1e3 / 128
    sess.close()
    model.close()
    del model, st, warm

    dims = PRESETS["1.5B"]
    model = HipModel.random_on_device(dims, hip.FMT_W8, seed=3)
    wbytes = model.weight_bytes()
    for B in (1, 8, 64):
        sess = Session(model)
        st = State(dims, B)
        lg = hip.DeviceArray((B, dims.V), np.float32)
        prompt = rng.integers(0, dims.V, (B, 256))
        for c0 in range(0, 256, 128):
            sess.forward(prompt[:, c0:c0 + 128], st, lg, sync=False)
        first = rng.integers(0, dims.V, (B,))
        sess.decode_greedy(first, 8, st, lg)
        hip.device_sync()
        t0 = time.perf_counter()
        sess.decode_greedy(first, 64, st, lg)
        hip.device_sync()
        dt = time.perf_counter() - t0
        sbytes = B * (2 * dims.L * dims.H * 64 * 64 * 4 + 2 * dims.L * 2 * dims.C * 2)
        res["cfg2_1p5b_w8_decode_bs%d_tok_s" % B] = 64 * B / dt
        res["cfg2_1p5b_w8_decode_bs%d_ms_per_step" % B] = dt * 1e3 / 64
        res["cfg2_1p5b_w8_decode_bs%d_hbm_fraction" % B] = (wbytes + sbytes) / (dt / 64) / 1e9 / HBM_PEAK_GBPS
        sess.close()
        del st, lg
    model.close()
    return res


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
    if args.copy_calibration > 0:
        src = hip.DeviceArray.zeros((args.copy_calibration,), np.uint8)
        dst = hip.DeviceArray((args.copy_calibration,), np.uint8)
        for _ in range(2):
            dst.copy_from(src)
        hip.device_sync()
        print(json.dumps({"copy_calibration_bytes": args.copy_calibration}))
        return
    if args.wkv7_op_only:
        print(json.dumps({"wkv7_op": wkv7_op_long_context(hip, 64, reps=1)}))
        return
    dims = PRESETS[args.preset]
    fmt = {"f16": hip.FMT_F16, "w8": hip.FMT_W8, "w4": hip.FMT_W4}[args.fmt]
    B = args.batch

    model = HipModel.random_on_device(dims, fmt, seed=1)
    sess = Session(model)
    if args.no_graph:
        sess.set_graph(False)
    if args.wkv_fp16:
        sess.set_wkv_fp16(True)
    if args.fused_ln >= 0:
        sess.set_fused_ln(bool(args.fused_ln))

    def new_state(b):
        return State(dims, b, wkv_fp16=args.wkv_fp16)

    state = new_state(B)
    logits = hip.DeviceArray((B, dims.V), np.float32)
    rng = np.random.default_rng(0)
    also = {}
    if args.prefill > 0:
        prompt = rng.integers(0, dims.V, (B, args.prefill))
        warm = new_state(B)
        sess.forward(prompt[:, :min(128, args.prefill)], warm, logits)  # sizes the arena, warms the kernels
        del warm
        hip.device_sync()
        tp = time.perf_counter()
        for t0 in range(0, args.prefill, 128):
            sess.forward(prompt[:, t0:t0 + 128], state, logits, sync=False)
        hip.device_sync()
        tp = time.perf_counter() - tp
        also["prefill_tok_s"] = B * args.prefill / tp
        also["prefill_workload"] = "%d-token prompt x batch %d in chunks of 128 (state carried in HBM)" % (args.prefill, B)
        if not args.no_also and args.prefill >= 128:
            # MFMA fraction of the chunk's GEMM launches: one more chunk, eagerly, GEMM launches bracketed by events
            scratch = new_state(B)
            sess.set_profile(True)
            sess.read_profile()
            sess.forward(prompt[:, :128], scratch, logits, sync=False)
            launches, total_ms = sess.read_profile()
            sess.set_profile(False)
            del scratch
            rows = B * 128
            flops = 2.0 * rows * dims.L * (4 * dims.C * dims.C + 2 * dims.C * dims.F)
            also["prefill_gemm"] = {"bound": "mfma", "achieved": flops / (total_ms * 1e-3) / 1e12,
                                    "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                    "frac": flops / (total_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS,
                                    "kernel": "gemm_stream_kernel (+ split-K reduce), M = %d rows" % rows,
                                    "launches": launches, "sum_launch_ms": total_ms,
                                    # at M = 128 the launches are weight-streaming bound: the same time against HBM
                                    "weights_gb_s": model.weight_bytes() / (total_ms * 1e-3) / 1e9,
                                    "hbm_frac": model.weight_bytes() / (total_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
            # the same prompt in chunks of 512 and 2048 (the chunk width is the caller's choice: wider chunks
            # stream the weights once per chunk), into a scratch state
            for width in (512, 2048):
                if B * width > 4096:
                    continue
                wide = new_state(B)
                sess.forward(prompt[:, :min(width, args.prefill)], wide, logits)
                hip.device_sync()
                tw = time.perf_counter()
                for t0 in range(0, args.prefill, width):
                    sess.forward(prompt[:, t0:t0 + width], wide, logits, sync=False)
                hip.device_sync()
                tw = time.perf_counter() - tw
                also["prefill_chunk%d_tok_s" % width] = B * args.prefill / tw
                del wide
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

    # one-sequence steps over int8 or fp16 weights skip the ffn.value rows with a zero activation (the reference's default
    # for rows == 1, include/rwkv7_fast_v4_common.hpp:198-211); the dense product is timed beside it below
    sparse_value = B == 1 and dims.F % 256 == 0 and dims.C % 16 == 0
    if sparse_value and not args.no_also:
        sess.set_sparse_ffn(0)
        sess.decode_greedy(first, min(args.warmup, 8) or 1, state, logits)
        hip.device_sync()
        td = time.perf_counter()
        sess.decode_greedy(first, min(args.steps, 64), state, logits)
        hip.device_sync()
        also["decode_dense_ffn_value_tok_s"] = min(args.steps, 64) * B / (time.perf_counter() - td)
        sess.set_sparse_ffn(4)
        act = sess.debug_buffer("act", (B, dims.F))
        also["ffn_value_rows_skipped_fraction_last_layer"] = float(np.mean(act == 0))

    weight_bytes = model.weight_bytes()
    state_bytes = B * (2 * dims.L * dims.H * 64 * 64 * (2 if args.wkv_fp16 else 4) + 2 * dims.L * 2 * dims.C * 2)
    # bytes the timed step really moved: the row-skipping ffn.value reads only the rows with a non-zero activation
    # (fraction measured on the last layer's activations of the last step)
    skipped = also.get("ffn_value_rows_skipped_fraction_last_layer", 0.0) if sparse_value else 0.0
    value_code_bytes = dims.L * dims.C * dims.F * {"f16": 2.0, "w8": 1.0, "w4": 0.5}[args.fmt]
    moved_bytes = weight_bytes + state_bytes - skipped * value_code_bytes
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
        "dtype": "f16",
        "data": "synthetic (random-init N(0,0.02) weights quantised on load, random token ids)",
        "config": {"workload": "RWKV-7 %s-shape greedy decode, batch %d, %d-token prefill, lm_head+argmax on device"
                               % (args.preset, B, args.prefill),
                   "L": dims.L, "C": dims.C, "H": dims.H, "F": dims.F, "V": dims.V,
                   "weight_format": args.fmt, "arithmetic": "fp16 activations, fp32 accumulate, %s WKV state" % ("fp16" if args.wkv_fp16 else "fp32"),
                   "hip_graph": not args.no_graph, "sparse_ffn_value": sparse_value,
                   "weight_bytes_per_step": weight_bytes,
                   "state_bytes_per_step": state_bytes,
                   # dense convention: every weight byte counted once per step, whether the step read it or not
                   "step_hbm_fraction": (weight_bytes + state_bytes) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                   # the bytes the step really moved (rows of ffn.value with a zero activation are not read)
                   "bytes_moved_per_step": moved_bytes,
                   "bytes_moved_fraction": moved_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                   "distinct_tokens": int(len(np.unique(toks)))},
    }
    if "decode_dense_ffn_value_tok_s" in also:
        # like for like: the same dense byte count over the step time with the dense ffn.value product
        out["config"]["step_hbm_fraction_dense_ffn_value"] = \
            (weight_bytes + state_bytes) * also["decode_dense_ffn_value_tok_s"] / B / 1e9 / HBM_PEAK_GBPS

    if not args.no_roofline:
        # The weight-streaming linear launches of the same steps alone, eagerly and back to back on the session
        # stream, each pass bracketed by one pair of HIP events (the kernels' duration does not depend on the
        # data; the small kernels between them are skipped so that no event sits between two launches).  All
        # 7 GB of weights stream from HBM on every pass, exactly as in the timed run.
        scratch_state = new_state(B)
        sess.set_profile(2)
        sess.read_profile()
        tok = toks[-1].reshape(B, 1).astype(np.int64)
        n_prof = min(args.steps, 32)
        for _ in range(n_prof):
            sess.forward(tok, scratch_state, logits, sync=False)
        launches, total_ms = sess.read_profile()
        sess.set_profile(0)
        del scratch_state
        gemv_bytes, per_step = gemv_bytes_per_step(dims, args.fmt, sparse_value)
        assert launches == per_step * n_prof, (launches, per_step, n_prof)
        bytes_per_launch = gemv_bytes / per_step
        avg_ms = total_ms / launches
        achieved = bytes_per_launch / (avg_ms * 1e-3) / 1e9
        traffic, traffic_rec = measured_traffic((args.preset, args.fmt, B))
        out["roofline"] = {
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic,
            "kernel": "linear_gemv_row1_kernel (weight-streaming GEMV: r/k/v + LoRA rank-ins with the LayerNorm prologue, "
                      "output, ffn.key with the LayerNorm prologue%s, lm_head)" % ("" if sparse_value else ", ffn.value"),
            "bytes_per_launch": bytes_per_launch, "avg_launch_us": avg_ms * 1e3, "launches_per_step": per_step,
            "traffic_source": (traffic_rec or {}).get("profile"),
            "traffic_stale": bool((traffic_rec or {}).get("stale", False)),
        }

    if not args.no_also:
        also.update(secondary_measurements(hip, model, dims, rng))
    sess.close()
    if not args.no_also and args.fmt == "w8":
        # the same shape with int4 weights (asymmetric, groups of 128), batch 1
        del model
        m4 = HipModel.random_on_device(dims, hip.FMT_W4, seed=1)
        s4 = Session(m4)
        st4 = State(dims, 1)
        lg4 = hip.DeviceArray((1, dims.V), np.float32)
        s4.forward(rng.integers(0, dims.V, (1, 128)), st4, lg4)
        f4 = rng.integers(0, dims.V, (1,))
        s4.decode_greedy(f4, 8, st4, lg4)
        hip.device_sync()
        t4 = time.perf_counter()
        s4.decode_greedy(f4, 64, st4, lg4)
        hip.device_sync()
        t4 = time.perf_counter() - t4
        also["decode_w4_bs1_tok_s"] = 64 / t4
        sb4 = 2 * dims.L * dims.H * 64 * 64 * 4 + 2 * dims.L * 2 * dims.C * 2
        also["decode_w4_bs1_hbm_fraction"] = (m4.weight_bytes() + sb4) / (t4 / 64) / 1e9 / HBM_PEAK_GBPS
        s4.close()
        del m4
    if not args.no_also and args.preset == "7.2B":
        also.update(other_configs(hip, rng))
        # what a launch that waits for its predecessor costs on this box: a captured graph of 260 near-empty launches
        also["launch_chain_us_per_link_graph"] = hip.measure_launch_chain(260, 256, 256, True, 20)
        also["launch_chain_us_per_link_direct"] = hip.measure_launch_chain(260, 256, 256, False, 20)
        also["engine_boundary"] = engine_boundary_rates(args.preset, args.fmt)
        also["sampler_us_per_call"] = sampler_call_us(hip, dims.V)
    if not args.no_parity and args.preset == "7.2B":
        out["parity"], more = parity_legs(hip, args.fmt, not args.no_also)
        also.update(more)
    if also:
        out["also"] = also
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(dims, args.fmt)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
