"""Teacher-forced greedy parity of the GPU layer graph against the CPU oracle, as figures (not assertions): used by
the GPU tests (which assert on them) and by bench.py (which reports them beside the rates, outside its timed
regions).  The oracle is the checker here, never the thing measured."""
import os

import numpy as np


def _cosine(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b)))


def _max_rel(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.max(np.abs(got - ref)) / max(float(np.max(np.abs(ref))), 1e-30))


def is_tie(oracle_row, want, got):
    """A top-1 that differs from the oracle's counts as a tie when the oracle's own two candidates are within two
    fp16 ulps (logits are fp16-rounded values; a random-init head is nearly flat at the top)."""
    gap = float(oracle_row[want] - oracle_row[got])
    ulp = float(np.spacing(np.float16(abs(oracle_row[want]))))
    return gap <= 2 * ulp


def greedy_parity(hip, orc, dims, weights, fmt, prompt, steps, chunk=128, wkv_fp16=False, models=None, control=False):
    """Prefills `prompt` [B,P] in chunks, then `steps` greedy steps in which both sides are fed the ORACLE's tokens;
    every step's logits are compared.  Returns a dict:
      cosine            smallest logits cosine over the prompt's last token and all steps (per row)
      max_rel           largest max|gpu - oracle| / max|oracle| over the same logit rows
      top1_match_steps  rows x steps whose GPU argmax is the oracle's
      ties              differing argmax where the oracle's best two are within 2 fp16 ulps
      mismatches        differing argmax that is no tie
      steps, rows       what was compared
      state_max_rel     WKV state against the oracle's after the last step (of its scale), worst layer;
      state_max_rel_by_layer  the same per layer
      control_*         (with control=True) the same prompt through a second GPU path - token by token through the
                        decode kernels instead of one call through the GEMM / sequence kernels - against the first:
                        how far two correct summation orders drift apart on this model (logits cosine after the
                        prompt, state per layer).  Random-init weights amplify the first tokens' differences from
                        layer to layer (an almost empty WKV state makes the per-head GroupNorm ill-conditioned), so
                        this is the yardstick for the oracle comparison at depth.
    `models` = (oracle model, GPU model) reuses models built by the caller."""
    from rwkv_lightning_cuda_amd.model import HipModel, Session, State
    orc.set_threads(min(16, os.cpu_count() or 1))  # the oracle's results do not depend on the thread count
    if models is None:
        omodel = orc.Model(dims, weights, fmt)
        gmodel = HipModel.from_host_weights(dims, weights, fmt)
    else:
        omodel, gmodel = models
    prompt = np.asarray(prompt, np.int64)
    B, P = prompt.shape
    sess = Session(gmodel)
    gstate = State(dims, B, wkv_fp16=wkv_fp16)
    glogits = hip.DeviceArray((B, dims.V), np.float32)
    ostate = omodel.new_state(B, wkv_fp16=wkv_fp16)
    for c0 in range(0, P, chunk):
        sess.forward(prompt[:, c0:c0 + chunk], gstate, glogits)
        ologits = omodel.forward(prompt[:, c0:c0 + chunk], ostate)
    res = {"cosine": 1.0, "max_rel": 0.0, "top1_match_steps": 0, "ties": 0, "mismatches": 0, "steps": steps, "rows": B}
    if control:
        cstate = State(dims, B, wkv_fp16=wkv_fp16)
        clogits = hip.DeviceArray((B, dims.V), np.float32)
        for t in range(P):
            sess.forward(prompt[:, t:t + 1], cstate, clogits)
        res["control_cosine"] = min(_cosine(a, b) for a, b in zip(glogits.numpy(), clogits.numpy()))
        ga, gb = gstate.wkv.numpy().astype(np.float32), cstate.wkv.numpy().astype(np.float32)
        res["control_state_max_rel_by_layer"] = [_max_rel(ga[l], gb[l]) for l in range(dims.L)]
        del cstate, clogits

    def compare(g, o, count):
        for b in range(B):
            res["cosine"] = min(res["cosine"], _cosine(g[b], o[b]))
            res["max_rel"] = max(res["max_rel"], _max_rel(g[b], o[b]))
            if not count:
                continue
            want, got = int(np.argmax(o[b])), int(np.argmax(g[b]))
            if want == got:
                res["top1_match_steps"] += 1
            elif is_tie(o[b], want, got):
                res["ties"] += 1
            else:
                res["mismatches"] += 1

    compare(glogits.numpy(), ologits, False)
    tok = np.argmax(ologits, axis=1).reshape(B, 1).astype(np.int64)
    for _ in range(steps):
        sess.forward(tok, gstate, glogits)
        ologits = omodel.forward(tok, ostate)
        compare(glogits.numpy(), ologits, True)
        tok = np.argmax(ologits, axis=1).reshape(B, 1).astype(np.int64)
    gw, ow = gstate.wkv.numpy().astype(np.float32), ostate[1].astype(np.float32)
    res["state_max_rel_by_layer"] = [_max_rel(gw[l], ow[l]) for l in range(dims.L)]
    res["state_max_rel"] = max(res["state_max_rel_by_layer"])
    res["elapsed_ok"] = gstate.elapsed.numpy().tolist() == [P + steps] * B
    sess.close()
    if models is None:
        gmodel.close()
    orc.set_threads(1)
    return res
