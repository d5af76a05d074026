"""Independent float64 numpy restatement of the RWKV-7 ("x070") layer graph, written from the model's
equations rather than from the oracle's code: it has no fp16 rounding points and no sequential
summation order, so it pins the oracle's graph (op order, layer-0 special cases, state handling) up
to fp16 noise.  Weights use the layout of rwkv_lightning_cuda_amd.model.synth_weights.
"""
import numpy as np


def _f(a):
    return np.asarray(a, dtype=np.float64)


def layer_norm(x, w, b, eps=1e-5):
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * _f(w) + _f(b)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def time_shift(x, prev_row):
    """x [T,C] -> the previous token's row for every t (prev_row at t=0)."""
    return np.concatenate([prev_row[None, :], x[:-1]], axis=0)


def forward(dims, weights, tokens, state=None, mats=None):
    """tokens [B,T] -> (logits [B,V] of the last token, new state).  state = dict(shift [L,2,B,C],
    wkv [L,B,H,64,64]).  mats, if given, maps (layer, name) -> float matrix replacing the fp16 one (used to
    feed the dequantised weights of a quantised model)."""
    tokens = np.asarray(tokens)
    B, T = tokens.shape
    L, C, H = dims.L, dims.C, dims.H
    if state is None:
        state = dict(shift=np.zeros((L, 2, B, C)), wkv=np.zeros((L, B, H, 64, 64)))

    def mat(layer, name):
        if mats is not None and (layer, name) in mats:
            return _f(mats[(layer, name)])
        return _f(weights["head"] if name == "head" else weights["layers"][layer][name])

    logits = np.zeros((B, dims.V))
    for bi in range(B):
        x = _f(weights["emb_ln0"])[tokens[bi]]  # [T,C], ln0 already applied
        v_first = None
        for l in range(L):
            w = weights["layers"][l]
            # ---- time mix
            xx = layer_norm(x, w["ln1_w"], w["ln1_b"])
            prev = time_shift(xx, state["shift"][l, 0, bi])
            state["shift"][l, 0, bi] = xx[-1]
            dx = prev - xx
            xr, xw, xk, xv, xa, xg = (xx + dx * _f(w[n]) for n in ("x_r", "x_w", "x_k", "x_v", "x_a", "x_g"))
            r = xr @ mat(l, "att_r").T
            k = xk @ mat(l, "att_k").T
            v = xv @ mat(l, "att_v").T
            w_raw = _f(w["w0"]) + np.tanh(xw @ _f(w["w1"]).T) @ _f(w["w2"]).T
            a = sigmoid(_f(w["a0"]) + (xa @ _f(w["a1"]).T) @ _f(w["a2"]).T)
            g = sigmoid(xg @ _f(w["g1"]).T) @ _f(w["g2"]).T
            if l == 0:
                v_first = v
            else:
                v = v + (v_first - v) * sigmoid(_f(w["v0"]) + (xv @ _f(w["v1"]).T) @ _f(w["v2"]).T)
            decay = np.exp(-np.exp(-0.5) * sigmoid(w_raw))
            kk = (k * _f(w["k_k"])).reshape(T, H, 64)
            kk = kk / np.maximum(np.linalg.norm(kk, axis=-1, keepdims=True), 1e-12)
            kk = kk.reshape(T, C)
            k = k * (1.0 + (a - 1.0) * _f(w["k_a"]))
            # ---- WKV recurrence per head: S <- S diag(d) + (S a~) b~^T + v k^T with a~ = -kk, b~ = kk*a
            y = np.zeros((T, C))
            S = state["wkv"][l, bi]
            for t in range(T):
                for h in range(H):
                    sl = slice(h * 64, (h + 1) * 64)
                    Sh = S[h]
                    sa = Sh @ (-kk[t, sl])
                    Sh = Sh * decay[t, sl][None, :] + np.outer(sa, kk[t, sl] * a[t, sl]) + np.outer(v[t, sl], k[t, sl])
                    S[h] = Sh
                    y[t, sl] = Sh @ r[t, sl]
            # ---- per-head GroupNorm, bonus term, gate, output projection
            yh = y.reshape(T, H, 64)
            mu = yh.mean(axis=-1, keepdims=True)
            var = ((yh - mu) ** 2).mean(axis=-1, keepdims=True)
            yn = ((yh - mu) / np.sqrt(var + 64e-5)).reshape(T, C) * _f(w["lnx_w"]) + _f(w["lnx_b"])
            bonus = (r * k * _f(w["r_k"])).reshape(T, H, 64).sum(axis=-1, keepdims=True) * v.reshape(T, H, 64)
            x = x + ((yn + bonus.reshape(T, C)) * g) @ mat(l, "att_o").T
            # ---- channel mix
            xx = layer_norm(x, w["ln2_w"], w["ln2_b"])
            prev = time_shift(xx, state["shift"][l, 1, bi])
            state["shift"][l, 1, bi] = xx[-1]
            kx = xx + (prev - xx) * _f(w["ffn_x_k"])
            hid = np.maximum(kx @ mat(l, "ffn_key").T, 0.0) ** 2
            x = x + hid @ mat(l, "ffn_value").T
        xo = layer_norm(x[-1], weights["ln_out_w"], weights["ln_out_b"])
        logits[bi] = xo @ mat(-1, "head").T
    return logits, state
