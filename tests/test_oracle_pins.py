"""CPU tests that pin the oracle (oracle/rwkv_oracle.cpp) against independent evidence: numpy's IEEE
fp16, float64 closed forms and brute force, special cases that reduce to textbook routines, the known
answers held by the reference's own tests, and an independent numpy restatement of the layer graph.
A dropped term, a wrong sign or a transposed operand in the oracle fails at least one of these.
"""
import numpy as np
import pytest

import np_model
import oracle as orc
from inputs import pattern_value, wkv_inputs


def f64(a):
    return np.asarray(a, np.float64)


# ------------------------------------------------------------------------------------------- fp16
def test_f16_to_f32_exhaustive():
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    got = orc.f16_to_f32(allh)
    ref = allh.astype(np.float32)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_f32_to_f16_rne_matches_numpy():
    rng = np.random.default_rng(0)
    parts = [rng.standard_normal(100000).astype(np.float32) * np.float32(s) for s in (1e-8, 1e-6, 1e-4, 1e-2, 1, 100, 3e4)]
    # every fp16 value, the midpoints between neighbours (ties) and their float32 neighbours
    allh = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mids = (allh[:-1].astype(np.float64) + allh[1:].astype(np.float64)) / 2
    mids32 = mids.astype(np.float32)
    edge = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                     2.0 ** -25 * 1.0000001, 2.0 ** -26, 5.96e-8, 6.1e-5], np.float32)
    x = np.concatenate(parts + [allh, -allh, mids32, np.nextafter(mids32, np.float32(np.inf)),
                                np.nextafter(mids32, np.float32(-np.inf)), edge])
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16)
    got = orc.f32_to_f16(x)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))
    nan = orc.f32_to_f16(np.array([np.nan], np.float32))
    assert np.isnan(nan[0])


# ------------------------------------------------------------------------------------------- WKV7
def wkv_bruteforce(state, r, d, k, v, a, b):
    """float64: S <- S diag(d) + (S a) b^T + v k^T ; y = S r, per (batch, head)."""
    B, T, C = r.shape
    H = C // 64
    S = f64(state).copy()
    y = np.zeros((B, T, C))
    for bi in range(B):
        for h in range(H):
            sl = slice(h * 64, (h + 1) * 64)
            M = S[bi, h]
            for t in range(T):
                sa = M @ f64(a[bi, t, sl])
                M = M * f64(d[bi, t, sl])[None, :] + np.outer(sa, f64(b[bi, t, sl])) + np.outer(f64(v[bi, t, sl]), f64(k[bi, t, sl]))
                y[bi, t, sl] = M @ f64(r[bi, t, sl])
            S[bi, h] = M
    return y, S


def test_wkv7_matches_float64_bruteforce():
    B, T, H = 2, 8, 2
    inp = wkv_inputs(B, T, H, seed=1)
    rng = np.random.default_rng(2)
    s0 = rng.standard_normal((B, H, 64, 64)).astype(np.float32) * 0.1
    y_ref, s_ref = wkv_bruteforce(s0, inp["r"], inp["decay"], inp["k"], inp["v"], inp["a"], inp["b"])
    s = s0.copy()
    y = orc.wkv7(s, inp["r"], inp["decay"], inp["k"], inp["v"], inp["a"], inp["b"], H, w_mode=1)
    assert np.max(np.abs(y - y_ref)) <= 1e-5 * np.max(np.abs(y_ref))
    assert np.max(np.abs(s - s_ref)) <= 1e-5 * np.max(np.abs(s_ref))
    # a wrong transpose of the state would survive neither check: v k^T is not symmetric
    assert not np.allclose(s, np.swapaxes(s, -1, -2), atol=1e-3)


def test_wkv7_raw_logit_equals_decay_mode():
    B, T, H = 1, 6, 3
    inp = wkv_inputs(B, T, H, seed=3)
    s1 = np.zeros((B, H, 64, 64), np.float32)
    s2 = np.zeros((B, H, 64, 64), np.float32)
    y1 = orc.wkv7(s1, inp["r"], inp["decay"], inp["k"], inp["v"], inp["a"], inp["b"], H, w_mode=1)
    y2 = orc.wkv7(s2, inp["r"], inp["w_raw"], inp["k"], inp["v"], inp["a"], inp["b"], H, w_mode=0)
    # decay = exp(-exp(x)) and the logit with exp(-e^-1/2 sigmoid(w)) = decay agree to fp32 rounding of the map
    assert np.max(np.abs(y1 - y2)) <= 2e-4 * np.max(np.abs(y1))
    # the decay map itself: w -> exp(-e^-0.5 * sigmoid(w)), checked on a one-token, one-nonzero-column state
    w = np.linspace(-8, 8, 64).astype(np.float32).reshape(1, 1, 64)
    s = np.ones((1, 1, 64, 64), np.float32)
    z = np.zeros((1, 1, 64), np.float32)
    orc.wkv7(s, z, w, z, z, z, z, 1, w_mode=0)
    want = np.exp(-np.exp(-0.5) / (1.0 + np.exp(-f64(w[0, 0]))))
    assert np.max(np.abs(s[0, 0, 5] - want)) <= 1e-6


def test_wkv7_special_cases():
    B, T, H = 1, 5, 1
    inp = wkv_inputs(B, T, H, seed=4)
    z = np.zeros_like(inp["a"])
    one = np.ones_like(inp["decay"])
    # a = b = 0, d = 1: plain cumulative sum of outer products v k^T
    s = np.zeros((B, H, 64, 64), np.float32)
    orc.wkv7(s, inp["r"], one, inp["k"], inp["v"], z, z, H, w_mode=1)
    want = sum(np.outer(f64(inp["v"][0, t]), f64(inp["k"][0, t])) for t in range(T))
    assert np.max(np.abs(s[0, 0] - want)) <= 1e-5
    # a = b = 0: decayed linear attention, S_T = sum_t v_t k_t^T prod_{tau>t} diag(d_tau)
    s = np.zeros((B, H, 64, 64), np.float32)
    y = orc.wkv7(s, inp["r"], inp["decay"], inp["k"], inp["v"], z, z, H, w_mode=1)
    want = np.zeros((64, 64))
    for t in range(T):
        dec = np.prod(f64(inp["decay"][0, t + 1:]), axis=0) if t + 1 < T else np.ones(64)
        want += np.outer(f64(inp["v"][0, t]), f64(inp["k"][0, t]) * dec)
    assert np.max(np.abs(s[0, 0] - want)) <= 1e-5
    # r = e_j reads column j of the updated state
    r = np.zeros_like(inp["r"])
    r[0, :, 17] = 1.0
    s = np.zeros((B, H, 64, 64), np.float32)
    for t in range(T):
        yt = orc.wkv7(s, r[:, t:t + 1], inp["decay"][:, t:t + 1], inp["k"][:, t:t + 1], inp["v"][:, t:t + 1],
                      inp["a"][:, t:t + 1], inp["b"][:, t:t + 1], H, w_mode=1)
        assert np.array_equal(yt[0, 0], s[0, 0, :, 17])


def test_wkv7_t_split_and_permutation():
    B, T, H = 2, 9, 2
    inp = wkv_inputs(B, T, H, seed=5, dtype=np.float16)
    names = ["r", "w_raw", "k", "v", "a", "b"]
    s1 = np.zeros((B, H, 64, 64), np.float32)
    y1 = orc.wkv7(s1, *[inp[n] for n in names], H, 0)
    s2 = np.zeros((B, H, 64, 64), np.float32)
    ya = orc.wkv7(s2, *[np.ascontiguousarray(inp[n][:, :4]) for n in names], H, 0)
    yb = orc.wkv7(s2, *[np.ascontiguousarray(inp[n][:, 4:]) for n in names], H, 0)
    assert np.array_equal(s1.view(np.uint32), s2.view(np.uint32))
    assert np.array_equal(np.concatenate([ya, yb], axis=1).view(np.uint16), y1.view(np.uint16))
    # swapping the two batch rows and the two heads permutes outputs and state the same way
    perm = {n: np.ascontiguousarray(inp[n][::-1].reshape(B, T, H, 64)[:, :, ::-1].reshape(B, T, H * 64)) for n in names}
    s3 = np.zeros((B, H, 64, 64), np.float32)
    y3 = orc.wkv7(s3, *[perm[n] for n in names], H, 0)
    assert np.array_equal(s3, s1[::-1, ::-1])
    assert np.array_equal(y3.reshape(B, T, H, 64), y1[::-1].reshape(B, T, H, 64)[:, :, ::-1])


# ------------------------------------------------------------------------------- LayerNorm family
def ln64(v, w, b, eps=1e-5):
    v = f64(v)
    mu = v.mean(axis=-1, keepdims=True)
    var = ((v - mu) ** 2).mean(axis=-1, keepdims=True)
    return (v - mu) / np.sqrt(var + eps) * f64(w) + f64(b)


def ref_inputs(rows, C, ox, orr, osh, ow, ob, scales):
    i = np.arange(rows * C)
    c = np.arange(C)
    x = pattern_value(i + ox, *scales[0]).reshape(rows, C).astype(np.float16)
    res = pattern_value(i + orr, *scales[1]).reshape(rows, C).astype(np.float16)
    sh = pattern_value(i + osh, *scales[2]).reshape(rows, C).astype(np.float16)
    w = pattern_value(c + ow, *scales[3]).astype(np.float16)
    b = pattern_value(c + ob, *scales[4]).astype(np.float16)
    return x, res, sh, w, b


def test_add_ln_cmix_mix_on_reference_test_inputs():
    """Shapes, input pattern and tolerance of test/cuda_non4096_kernels_test.cpp:283-339 (C = 2560, rows = 3)."""
    C, rows = 2560, 3
    x, res, sh, w, b = ref_inputs(rows, C, 0, 17, 33, 5, 9, [(0.2, -0.05), (0.15, 0.03), (0.25, -0.02), (0.08, 1.0), (0.03, 0.01)])
    mu = (0.5 + 0.4 * np.sin(np.arange(C, dtype=np.float32) * np.float32(0.007))).astype(np.float16)
    v = f64(x) + f64(res)
    yv = ln64(v, w, b)
    exp_mixed = yv + (f64(sh) - yv) * f64(mu)
    sh_io = sh.copy()
    xo, mixed = orc.add_layer_norm_cmix_mix(x, res, sh_io, w, b, mu)
    for got, want in ((xo, v), (mixed, exp_mixed), (sh_io, yv)):
        assert np.max(np.abs(f64(got) - want)) <= 2.5e-2      # the reference's bar
        assert np.max(np.abs(f64(got) - want)) <= 4e-3        # fp16 output rounding only


def test_add_ln_tmix_mix6_and_last_ln_on_reference_test_inputs():
    """test/cuda_non4096_kernels_test.cpp:341-489."""
    C, rows = 2560, 2
    x, res, sh, w, b = ref_inputs(rows, C, 101, 203, 307, 11, 19, [(0.18, -0.04), (0.12, 0.02), (0.22, 0.01), (0.06, 1.0), (0.02, 0.0)])
    c = np.arange(C)
    mus = [pattern_value(c + o, s, bb).astype(np.float16) for o, s, bb in
           ((23, 0.09, 0.5), (29, 0.07, 0.4), (31, 0.05, 0.3), (37, 0.08, 0.2), (41, 0.06, 0.1), (43, 0.04, 0.6))]
    v = f64(x) + f64(res)
    yv = ln64(v, w, b)
    sh_io = sh.copy()
    xo, outs = orc.add_layer_norm_tmix_mix6(x, res, sh_io, w, b, mus)
    assert np.max(np.abs(f64(xo) - v)) <= 2e-3
    for o, m in zip(outs, mus):
        assert np.max(np.abs(f64(o) - (yv + (f64(sh) - yv) * f64(m)))) <= 4e-3
    assert np.max(np.abs(f64(sh_io) - yv)) <= 4e-3

    B, T = 2, 3
    i = np.arange(B * T * C)
    x = pattern_value(i + 401, 0.17, -0.01).reshape(B * T, C).astype(np.float16)
    res = pattern_value(i + 503, 0.11, 0.05).reshape(B * T, C).astype(np.float16)
    w = pattern_value(c + 47, 0.05, 1.0).astype(np.float16)
    b = pattern_value(c + 59, 0.015, -0.02).astype(np.float16)
    y = orc.add_last_layer_norm(x, res, w, b, B, T)
    want = ln64((f64(x) + f64(res)).reshape(B, T, C)[:, -1], w, b)
    assert np.max(np.abs(f64(y) - want)) <= 4e-3
    # plain LN and add+LN
    assert np.max(np.abs(f64(orc.layer_norm(x, w, b)) - ln64(x, w, b))) <= 4e-3
    xo, y2 = orc.add_layer_norm(x, res, w, b)
    assert np.max(np.abs(f64(y2) - ln64(f64(x) + f64(res), w, b))) <= 4e-3


def test_token_shift_special_cases():
    rng = np.random.default_rng(6)
    B, T, C = 2, 4, 64
    x = rng.standard_normal((B * T, C)).astype(np.float16)
    sh = rng.standard_normal((B, C)).astype(np.float16)
    zero, one = np.zeros(C, np.float16), np.ones(C, np.float16)
    half = np.full(C, 0.5, np.float16)
    s = sh.copy()
    o0, o1, oh = orc.token_shift_mix(x, s, [zero, one, half], B, T)
    assert np.array_equal(o0, x)                                     # mu = 0: identity
    prev = np.concatenate([sh[:, None, :], x.reshape(B, T, C)[:, :-1]], axis=1).reshape(B * T, C)
    assert np.array_equal(o1, prev)                                  # mu = 1: the shifted sequence
    assert np.max(np.abs(f64(oh) - (f64(x) + f64(prev)) / 2)) <= 2e-3
    assert np.array_equal(s, x.reshape(B, T, C)[:, -1])              # shift <- last token


# ----------------------------------------------------------------------- gating / GroupNorm / LoRA
def test_kk_a_gate_closed_form_and_special_cases():
    rng = np.random.default_rng(7)
    rows, H = 3, 2
    C = H * 64
    k = rng.standard_normal((rows, C)).astype(np.float16)
    a12 = rng.standard_normal((rows, C)).astype(np.float16)
    k_k = (1 + 0.3 * rng.standard_normal(C)).astype(np.float16)
    a0 = (0.2 * rng.standard_normal(C)).astype(np.float16)
    k_a = (1 + 0.3 * rng.standard_normal(C)).astype(np.float16)
    nk, nkk, kka = orc.kk_a_gate(k, k_k, a0, a12, k_a, H)
    u = (f64(k) * f64(k_k)).reshape(rows, H, 64)
    kk = (u / np.linalg.norm(u, axis=-1, keepdims=True)).reshape(rows, C)
    a = 1 / (1 + np.exp(-(f64(a0) + f64(a12))))
    assert np.max(np.abs(f64(nk) - f64(k) * (1 + (a - 1) * f64(k_a)))) <= 4e-3
    assert np.max(np.abs(f64(nkk) + kk)) <= 1e-3
    assert np.max(np.abs(f64(kka) - kk * a)) <= 1e-3
    # -kk is a unit vector per head
    assert np.max(np.abs(np.linalg.norm(f64(nkk).reshape(rows, H, 64), axis=-1) - 1)) <= 2e-3
    # k_a = 0 leaves k untouched
    nk0, _, _ = orc.kk_a_gate(k, k_k, a0, a12, np.zeros(C, np.float16), H)
    assert np.array_equal(nk0, k)
    # an all-zero head does not divide by zero
    kz = k.copy()
    kz[:, :64] = 0
    _, nkkz, _ = orc.kk_a_gate(kz, k_k, a0, a12, k_a, H)
    assert np.all(np.isfinite(f64(nkkz))) and np.all(nkkz[:, :64] == 0)


def test_lnx_rkvres_xg_closed_form_and_special_cases():
    rng = np.random.default_rng(8)
    rows, H = 4, 3
    C = H * 64

    def rnd(*s, sc=1.0):
        return (rng.standard_normal(s) * sc).astype(np.float16)

    y, r, k, v, g = rnd(rows, C), rnd(rows, C), rnd(rows, C), rnd(rows, C), rnd(rows, C)
    r_k, lnw, lnb = rnd(C, sc=0.2), (1 + 0.1 * rng.standard_normal(C)).astype(np.float16), rnd(C, sc=0.1)
    out = orc.lnx_rkvres_xg(y, r, k, v, r_k, lnw, lnb, g, H)
    yh = f64(y).reshape(rows, H, 64)
    mu = yh.mean(-1, keepdims=True)
    var = ((yh - mu) ** 2).mean(-1, keepdims=True)
    gn = ((yh - mu) / np.sqrt(var + 64e-5)).reshape(rows, C) * f64(lnw) + f64(lnb)
    bonus = (f64(r) * f64(k) * f64(r_k)).reshape(rows, H, 64).sum(-1, keepdims=True) * f64(v).reshape(rows, H, 64)
    want = (gn + bonus.reshape(rows, C)) * f64(g)
    assert np.max(np.abs(f64(out) - want)) <= 2e-3 * np.max(np.abs(want))
    # g = 1, r_k = 0: a pure per-head GroupNorm
    out2 = orc.lnx_rkvres_xg(y, r, k, v, np.zeros(C, np.float16), lnw, lnb, np.ones((rows, C), np.float16), H)
    assert np.max(np.abs(f64(out2) - gn)) <= 4e-3


def test_vres_relu_addvec_lora():
    rng = np.random.default_rng(9)
    rows, C, R = 3, 128, 40
    v = rng.standard_normal((rows, C)).astype(np.float16)
    vf = rng.standard_normal((rows, C)).astype(np.float16)
    v12 = rng.standard_normal((rows, C)).astype(np.float32)
    v0 = rng.standard_normal(C).astype(np.float16)
    got = orc.vres_gate(v, vf, v0, v12)
    want = f64(v) + (f64(vf) - f64(v)) / (1 + np.exp(-(f64(v0) + f64(v12))))
    assert np.max(np.abs(f64(got) - want)) <= 2e-3
    assert np.array_equal(orc.vres_gate(v, vf, v0, np.full((rows, C), -1e4, np.float32)), v)       # gate -> 0
    assert np.array_equal(orc.vres_gate(v, vf, v0, np.full((rows, C), 1e4, np.float32)), vf)       # gate -> 1
    x = rng.standard_normal((rows, C)).astype(np.float16)
    assert np.array_equal(orc.relu_square(x), (np.maximum(x.astype(np.float32), 0) ** 2).astype(np.float16))
    assert np.array_equal(orc.add_vec(x, v0), (x.astype(np.float32) + v0.astype(np.float32)).astype(np.float16))
    w1 = (rng.standard_normal((R, C)) * 0.1).astype(np.float16)
    w2 = (rng.standard_normal((C, R)) * 0.1).astype(np.float16)
    for act, fn in ((0, lambda t: t), (1, np.tanh), (2, lambda t: 1 / (1 + np.exp(-t)))):
        hid = (f64(x) @ f64(w1).T).astype(np.float16)
        want = fn(f64(hid)) @ f64(w2).T
        got = orc.lora(x, w1, w2, act)
        assert np.max(np.abs(got - want)) <= 2e-3 * max(1.0, np.max(np.abs(want)))
    # a transposed W2 or W1 would not even have the right shape; a swapped activation is caught above


# -------------------------------------------------------------------------------- weight formats
def test_w8_format_properties():
    rng = np.random.default_rng(10)
    N, K = 33, 256
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    w[3] = 0
    q, s = orc.quantize_w8(w)
    assert q.dtype == np.int8 and q.min() >= -127 and q.max() <= 127
    assert np.all(q[3] == 0) and s[3] == 0
    amax = np.abs(w.astype(np.float32)).max(axis=1)
    assert np.array_equal(s, (amax / np.float32(127)).astype(np.float16))
    # the row maximum maps to +-127 (or 126 after fp16 rounding of the scale) and the error is half a step
    deq = orc.dequant_w8(q, s)
    step = s.astype(np.float32)[:, None]
    assert np.all(np.abs(deq.astype(np.float32) - w.astype(np.float32)) <= step * 0.5 + np.abs(w.astype(np.float32)) * 1e-3 + 1e-8)
    # idempotence: quantising the dequantised weights returns the same codes and scale
    q2, s2 = orc.quantize_w8(deq)
    assert np.array_equal(q2, q) and np.array_equal(s2, s)
    # dequant of every code == fp16(scale * code), all 256 codes
    codes = np.tile(np.arange(-128, 128, dtype=np.int8), (4, 1))
    sc = np.array([1e-3, 0.0137, 1.0, 3.3], np.float16)
    want = (sc.astype(np.float32)[:, None] * codes.astype(np.float32)).astype(np.float16)
    assert np.array_equal(orc.dequant_w8(codes, sc).view(np.uint16), want.view(np.uint16))


def test_w4_format_properties():
    rng = np.random.default_rng(11)
    N, K = 9, 384
    w = (rng.standard_normal((N, K)) * 0.02 + 0.005).astype(np.float16)
    w[2, :128] = 0
    w[4, 128:256] = np.abs(w[4, 128:256])      # one-sided group: zero stays representable
    q, s, z = orc.quantize_w4(w)
    assert q.shape == (N, K // 2) and s.shape == (N, 3) and z.shape == (N, 3)
    assert z.max() <= 15 and s[2, 0] == np.float16(1.0) and z[4, 1] == 0
    deq = orc.dequant_w4(q, s, z).astype(np.float32)
    step = np.repeat(s.astype(np.float32), 128, axis=1)
    assert np.all(np.abs(deq - w.astype(np.float32)) <= step * 1.01 + 1e-8)
    assert np.all(deq[2, :128] == 0)
    # nibble order: element 2i in the low nibble, 2i+1 in the high nibble; every code x zero point
    for zp in range(16):
        codes = np.roll(np.tile(np.arange(16, dtype=np.uint8), 8), zp)
        packed = (codes[0::2] | (codes[1::2] << 4)).astype(np.uint8).reshape(1, 64)
        sc = np.array([[0.37]], np.float16)
        got = orc.dequant_w4(packed, sc, np.array([[zp]], np.uint8))
        want = (sc.astype(np.float32) * (codes.astype(np.float32) - zp)).astype(np.float16)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    q2, s2, z2 = orc.quantize_w4(orc.dequant_w4(q, s, z))
    assert np.array_equal(orc.dequant_w4(q2, s2, z2), orc.dequant_w4(q, s, z))


@pytest.mark.parametrize("fmt", [0, 1, 2])
def test_gemv_matches_numpy_matmul(fmt):
    rng = np.random.default_rng(12 + fmt)
    M, N, K = 3, 40, 512
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    if fmt == 0:
        parts, wd = (w, None, None), f64(w)
    elif fmt == 1:
        q, s = orc.quantize_w8(w)
        parts, wd = (q, s, None), f64(s)[:, None] * f64(q)
    else:
        q, s, z = orc.quantize_w4(w)
        codes = np.stack([q & 15, q >> 4], axis=-1).reshape(N, K).astype(np.float64)
        parts, wd = (q, s, z), np.repeat(f64(s), 128, axis=1) * (codes - np.repeat(f64(z), 128, axis=1))
    want = f64(x) @ wd.T                      # x . W^T: a transposed operand changes the shape or the values
    got = orc.gemv(fmt, x, *parts)
    assert got.shape == (M, N)
    assert np.max(np.abs(f64(got) - want)) <= 1.5e-3 * np.max(np.abs(want))
    got32 = orc.gemv(fmt, x, *parts, f32_out=True)
    assert np.max(np.abs(got32 - want)) <= 1e-5 * np.max(np.abs(want)) + 1e-6


# --------------------------------------------------------------------------------------- sampler
def test_sampler_known_answers_of_reference_test():
    """test/sampler_test.cpp:30-76: argmax under top_p = 0; penalties stay 0; 2.0 then 6.0."""
    logits = np.array([0.25, 3.0, 1.0, -1.0], np.float32)
    pen = np.zeros(4, np.float32)
    assert orc.sample_greedy_penalty(logits, pen, 0.0, 0.0, 0.996) == 1
    assert np.all(pen == 0)
    kept, probs = orc.sample_filter(logits, None, 1.0, 0, 0.0)
    assert kept == 1 and np.argmax(probs) == 1 and probs[1] > 0
    logits = np.array([100.0, 0.0, 0.0, 0.0], np.float32)
    pen = np.zeros(4, np.float32)
    assert orc.sample_greedy_penalty(logits, pen, 2.0, 5.0, 0.5) == 0
    assert abs(pen[0] - 2.0) <= 1e-4 and pen[1] == 0
    assert orc.sample_greedy_penalty(logits, pen, 2.0, 5.0, 0.5) == 0
    assert abs(pen[0] - 6.0) <= 1e-4


def test_sampler_filter_topk_topp():
    rng = np.random.default_rng(13)
    V = 512
    logits = rng.standard_normal(V).astype(np.float32) * 3
    p = np.exp(f64(logits) - f64(logits).max())
    p /= p.sum()
    order = np.argsort(-p)
    kept, probs = orc.sample_filter(logits, None, 1.0, 10, 1.0)
    assert kept == 10 and set(np.nonzero(probs)[0]) == set(order[:10])
    assert np.max(np.abs(probs[order[:10]] - p[order[:10]])) <= 1e-6
    kept, probs = orc.sample_filter(logits, None, 1.0, 0, 0.5)
    csum = np.cumsum(p[order])
    n = int(np.searchsorted(csum, 0.5) + 1)            # smallest prefix reaching the mass
    assert set(np.nonzero(probs)[0]) == set(order[:n])
    assert abs(probs.sum() - 0.5) <= 1e-4               # the boundary entry is scaled to hit top_p exactly
    # temperature rescales the logits, penalties subtract
    kept, probs = orc.sample_filter(logits, None, 2.0, 0, 1.0)
    p2 = np.exp((f64(logits) - f64(logits).max()) / 2)
    assert kept == V and np.max(np.abs(probs - p2 / p2.sum())) <= 1e-6
    pen = np.zeros(V, np.float32)
    pen[order[0]] = 50.0
    kept, probs = orc.sample_filter(logits, pen, 1.0, 1, 1.0)
    assert np.argmax(probs) == order[1]


# ------------------------------------------------------------------------------------ layer graph
def small_dims():
    from rwkv_lightning_cuda_amd.model import ModelDims
    return ModelDims(L=3, C=128, H=2, F=256, V=512, Rw=16, Ra=16, Rg=24, Rv=8)


def cosine(a, b):
    a, b = f64(a).ravel(), f64(b).ravel()
    return float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b)))


def test_model_graph_matches_independent_numpy_restatement():
    from rwkv_lightning_cuda_amd.model import synth_weights
    dims = small_dims()
    weights = synth_weights(dims, seed=14)
    om = orc.Model(dims, weights, orc.FMT_F16)
    rng = np.random.default_rng(15)
    tokens = rng.integers(0, dims.V, (2, 7))
    ost = om.new_state(2)
    ol = om.forward(tokens, ost)
    nl, nst = np_model.forward(dims, weights, tokens)
    assert cosine(ol, nl) >= 0.9999
    assert np.max(np.abs(ol - nl)) <= 6e-3 * np.max(np.abs(nl))
    assert np.max(np.abs(ost[1] - nst["wkv"])) <= 5e-3 * np.max(np.abs(nst["wkv"]))
    assert np.max(np.abs(f64(ost[0]) - nst["shift"])) <= 5e-3 * np.max(np.abs(nst["shift"]))
    assert ost[2].tolist() == [7, 7]
    # a decode step continues from the carried state in both
    nxt = rng.integers(0, dims.V, (2, 1))
    ol = om.forward(nxt, ost)
    nl, nst = np_model.forward(dims, weights, nxt, nst)
    assert cosine(ol, nl) >= 0.9999
    assert ost[2].tolist() == [8, 8]


@pytest.mark.parametrize("fmt", [1, 2])
def test_quantised_model_graph_matches_numpy_on_dequantised_weights(fmt):
    from rwkv_lightning_cuda_amd.model import synth_weights
    dims = small_dims()
    weights = synth_weights(dims, seed=16)
    om = orc.Model(dims, weights, fmt)
    mats = {}
    for (layer, name), (q, s, z) in om.quant.items():
        if fmt == 1:
            mats[(layer, name)] = f64(s)[:, None] * f64(q)
        else:
            N, K2 = q.shape
            codes = np.stack([q & 15, q >> 4], axis=-1).reshape(N, K2 * 2).astype(np.float64)
            mats[(layer, name)] = np.repeat(f64(s), 128, axis=1) * (codes - np.repeat(f64(z), 128, axis=1))
    tokens = np.random.default_rng(17).integers(0, dims.V, (1, 5))
    ol = om.forward(tokens, om.new_state(1))
    nl, _ = np_model.forward(dims, weights, tokens, mats=mats)
    assert cosine(ol, nl) >= 0.9999


def test_chunked_prefill_equals_one_call_in_oracle():
    from rwkv_lightning_cuda_amd.model import synth_weights
    dims = small_dims()
    om = orc.Model(dims, synth_weights(dims, seed=18), orc.FMT_W8)
    tokens = np.random.default_rng(19).integers(0, dims.V, (2, 9))
    s1, s2 = om.new_state(2), om.new_state(2)
    l1 = om.forward(tokens, s1)
    om.forward(tokens[:, :4], s2)
    l2 = om.forward(tokens[:, 4:], s2)
    assert np.array_equal(l1, l2) and np.array_equal(s1[1], s2[1]) and np.array_equal(s1[0], s2[0])
    with pytest.raises(ValueError):
        om.forward(np.array([[dims.V]]), om.new_state(1))


def test_fp16_state_model_graph_branches_on_the_call_length():
    """orc_model_forward_f16state follows the reference's dispatch (src/rwkv7_fast_v4.cu:1266-1271): calls of up to 16
    tokens hand w12 and w0 to the recurrence apart (added unrounded there), longer calls round f16(w12 + w0) first.
    Which branch runs depends on the call's length only: splitting a call inside one branch changes no bit, crossing
    the boundary (17 tokens at once against 16 + 1) changes bits but stays within fp16 noise.  The graph around the
    recurrence is the fp32-state one (pinned against the numpy restatement above): both follow each other to fp16
    accuracy."""
    from rwkv_lightning_cuda_amd.model import synth_weights
    dims = small_dims()
    om = orc.Model(dims, synth_weights(dims, seed=23), orc.FMT_F16)
    rng = np.random.default_rng(24)

    def run(tokens, cuts, fp16=True):
        st = om.new_state(tokens.shape[0], wkv_fp16=fp16)
        lo = 0
        for hi in list(cuts) + [tokens.shape[1]]:
            logits = om.forward(tokens[:, lo:hi], st)
            lo = hi
        return logits, st

    def same_bits(a, b):
        return all(np.array_equal(x.view(np.uint16) if x.dtype == np.float16 else x,
                                  y.view(np.uint16) if y.dtype == np.float16 else y) for x, y in zip(a[1], b[1])) \
            and np.array_equal(a[0], b[0])

    t16 = rng.integers(0, dims.V, (2, 16))
    assert same_bits(run(t16, []), run(t16, [9]))             # both calls in the short branch
    t34 = rng.integers(0, dims.V, (2, 34))
    assert same_bits(run(t34, []), run(t34, [17]))            # both calls in the long branch
    t17 = rng.integers(0, dims.V, (2, 17))
    whole, split = run(t17, []), run(t17, [16])               # long branch against short + short
    assert not np.array_equal(whole[1][1].view(np.uint16), split[1][1].view(np.uint16))
    assert cosine(whole[0], split[0]) >= 0.9999
    scale = np.max(np.abs(f64(split[1][1])))
    assert np.max(np.abs(f64(whole[1][1]) - f64(split[1][1]))) <= 2e-2 * scale
    assert whole[1][2].tolist() == split[1][2].tolist() == [17, 17]
    # against the fp32-state graph on the same tokens
    ref = run(t17, [], fp16=False)
    assert cosine(whole[0], ref[0]) >= 0.999 and cosine(split[0], ref[0]) >= 0.999
    assert np.max(np.abs(f64(whole[1][1]) - f64(ref[1][1]))) <= 3e-2 * np.max(np.abs(ref[1][1]))


# ------------------------------------------------------------------------------- checkpoint tensors (bf16 -> fp16)
def _bf16_bits_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def test_bf16_to_f16_over_every_pattern_against_numpy():
    """Widening a bf16 pattern is exact by construction of the format; rounding the fp32 to fp16 is IEEE
    round-to-nearest-even, which numpy implements independently.  All 65536 patterns, plain and transposed."""
    bits = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    with np.errstate(over="ignore"):   # bf16 values beyond 65504 become infinity, as they should
        want = _bf16_bits_to_f32(bits).astype(np.float16)
    got = orc.bf16_to_f16(bits)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])
    got_t = orc.bf16_to_f16(bits[:37, :70].copy(), transpose=True)
    assert got_t.shape == (70, 37)
    keep = ~np.isnan(want[:37, :70].T)
    assert np.array_equal(got_t.view(np.uint16)[keep], want[:37, :70].T.view(np.uint16)[keep])
    # inside fp16's normal range a bf16 value has few enough fraction bits to be exact
    f = _bf16_bits_to_f32(bits)
    normal = np.isfinite(f) & (np.abs(f) >= 2.0 ** -14) & (np.abs(f) <= 65504.0)
    assert np.array_equal(got[normal].astype(np.float32), f[normal])


def test_emb_ln0_against_float64_and_invariants():
    rng = np.random.default_rng(20)
    V, C = 19, 192
    to_bf16 = lambda a: (a.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)  # truncation: still a bf16 value
    emb, w, b = to_bf16(rng.standard_normal((V, C))), to_bf16(1 + 0.1 * rng.standard_normal(C)), to_bf16(0.1 * rng.standard_normal(C))
    e64, w64, b64 = (f64(_bf16_bits_to_f32(a)) for a in (emb, w, b))
    mu = e64.mean(axis=1, keepdims=True)
    var = ((e64 - mu) ** 2).mean(axis=1, keepdims=True)
    want = (e64 - mu) / np.sqrt(var + 1e-5) * w64 + b64
    got = f64(orc.emb_ln0(emb, w, b))
    assert np.max(np.abs(got - want) / (np.abs(want) + 1e-2)) <= 1.5e-3           # fp16 rounding of the result
    # weight 1, bias 0: every row comes out with mean 0 and variance 1 (up to eps and fp16 rounding)
    one, zero = to_bf16(np.ones(C)), to_bf16(np.zeros(C))
    plain = f64(orc.emb_ln0(emb, one, zero))
    assert np.max(np.abs(plain.mean(axis=1))) <= 2e-3 and np.max(np.abs(plain.var(axis=1) - 1)) <= 5e-3
    # a constant row has no variance: the output is the bias
    const = to_bf16(np.full((2, C), 3.0))
    assert np.array_equal(orc.emb_ln0(const, w, b), np.broadcast_to(_bf16_bits_to_f32(b).astype(np.float16), (2, C)))


# ------------------------------------------------------------------------------- WKV7 with an fp16 state
from conftest import rel_err


def _f16(x):
    return np.asarray(x, np.float16)


def _bits(h):
    return int(np.asarray(h, np.float16).view(np.uint16))


def test_f64_to_f16_rounds_like_numpy_and_fma_rounds_once():
    """double -> fp16 against numpy's own correctly rounded conversion (normals, subnormals, ties, overflow), and
    the fp16 fma against exact rational arithmetic: a*b+c evaluated in Fractions and rounded once - including
    cases where rounding the product first would give another result."""
    from fractions import Fraction
    L = orc.lib()
    rng = np.random.default_rng(1)
    xs = np.concatenate([
        rng.standard_normal(20000) * np.exp(rng.uniform(-20, 12, 20000)),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001,
                  2.0 ** -14, 2.0 ** -14 - 2.0 ** -25, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1.0 + 2.0 ** -11 + 2.0 ** -40]),
    ])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_f64_to_f16(float(x)) for x in xs], np.uint16)
    assert np.array_equal(got, want)

    def exact_round(fr):
        # nearest fp16 to an exact rational (ties to even), by searching numpy's float16 neighbours
        approx = np.float16(float(fr))
        cands = {approx, np.nextafter(approx, np.float16(np.inf)), np.nextafter(approx, np.float16(-np.inf))}
        best = None
        for c in cands:
            if not np.isfinite(c):
                continue
            d = abs(Fraction(float(c)) - fr)
            key = (d, int(np.float16(c).view(np.uint16)) & 1)
            if best is None or key < best[0]:
                best = (key, c)
        return best[1]

    halfs = rng.standard_normal((3000, 3)).astype(np.float16)
    halfs[:200] = (rng.standard_normal((200, 3)) * 2.0 ** rng.integers(-12, 8, (200, 3))).astype(np.float16)
    # a case where f16(a*b) + c differs from fma(a, b, c): a*b = 1 + 2^-10 + 2^-20, c = -1
    extra = np.array([[1.0 + 2.0 ** -10, 1.0, -1.0], [1.0009765625, 1.0009765625, -1.0], [0.333251953125, 3.0, -1.0]], np.float16)
    for a, b, c in np.concatenate([halfs, extra]):
        fr = Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c))
        want_h = exact_round(fr)
        got_h = np.uint16(L.orc_f16_fma(_bits(a), _bits(b), _bits(c))).view(np.float16)
        assert got_h == want_h or (got_h == 0 and want_h == 0), (a, b, c, got_h, want_h)


def test_wkv16_dither_known_values_range_and_zero_mean():
    """rotator1(x) = 2^-41 * int32(2654435769 * x) (cuda/rwkv7_wkv_fp16_v2.cu:19-21,41-43): known values from integer
    arithmetic, |value| < 2^-10 (below fp16 resolution of d - 1 near -0), mean ~ 0 over consecutive phases; and what
    it is for: the fp16 decay delta averaged over consecutive phases approaches the unrounded d - 1 far closer
    than one fp16 rounding does."""
    L = orc.lib()
    assert L.orc_wkv16_rotator(0) == 0.0
    for x in (1, 2, 3, 1000, 123456789):
        prod = (2654435769 * x) & 0xffffffff
        sp = prod - (1 << 32) if prod >= (1 << 31) else prod
        assert L.orc_wkv16_rotator(x) == np.float32(4.547473508864641e-13) * np.float32(sp)
    vals = np.array([L.orc_wkv16_rotator(x) for x in range(1, 20001)])
    assert np.abs(vals).max() < 2.0 ** -10
    assert abs(vals.mean()) < 2e-6
    for w in (-3.0, -0.5, 1.0, 2.5):
        wh = np.float16(w)
        true = np.exp(-np.exp(-0.5) / (1.0 + np.exp(-np.float64(wh)))) - 1.0
        deltas = np.array([np.uint16(L.orc_wkv16_w_delta(_bits(wh), None, 0, ph)).view(np.float16)
                           for ph in range(4096)], np.float64)
        assert abs(deltas.mean() - true) < 2e-5                         # dithered: unbiased
        assert np.abs(deltas - true).max() <= 2.0 ** -10 + 2.0 ** -11   # each within dither + one rounding
    # w0 is added unrounded: f16(w + w0) would differ here
    w_raw, w0 = np.float16(0.7001953125), np.array([np.float16(0.00030517578125)], np.float16)
    d_sum = np.uint16(L.orc_wkv16_w_delta(_bits(w_raw), w0.ctypes.data_as(__import__("ctypes").c_void_p), 0, 0)).view(np.float16)
    true = np.exp(-np.exp(-0.5) / (1.0 + np.exp(-(np.float64(w_raw) + np.float64(w0[0]))))) - 1.0
    assert abs(np.float64(d_sum) - true) <= 2.0 ** -12


def test_wkv7_f16state_one_step_closed_forms_and_orientation():
    """From an empty state one token leaves S[i][j] = f16(k[j] * v[i]) (sa = 0, so the decay and b do not enter),
    and y[i] = the fp16 dot of that row with r in the reference's order; with r = e_j the output reads column j of
    the NEW state exactly.  A second token with a = b = 0 multiplies by the decay: S' = fma(S, wd, fma(k, v, S))."""
    rng = np.random.default_rng(3)
    H, C = 2, 128
    k = _f16(rng.standard_normal((1, 1, C)))
    v = _f16(rng.standard_normal((1, 1, C)))
    w = _f16(rng.uniform(-4, 2, (1, 1, C)))
    a = _f16(rng.standard_normal((1, 1, C)) * 0.1)
    b = _f16(rng.standard_normal((1, 1, C)) * 0.1)
    elapsed = np.array([5], np.int32)
    for j in (0, 1, 37, 63):
        r = np.zeros((1, 1, C), np.float16)
        r[0, 0, j] = 1.0
        r[0, 0, 64 + j] = 1.0
        S = np.zeros((1, H, 64, 64), np.float16)
        y = orc.wkv7_f16state(S, r, w, k, v, a, b, H, elapsed)
        for h in range(H):
            kv = (k[0, 0, h * 64:(h + 1) * 64].astype(np.float32)[None, :] * v[0, 0, h * 64:(h + 1) * 64].astype(np.float32)[:, None]).astype(np.float16)
            assert np.array_equal(S[0, h].view(np.uint16), kv.view(np.uint16))      # row i = value index, column j = key index
            assert np.array_equal(y[0, 0, h * 64:(h + 1) * 64].view(np.uint16), S[0, h][:, j].copy().view(np.uint16))
    # second token, a = b = 0: pure decay + outer product, every element one fp16 fma chain
    S = np.zeros((1, H, 64, 64), np.float16)
    zeros = np.zeros((1, 1, C), np.float16)
    r = _f16(rng.standard_normal((1, 1, C)))
    orc.wkv7_f16state(S, r, w, k, v, zeros, zeros, H, elapsed)
    S1 = S.copy()
    k2 = _f16(rng.standard_normal((1, 1, C)))
    v2 = _f16(rng.standard_normal((1, 1, C)))
    elapsed2 = np.array([6], np.int32)
    orc.wkv7_f16state(S, r, w, k2, v2, zeros, zeros, H, elapsed2)
    L = orc.lib()
    for h in range(H):
        for i in (0, 13, 63):
            for j in (0, 22, 63):
                c = h * 64 + j
                wd = np.uint16(L.orc_wkv16_w_delta(_bits(w[0, 0, c]), None, c, 6 + c)).view(np.float16)
                s = np.float64(S1[0, h, i, j])
                mid = np.float16(np.float64(k2[0, 0, c]) * np.float64(v2[0, 0, h * 64 + i]) + s)   # exact in float64
                want = np.float16(s * np.float64(wd) + np.float64(mid))
                assert S[0, h, i, j] == want, (h, i, j)


def test_wkv7_f16state_call_split_invariance_and_agreement_with_the_fp32_state():
    """Running T1 + T2 tokens in one call or in two (elapsed advanced by T1 in between) is bitwise the same; and on
    config-0 style inputs the fp16-state recurrence follows the fp32-state oracle (itself pinned by float64 brute
    force) to fp16 accuracy: outputs within 1.5e-2 of their scale over 48 tokens."""
    B, T, H = 2, 48, 3
    C = H * 64
    inp = wkv_inputs(B, T, H, seed=21, dtype=np.float16)
    names = ["r", "w_raw", "k", "v", "a", "b"]
    elapsed = np.array([7, 1000], np.int32)
    S = np.zeros((B, H, 64, 64), np.float16)
    y = orc.wkv7_f16state(S, *[inp[n] for n in names], H, elapsed)
    S2 = np.zeros((B, H, 64, 64), np.float16)
    T1 = 17
    ya = orc.wkv7_f16state(S2, *[np.ascontiguousarray(inp[n][:, :T1]) for n in names], H, elapsed)
    yb = orc.wkv7_f16state(S2, *[np.ascontiguousarray(inp[n][:, T1:]) for n in names], H, elapsed + T1)
    assert np.array_equal(S.view(np.uint16), S2.view(np.uint16))
    assert np.array_equal(np.concatenate([ya, yb], axis=1).view(np.uint16), y.view(np.uint16))
    S32 = np.zeros((B, H, 64, 64), np.float32)
    y32 = orc.wkv7(S32, *[inp[n] for n in names], H, 0)
    err = rel_err(y.astype(np.float32), y32.astype(np.float32))
    assert err <= 1.5e-2, err
    err = rel_err(S.astype(np.float32), S32)
    assert err <= 1.5e-2, err
