"""GPU parity tests of the individual C-ABI ops against the CPU oracle (same seeded inputs).

Bars: integer / byte work bit-exact; WKV fp32 state max-rel <= 1e-4; fp16 paths <= 2e-3.
"""
import numpy as np
import pytest

from conftest import elem_err, rel_err
from inputs import pattern_value, wkv_inputs

pytestmark = pytest.mark.gpu

WKV_TOL = 1e-4
F16_TOL = 2e-3


def dev(hip, a):
    return hip.DeviceArray.from_numpy(a)


# ---------------------------------------------------------------------------------------------- WKV7
@pytest.mark.parametrize("B,T,H", [(1, 64, 12), (2, 7, 3), (3, 1, 2)])
@pytest.mark.parametrize("mode", ["decay", "raw"])
def test_wkv7_f32_matches_oracle(gpu, orc, B, T, H, mode):
    hip = gpu
    C = H * 64
    inp = wkv_inputs(B, T, H, seed=100 + B + T)
    w = inp["decay"] if mode == "decay" else inp["w_raw"]
    w_mode = hip.W_DECAY if mode == "decay" else hip.W_RAW_LOGIT
    s_ref = np.zeros((B, H, 64, 64), np.float32)
    y_ref = orc.wkv7(s_ref, inp["r"], w, inp["k"], inp["v"], inp["a"], inp["b"], H, w_mode)
    state = hip.DeviceArray.zeros((B, H, 64, 64), np.float32)
    y = hip.DeviceArray((B, T, C), np.float32)
    hip.wkv7(B, T, C, H, w_mode, hip.IO_F32, state, dev(hip, inp["r"]), dev(hip, w), dev(hip, inp["k"]),
             dev(hip, inp["v"]), dev(hip, inp["a"]), dev(hip, inp["b"]), y)
    hip.device_sync()
    err = rel_err(y.numpy(), y_ref)
    assert err <= WKV_TOL
    err = elem_err(y.numpy(), y_ref)          # per element, not only against the largest output
    assert err <= WKV_TOL
    err = rel_err(state.numpy(), s_ref)
    assert err <= WKV_TOL
    err = elem_err(state.numpy(), s_ref)
    assert err <= WKV_TOL


def test_wkv7_drift_over_16384_tokens_against_the_fp32_oracle(gpu, orc):
    """The long-context configuration's length against the oracle (B = 1, H = 2, T = 16384, fp16 operands with the
    configuration-0 distributions, fp32 state): the state after 16384 sequential updates within 1e-4 of the
    oracle's, relative to its scale and per element, and the outputs of the last 128 tokens within the fp16 bar -
    the two sides differ only in summation order and in the last bits of the decay map, and the decay keeps
    those differences from accumulating."""
    hip = gpu
    B, T, H = 1, 16384, 2
    C = H * 64
    inp = wkv_inputs(B, T, H, seed=16384, dtype=np.float16)
    names = ["r", "w_raw", "k", "v", "a", "b"]
    s_ref = np.zeros((B, H, 64, 64), np.float32)
    y_ref = orc.wkv7(s_ref, *[inp[n] for n in names], H, 0)
    d = {n: dev(hip, inp[n]) for n in names}
    state = hip.DeviceArray.zeros((B, H, 64, 64), np.float32)
    y = hip.DeviceArray((B, T, C), np.float16)
    hip.wkv7(B, T, C, H, hip.W_RAW_LOGIT, hip.IO_F16, state, *[d[n] for n in names], y)
    hip.device_sync()
    s_rel = rel_err(state.numpy(), s_ref)
    s_elem = elem_err(state.numpy(), s_ref)
    y_last = rel_err(y.numpy()[:, -128:].astype(np.float32), y_ref[:, -128:].astype(np.float32))
    y_all = rel_err(y.numpy().astype(np.float32), y_ref.astype(np.float32))
    print("wkv7 T=16384: state max-rel %.2e, per element %.2e; y last 128 tokens %.2e, all tokens %.2e"
          % (s_rel, s_elem, y_last, y_all))
    assert s_rel <= WKV_TOL
    assert s_elem <= WKV_TOL
    assert y_last <= F16_TOL
    assert y_all <= F16_TOL


# (the last two: more than one and more than two heads per CU of a 256-CU chip, i.e. two and one lanes per state row)
@pytest.mark.parametrize("B,T,H,with_w0", [(1, 64, 12, False), (2, 7, 3, True), (3, 1, 2, True), (5, 33, 2, False),
                                          (5, 9, 64, True), (9, 6, 64, False)])
def test_wkv7_f16state_matches_oracle(gpu, orc, B, T, H, with_w0):
    """The fp16-state recurrence (the reference server's default mode) against the oracle's restatement of
    cuda/rwkv7_wkv_fp16_v2.cu: same fp16 fused multiply-adds in the same order, so outputs and state agree
    bit for bit except where the decay delta rounds differently (v_exp_f32 against the host's exp2f, one fp16 ulp
    of d - 1 in a few channels): at most 2e-3 of the tensors' scale, and most elements identical."""
    hip = gpu
    C = H * 64
    inp = wkv_inputs(B, T, H, seed=300 + B + T, dtype=np.float16)
    names = ["r", "w_raw", "k", "v", "a", "b"]
    rng = np.random.default_rng(B * T)
    w0 = (rng.standard_normal(C) * 0.3).astype(np.float16) if with_w0 else None
    elapsed = rng.integers(0, 5000, B).astype(np.int32)
    s0 = (rng.standard_normal((B, H, 64, 64)) * 0.2).astype(np.float16)     # a state that is already in use
    s_ref = s0.copy()
    y_ref = orc.wkv7_f16state(s_ref, *[inp[n] for n in names], H, elapsed, w0=w0)
    state = dev(hip, s0)
    y = hip.DeviceArray((B, T, C), np.float16)
    d = {n: dev(hip, inp[n]) for n in names}
    d_elapsed = dev(hip, elapsed)
    hip.wkv7_f16state(B, T, C, H, state, d["r"], d["w_raw"], d["k"], d["v"], d["a"], d["b"], y, d_elapsed,
                      w0=None if w0 is None else dev(hip, w0))
    hip.device_sync()
    got_y, got_s = y.numpy(), state.numpy()
    err = rel_err(got_y.astype(np.float32), y_ref.astype(np.float32))
    assert err <= F16_TOL
    err = rel_err(got_s.astype(np.float32), s_ref.astype(np.float32))
    assert err <= F16_TOL
    same = float(np.mean(got_s.view(np.uint16) == s_ref.view(np.uint16)))
    assert same >= 0.9, same
    assert d_elapsed.numpy().tolist() == elapsed.tolist()   # the kernel only reads elapsed


def test_wkv7_f16state_lanes_per_row_variants_are_bitwise(gpu):
    """The kernel gives a state row to one, two or four lanes by how many heads the call has (four while every head
    can have a CU to itself).  The sums run over the columns in the same order in all three, so a batch row gives
    the same bits whether it is computed alone, among five or among nine."""
    hip = gpu
    B, T, H = 9, 6, 64
    C = H * 64
    inp = wkv_inputs(B, T, H, seed=77, dtype=np.float16)
    names = ["r", "w_raw", "k", "v", "a", "b"]
    rng = np.random.default_rng(5)
    w0 = dev(hip, (rng.standard_normal(C) * 0.3).astype(np.float16))
    elapsed = rng.integers(0, 900, B).astype(np.int32)
    s0 = (rng.standard_normal((B, H, 64, 64)) * 0.2).astype(np.float16)

    def run(rows):
        n = len(rows)
        state = dev(hip, np.ascontiguousarray(s0[rows]))
        y = hip.DeviceArray((n, T, C), np.float16)
        d = [dev(hip, np.ascontiguousarray(inp[name][rows])) for name in names]
        hip.wkv7_f16state(n, T, C, H, state, *d, y, dev(hip, np.ascontiguousarray(elapsed[rows])), w0=w0)
        hip.device_sync()
        return y.numpy().view(np.uint16), state.numpy().view(np.uint16)

    y9, s9 = run(list(range(9)))        # 576 heads: one lane per row
    y5, s5 = run(list(range(5)))        # 320 heads: two lanes per row
    assert np.array_equal(y5, y9[:5]) and np.array_equal(s5, s9[:5])
    for b in (0, 8):                    # 64 heads: four lanes per row
        y1, s1 = run([b])
        assert np.array_equal(y1[0], y9[b]) and np.array_equal(s1[0], s9[b])


def test_wkv7_f16state_call_split_is_bitwise(gpu):
    hip = gpu
    B, T, H, T1 = 2, 29, 4, 11
    C = H * 64
    inp = wkv_inputs(B, T, H, seed=9, dtype=np.float16)
    names = ["r", "w_raw", "k", "v", "a", "b"]
    w0 = dev(hip, (np.random.default_rng(1).standard_normal(C) * 0.3).astype(np.float16))
    elapsed = np.array([3, 77], np.int32)
    state = hip.DeviceArray.zeros((B, H, 64, 64), np.float16)
    y = hip.DeviceArray((B, T, C), np.float16)
    d = {n: dev(hip, inp[n]) for n in names}
    hip.wkv7_f16state(B, T, C, H, state, *[d[n] for n in names], y, dev(hip, elapsed), w0=w0)
    hip.device_sync()
    state2 = hip.DeviceArray.zeros((B, H, 64, 64), np.float16)
    y2 = np.zeros((B, T, C), np.float16)
    for t0, tn in ((0, T1), (T1, T - T1)):
        part = {n: dev(hip, np.ascontiguousarray(inp[n][:, t0:t0 + tn])) for n in names}
        yp = hip.DeviceArray((B, tn, C), np.float16)
        hip.wkv7_f16state(B, tn, C, H, state2, *[part[n] for n in names], yp, dev(hip, elapsed + t0), w0=w0)
        hip.device_sync()
        y2[:, t0:t0 + tn] = yp.numpy()
    same = np.array_equal(state2.numpy().view(np.uint16), state.numpy().view(np.uint16))
    assert same
    same = np.array_equal(y2.view(np.uint16), y.numpy().view(np.uint16))
    assert same
    with pytest.raises(hip.RwkvHipError, match="H\\*64"):
        hip.wkv7_f16state(1, 1, 100, 1, state, d["r"], d["w_raw"], d["k"], d["v"], d["a"], d["b"], y, dev(hip, elapsed))


def test_wkv7_f16_io_and_t_split_bitwise(gpu, orc):
    hip = gpu
    B, T, H = 2, 40, 4
    C = H * 64
    inp = wkv_inputs(B, T, H, seed=7, dtype=np.float16)
    names = ["r", "w_raw", "k", "v", "a", "b"]
    s_ref = np.zeros((B, H, 64, 64), np.float32)
    y_ref = orc.wkv7(s_ref, *[inp[n] for n in names], H, 0)
    d = {n: dev(hip, inp[n]) for n in names}
    state = hip.DeviceArray.zeros((B, H, 64, 64), np.float32)
    y = hip.DeviceArray((B, T, C), np.float16)
    hip.wkv7(B, T, C, H, hip.W_RAW_LOGIT, hip.IO_F16, state, *[d[n] for n in names], y)
    hip.device_sync()
    err = rel_err(y.numpy().astype(np.float32), y_ref.astype(np.float32))
    assert err <= F16_TOL
    err = rel_err(state.numpy(), s_ref)
    assert err <= WKV_TOL

    # the same tokens in two calls (T1 + T2): bitwise identical state and outputs
    T1 = 13
    state2 = hip.DeviceArray.zeros((B, H, 64, 64), np.float32)
    y2 = np.zeros((B, T, C), np.float16)
    for t0, tn in ((0, T1), (T1, T - T1)):
        part = {n: dev(hip, np.ascontiguousarray(inp[n][:, t0:t0 + tn])) for n in names}
        yp = hip.DeviceArray((B, tn, C), np.float16)
        hip.wkv7(B, tn, C, H, hip.W_RAW_LOGIT, hip.IO_F16, state2, *[part[n] for n in names], yp)
        hip.device_sync()
        y2[:, t0:t0 + tn] = yp.numpy()
    same = np.array_equal(state2.numpy().view(np.uint32), state.numpy().view(np.uint32))
    assert same
    same = np.array_equal(y2.view(np.uint16), y.numpy().view(np.uint16))
    assert same


def test_wkv7_small_and_large_grids_agree_bitwise(gpu):
    """With up to 64 heads in flight a head runs as four blocks of 16 state rows each (sixteen wavefronts per head),
    up to 128 as two blocks of 32 rows (eight), above as one block (four); a state element sees the same
    arithmetic in each, so the same sequence gives bitwise the same outputs and state inside a batch of 1, of 40
    and of 70 (two heads each)."""
    hip = gpu
    T, H = 37, 2
    C = H * 64
    one = wkv_inputs(1, T, H, seed=5, dtype=np.float16)
    names = ["r", "w_raw", "k", "v", "a", "b"]
    outs = []
    for B in (1, 40, 70):
        rng = np.random.default_rng(B)
        full = {n: np.concatenate([one[n]] + [rng.permutation(one[n].reshape(-1)).reshape(one[n].shape)
                                              for _ in range(B - 1)], axis=0) for n in names}
        d = {n: dev(hip, full[n]) for n in names}
        state = hip.DeviceArray.zeros((B, H, 64, 64), np.float32)
        y = hip.DeviceArray((B, T, C), np.float16)
        hip.wkv7(B, T, C, H, hip.W_RAW_LOGIT, hip.IO_F16, state, *[d[n] for n in names], y)
        hip.device_sync()
        outs.append((y.numpy()[0].copy(), state.numpy()[0].copy()))
    for other in outs[1:]:
        same = np.array_equal(outs[0][0].view(np.uint16), other[0].view(np.uint16))
        assert same
        same = np.array_equal(outs[0][1].view(np.uint32), other[1].view(np.uint32))
        assert same


# ------------------------------------------------------------------------------- checkpoint tensors
def test_bf16_to_f16_every_pattern_and_transposes_bit_exact(gpu, orc):
    hip = gpu
    bits = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    want = orc.bf16_to_f16(bits)
    out = hip.DeviceArray((256, 256), np.float16)
    hip.bf16_to_f16(bits.size, dev(hip, bits), out)
    hip.device_sync()
    got = out.numpy()
    nan = np.isnan(want)
    same = np.array_equal(np.isnan(got), nan) and np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])
    assert same
    # a length that is not a multiple of the 8-element vectors
    tail = hip.DeviceArray((1003,), np.float16)
    hip.bf16_to_f16(1003, dev(hip, bits.reshape(-1)[:1003].copy()), tail)
    for rows, cols in [(37, 70), (64, 16), (1, 200), (96, 33)]:
        src = np.random.default_rng(rows).integers(0, 0x7f00, (rows, cols)).astype(np.uint16)   # finite values
        t = hip.DeviceArray((cols, rows), np.float16)
        hip.bf16_to_f16_transpose(rows, cols, dev(hip, src), t)
        hip.device_sync()
        same = np.array_equal(t.numpy().view(np.uint16), orc.bf16_to_f16(src, transpose=True).view(np.uint16))
        assert same
    hip.device_sync()
    same = np.array_equal(tail.numpy().view(np.uint16)[:1000], want.reshape(-1).view(np.uint16)[:1000])
    assert same
    with pytest.raises(hip.RwkvHipError):
        hip.bf16_to_f16_transpose(0, 4, dev(hip, bits), out)


def test_emb_ln0_matches_oracle(gpu, orc):
    hip = gpu
    rng = np.random.default_rng(21)
    V, C = 50, 768
    to_bf16 = lambda a: (a.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    emb = to_bf16(rng.standard_normal((V, C)))
    w, b = to_bf16(1 + 0.1 * rng.standard_normal(C)), to_bf16(0.1 * rng.standard_normal(C))
    out = hip.DeviceArray((V, C), np.float16)
    hip.emb_ln0_bf16_to_f16(V, C, dev(hip, emb), dev(hip, w), dev(hip, b), 1e-5, out)
    hip.device_sync()
    err = rel_err(out.numpy().astype(np.float32), orc.emb_ln0(emb, w, b).astype(np.float32))
    assert err <= F16_TOL


# ------------------------------------------------------------------------------------------- formats
def test_quantize_dequant_bit_exact(gpu, orc):
    hip = gpu
    rng = np.random.default_rng(3)
    N, K = 96, 1024
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    w[5] = 0  # an all-zero row exercises scale == 0
    w[6, :128] = 0
    wd = dev(hip, w)
    q_ref, s_ref = orc.quantize_w8(w)
    q = hip.DeviceArray((N, K), np.int8)
    s = hip.DeviceArray((N,), np.float16)
    hip.quantize_w8(N, K, wd, q, s)
    out = hip.DeviceArray((N, K), np.float16)
    hip.dequant_w8(N, K, q, s, out)
    hip.device_sync()
    same = np.array_equal(q.numpy(), q_ref)
    assert same
    same = np.array_equal(s.numpy().view(np.uint16), s_ref.view(np.uint16))
    assert same
    same = np.array_equal(out.numpy().view(np.uint16), orc.dequant_w8(q_ref, s_ref).view(np.uint16))
    assert same

    q4_ref, s4_ref, z4_ref = orc.quantize_w4(w)
    q4 = hip.DeviceArray((N, K // 2), np.uint8)
    s4 = hip.DeviceArray((N, K // 128), np.float16)
    z4 = hip.DeviceArray((N, K // 128), np.uint8)
    hip.quantize_w4(N, K, wd, q4, s4, z4)
    out4 = hip.DeviceArray((N, K), np.float16)
    hip.dequant_w4(N, K, q4, s4, z4, out4)
    hip.device_sync()
    same = np.array_equal(q4.numpy(), q4_ref)
    assert same
    same = np.array_equal(s4.numpy().view(np.uint16), s4_ref.view(np.uint16))
    assert same
    same = np.array_equal(z4.numpy(), z4_ref)
    assert same
    same = np.array_equal(out4.numpy().view(np.uint16), orc.dequant_w4(q4_ref, s4_ref, z4_ref).view(np.uint16))
    assert same


def test_dequant_all_codes_bit_exact(gpu, orc):
    """Every int8 code and every (int4 code, zero point) pair against a spread of scales."""
    hip = gpu
    scales = np.array([6.1e-5, 1e-3, 0.0137, 0.5, 1.0, 3.3, 6.0e-8, 100.0], np.float16)
    q = np.tile(np.arange(-128, 128, dtype=np.int8), (len(scales), 1))
    out = hip.DeviceArray(q.shape, np.float16)
    hip.dequant_w8(q.shape[0], q.shape[1], dev(hip, q), dev(hip, scales), out)
    hip.device_sync()
    same = np.array_equal(out.numpy().view(np.uint16), orc.dequant_w8(q, scales).view(np.uint16))
    assert same

    rows = []
    zps = []
    for zp in range(16):
        codes = np.tile(np.arange(16, dtype=np.uint8), 8)  # 128 codes: every nibble value at even and odd k
        codes = np.roll(codes, zp)  # shift parity so each code lands in both nibble positions
        rows.append((codes[0::2] | (codes[1::2] << 4)).astype(np.uint8))
        zps.append(zp)
    q4 = np.stack(rows)
    z4 = np.array(zps, np.uint8).reshape(16, 1)
    s4 = np.linspace(0.001, 2.0, 16).astype(np.float16).reshape(16, 1)
    out4 = hip.DeviceArray((16, 128), np.float16)
    hip.dequant_w4(16, 128, dev(hip, q4), dev(hip, s4), dev(hip, z4), out4)
    hip.device_sync()
    same = np.array_equal(out4.numpy().view(np.uint16), orc.dequant_w4(q4, s4, z4).view(np.uint16))
    assert same


# -------------------------------------------------------------------------------------------- linear
@pytest.mark.parametrize("fmt_name", ["f16", "w8", "w4"])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 11, 16, 37, 128, 200])
def test_linear_small_m(gpu, orc, fmt_name, M):
    hip = gpu
    rng = np.random.default_rng(11 + M)
    N, K = 264, 768
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    fmt = {"f16": hip.FMT_F16, "w8": hip.FMT_W8, "w4": hip.FMT_W4}[fmt_name]
    if fmt == hip.FMT_F16:
        parts = (w, None, None)
    elif fmt == hip.FMT_W8:
        parts = orc.quantize_w8(w) + (None,)
    else:
        parts = orc.quantize_w4(w)
    y_ref = orc.gemv(fmt, x, parts[0], parts[1], parts[2])
    y = hip.DeviceArray((M, N), np.float16)
    dparts = [dev(hip, p) if p is not None else None for p in parts]
    hip.linear(fmt, M, N, K, dev(hip, x), dparts[0], dparts[1], dparts[2], y)
    hip.device_sync()
    err = rel_err(y.numpy().astype(np.float32), y_ref.astype(np.float32))
    assert err <= F16_TOL


@pytest.mark.parametrize("fmt_name", ["w8", "f16"])
@pytest.mark.parametrize("M,N,K", [(5, 272, 4096), (8, 64, 2048), (11, 1040, 4096), (16, 16384, 4096), (13, 96, 1024),
                                   (7, 12304, 3072), (6, 4096, 4096), (37, 128, 1024), (8, 16400, 2048)])
def test_linear_few_rows_on_the_matrix_core(gpu, orc, fmt_name, M, N, K):
    """5..16 rows of int8 or fp16 weights whose K is a multiple of 1024 (<= 4096): the whole-rows-in-flight launch
    with the products on the matrix core (more rows: tiles of 16 of the same launch).  fp16 output, the relu^2
    epilogue and the fp32 output against the oracle; both block shapes (16 and 64 rows of W), both ways of staging
    x (up to 8 rows / more), N that is no multiple of the block's rows."""
    hip = gpu
    rng = np.random.default_rng(M * 131 + N + K)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    fmt = {"f16": hip.FMT_F16, "w8": hip.FMT_W8}[fmt_name]
    parts = (w, None, None) if fmt == hip.FMT_F16 else orc.quantize_w8(w) + (None,)
    hid = orc.gemv(fmt, x, parts[0], parts[1], parts[2])
    dparts = [dev(hip, p) if p is not None else None for p in parts]
    dx = dev(hip, x)
    y = hip.DeviceArray((M, N), np.float16)
    hip.linear(fmt, M, N, K, dx, dparts[0], dparts[1], dparts[2], y)
    act = hip.DeviceArray((M, N), np.float16)
    hip.linear(fmt, M, N, K, dx, dparts[0], dparts[1], dparts[2], act, epilogue=hip.EPI_RELU_SQUARE)
    y32 = hip.DeviceArray((M, N), np.float32)
    hip.linear(fmt, M, N, K, dx, dparts[0], dparts[1], dparts[2], y32, out_f32=1)
    hip.device_sync()
    assert rel_err(y.numpy().astype(np.float32), hid.astype(np.float32)) <= F16_TOL
    assert rel_err(act.numpy().astype(np.float32), orc.relu_square(hid).astype(np.float32)) <= 2 * F16_TOL
    got32 = y32.numpy()
    assert rel_err(got32, hid.astype(np.float32)) <= F16_TOL
    same = np.array_equal(got32, got32.astype(np.float16).astype(np.float32))
    assert same


@pytest.mark.parametrize("K", [1024, 2560, 4096, 16384])
def test_linear_w8_relu_square_and_f32_out(gpu, orc, K):
    hip = gpu
    rng = np.random.default_rng(K)
    N, M = 128, 2
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    q, s = orc.quantize_w8(w)
    hid = orc.gemv(orc.FMT_W8, x, q, s)
    act_ref = orc.relu_square(hid)
    y = hip.DeviceArray((M, N), np.float16)
    hip.linear(hip.FMT_W8, M, N, K, dev(hip, x), dev(hip, q), dev(hip, s), None, y, epilogue=hip.EPI_RELU_SQUARE)
    y32 = hip.DeviceArray((M, N), np.float32)
    hip.linear(hip.FMT_W8, M, N, K, dev(hip, x), dev(hip, q), dev(hip, s), None, y32, out_f32=1)
    hip.device_sync()
    err = rel_err(y.numpy().astype(np.float32), act_ref.astype(np.float32))
    assert err <= 2 * F16_TOL
    got32 = y32.numpy()
    err = rel_err(got32, hid.astype(np.float32))
    assert err <= F16_TOL
    # fp32 logits hold fp16-representable values
    same = np.array_equal(got32, got32.astype(np.float16).astype(np.float32))
    assert same


def test_linear_rejects_bad_shapes(gpu):
    hip = gpu
    x = hip.DeviceArray((1, 100), np.float16)
    with pytest.raises(hip.RwkvHipError):
        hip.linear(hip.FMT_W8, 1, 8, 100, x, x, x, None, x)  # K not a multiple of 16
    with pytest.raises(hip.RwkvHipError):
        hip.linear(hip.FMT_W8, 1, 8, 128, x, x, None, None, x)  # missing scale


# ----------------------------------------------------------------------------------------- fused ops
def _ref_test_inputs(rows, C, offs):
    i = np.arange(rows * C)
    x = pattern_value(i + offs[0], 0.2, -0.05).reshape(rows, C)
    res = pattern_value(i + offs[1], 0.15, 0.03).reshape(rows, C)
    sh = pattern_value(i + offs[2], 0.25, -0.02).reshape(rows, C)
    c = np.arange(C)
    w = pattern_value(c + 5, 0.08, 1.0)
    b = pattern_value(c + 9, 0.03, 0.01)
    return [t.astype(np.float16) for t in (x, res, sh, w, b)]


@pytest.mark.parametrize("C", [768, 2560, 4096])
def test_layer_norm_family(gpu, orc, C):
    hip = gpu
    rows = 3
    x, res, sh, w, b = _ref_test_inputs(rows, C, (0, 17, 33))
    y = hip.DeviceArray((rows, C), np.float16)
    hip.layer_norm(rows, C, dev(hip, x), dev(hip, w), dev(hip, b), y)
    xo = hip.DeviceArray((rows, C), np.float16)
    y2 = hip.DeviceArray((rows, C), np.float16)
    hip.add_layer_norm(rows, C, dev(hip, x), dev(hip, res), dev(hip, w), dev(hip, b), xo, y2)
    hip.device_sync()
    err = rel_err(y.numpy().astype(np.float32), orc.layer_norm(x, w, b).astype(np.float32))
    assert err <= F16_TOL
    xo_ref, y2_ref = orc.add_layer_norm(x, res, w, b)
    same = np.array_equal(xo.numpy().view(np.uint16), xo_ref.view(np.uint16))
    assert same
    err = rel_err(y2.numpy().astype(np.float32), y2_ref.astype(np.float32))
    assert err <= F16_TOL

    # add + last-token LN (B=1, T=rows)
    yl = hip.DeviceArray((1, C), np.float16)
    hip.add_last_layer_norm(1, rows, C, dev(hip, x), dev(hip, res), dev(hip, w), dev(hip, b), yl)
    hip.device_sync()
    err = rel_err(yl.numpy().astype(np.float32), orc.add_last_layer_norm(x, res, w, b, 1, rows).astype(np.float32))
    assert err <= F16_TOL

    # add + LN + cmix lerp + shift write (T == 1 fusion)
    c = np.arange(C)
    mu = (0.5 + 0.4 * np.sin(c.astype(np.float32) * 0.007)).astype(np.float16)
    sh_ref = sh.copy()
    xo_r, mixed_r = orc.add_layer_norm_cmix_mix(x, res, sh_ref, w, b, mu)
    shd = dev(hip, sh)
    xo3 = hip.DeviceArray((rows, C), np.float16)
    mixed = hip.DeviceArray((rows, C), np.float16)
    hip.add_layer_norm_cmix_mix(rows, C, dev(hip, x), dev(hip, res), shd, dev(hip, w), dev(hip, b), dev(hip, mu), xo3, mixed)
    hip.device_sync()
    same = np.array_equal(xo3.numpy().view(np.uint16), xo_r.view(np.uint16))
    assert same
    err = rel_err(mixed.numpy().astype(np.float32), mixed_r.astype(np.float32))
    assert err <= F16_TOL
    err = rel_err(shd.numpy().astype(np.float32), sh_ref.astype(np.float32))
    assert err <= F16_TOL

    # add + LN + six lerps
    mus = [pattern_value(c + o, s, bb).astype(np.float16) for o, s, bb in
           ((23, 0.09, 0.5), (29, 0.07, 0.4), (31, 0.05, 0.3), (37, 0.08, 0.2), (41, 0.06, 0.1), (43, 0.04, 0.6))]
    sh_ref = sh.copy()
    xo_r, outs_r = orc.add_layer_norm_tmix_mix6(x, res, sh_ref, w, b, mus)
    shd = dev(hip, sh)
    outs = [hip.DeviceArray((rows, C), np.float16) for _ in range(6)]
    hip.add_layer_norm_tmix_mix6(rows, C, dev(hip, x), dev(hip, res), shd, dev(hip, w), dev(hip, b),
                                 [dev(hip, m) for m in mus], xo3, outs)
    hip.device_sync()
    for o, o_r in zip(outs, outs_r):
        err = rel_err(o.numpy().astype(np.float32), o_r.astype(np.float32))
        assert err <= F16_TOL
    err = rel_err(shd.numpy().astype(np.float32), sh_ref.astype(np.float32))
    assert err <= F16_TOL


@pytest.mark.parametrize("B,T", [(1, 1), (2, 5), (3, 1)])
def test_token_shift_mix(gpu, orc, B, T):
    hip = gpu
    C = 256
    rng = np.random.default_rng(5)
    x = rng.standard_normal((B * T, C)).astype(np.float16)
    sh = rng.standard_normal((B, C)).astype(np.float16)
    mus = [rng.uniform(0, 1, C).astype(np.float16) for _ in range(6)]
    sh_ref = sh.copy()
    outs_r = orc.token_shift_mix(x, sh_ref, mus, B, T)
    shd = dev(hip, sh)
    outs = [hip.DeviceArray((B * T, C), np.float16) for _ in range(6)]
    hip.token_shift_mix(B, T, C, dev(hip, x), shd, [dev(hip, m) for m in mus], outs)
    hip.device_sync()
    for o, o_r in zip(outs, outs_r):
        err = rel_err(o.numpy().astype(np.float32), o_r.astype(np.float32))
        assert err <= F16_TOL
    same = np.array_equal(shd.numpy().view(np.uint16), sh_ref.view(np.uint16))
    assert same


def test_kk_gate_groupnorm_lora(gpu, orc):
    hip = gpu
    rng = np.random.default_rng(9)
    rows, H = 5, 6
    C = H * 64

    def rnd(*shape, s=1.0):
        return (rng.standard_normal(shape) * s).astype(np.float16)

    k, a12 = rnd(rows, C), rnd(rows, C, s=0.5)
    k_k, a0, k_a = rnd(C, s=0.3) + np.float16(1), rnd(C, s=0.2), rnd(C, s=0.3) + np.float16(1)
    nk_r, nkk_r, kka_r = orc.kk_a_gate(k, k_k, a0, a12, k_a, H)
    nk, nkk, kka = (hip.DeviceArray((rows, C), np.float16) for _ in range(3))
    hip.kk_a_gate(rows, C, H, dev(hip, k), dev(hip, k_k), dev(hip, a0), dev(hip, a12), dev(hip, k_a), nk, nkk, kka)
    hip.device_sync()
    for got, ref in ((nk, nk_r), (nkk, nkk_r), (kka, kka_r)):
        err = rel_err(got.numpy().astype(np.float32), ref.astype(np.float32))
        assert err <= F16_TOL

    y, r, v, g = rnd(rows, C), rnd(rows, C), rnd(rows, C), rnd(rows, C)
    r_k, lnw, lnb = rnd(C, s=0.1), rnd(C, s=0.1) + np.float16(1), rnd(C, s=0.1)
    out_r = orc.lnx_rkvres_xg(y, r, k, v, r_k, lnw, lnb, g, H)
    out = hip.DeviceArray((rows, C), np.float16)
    hip.lnx_rkvres_xg(rows, C, H, dev(hip, y), dev(hip, r), dev(hip, k), dev(hip, v), dev(hip, r_k), dev(hip, lnw),
                      dev(hip, lnb), dev(hip, g), out)
    hip.device_sync()
    err = rel_err(out.numpy().astype(np.float32), out_r.astype(np.float32))
    assert err <= F16_TOL

    # LoRA pair, each activation, and the v-residual epilogue
    for R, act in ((64, hip.ACT_TANH), (32, hip.ACT_NONE), (136, hip.ACT_SIGMOID)):
        x = rnd(rows, C)
        w1, w2 = rnd(R, C, s=0.05), rnd(C, R, s=0.05)
        o32 = orc.lora(x, w1, w2, act)
        h = hip.DeviceArray((rows, R), np.float16)
        hip.lora_in(rows, C, R, dev(hip, x), dev(hip, w1), h)
        o = hip.DeviceArray((rows, C), np.float16)
        hip.lora_out(rows, C, R, act, h, dev(hip, w2), o)
        hip.device_sync()
        err = rel_err(o.numpy().astype(np.float32), o32)
        assert err <= F16_TOL
        if act == hip.ACT_NONE:
            v_first, v0 = rnd(rows, C), rnd(C, s=0.3)
            ref = orc.vres_gate(v, v_first, v0, o32)
            og = hip.DeviceArray((rows, C), np.float16)
            hip.lora_out(rows, C, R, act, h, dev(hip, w2), og, bias=dev(hip, v0), vres=1, v=dev(hip, v), v_first=dev(hip, v_first))
            hip.device_sync()
            err = rel_err(og.numpy().astype(np.float32), ref.astype(np.float32))
            assert err <= F16_TOL


def test_lora_out_blocks_walk_several_row_tiles(gpu, orc):
    """Beyond 256 rows a block keeps its weights and walks several 32-row tiles; the last tile here is partial.  The
    v-residual epilogue is checked on the same rows."""
    hip = gpu
    rng = np.random.default_rng(77)
    rows, C, R = 300 + 13, 256, 40
    h = rng.standard_normal((rows, R)).astype(np.float16)
    w2 = (rng.standard_normal((C, R)) * 0.1).astype(np.float16)
    v, v_first = (rng.standard_normal((rows, C)).astype(np.float16) for _ in range(2))
    v0 = (rng.standard_normal(C) * 0.3).astype(np.float16)
    o32 = (h.astype(np.float64) @ w2.astype(np.float64).T).astype(np.float32)
    o = hip.DeviceArray((rows, C), np.float16)
    hip.lora_out(rows, C, R, hip.ACT_NONE, dev(hip, h), dev(hip, w2), o)
    og = hip.DeviceArray((rows, C), np.float16)
    hip.lora_out(rows, C, R, hip.ACT_NONE, dev(hip, h), dev(hip, w2), og, bias=dev(hip, v0), vres=1, v=dev(hip, v),
                 v_first=dev(hip, v_first))
    hip.device_sync()
    assert rel_err(o.numpy().astype(np.float32), o32) <= F16_TOL
    ref = orc.vres_gate(v, v_first, v0, o32)
    assert rel_err(og.numpy().astype(np.float32), ref.astype(np.float32)) <= F16_TOL


@pytest.mark.parametrize("rows,C,R", [(1, 96, 8), (33, 256, 136), (70, 768, 480), (128, 4096, 512), (64, 4096, 96),
                                      (700, 384, 136)])
def test_lora_out_keeps_the_activated_hidden_in_fp32(gpu, rows, C, R):
    """The rank-out product feeds act(h) to the matrix core as an fp16 hi + lo pair.  Against a float64 dot over
    the float32 activation, the fp16 result is the correctly rounded one except at near-ties; with the lo term
    dropped a third of the outputs would move by an ulp."""
    hip = gpu
    rng = np.random.default_rng(rows * 1000 + R)
    h = (rng.standard_normal((rows, R)) * 1.5).astype(np.float16)
    w2 = (rng.standard_normal((C, R)) * 0.1).astype(np.float16)
    for act in (hip.ACT_TANH, hip.ACT_SIGMOID, hip.ACT_NONE):
        hf = h.astype(np.float32)
        if act == hip.ACT_TANH:
            hf = np.tanh(hf)
        elif act == hip.ACT_SIGMOID:
            hf = (1.0 / (1.0 + np.exp(-hf))).astype(np.float32)
        exact = hf.astype(np.float64) @ w2.astype(np.float64).T
        want = exact.astype(np.float16)
        o = hip.DeviceArray((rows, C), np.float16)
        hip.lora_out(rows, C, R, act, dev(hip, h), dev(hip, w2), o)
        hip.device_sync()
        got = o.numpy()
        # half an fp16 ulp of rounding + the fp32 accumulation error (a few 1e-8 of the sum of magnitudes)
        mags = np.abs(hf).astype(np.float64) @ np.abs(w2).astype(np.float64).T
        bound = 0.5 * np.spacing(np.abs(want)).astype(np.float64) + 1e-6 * mags
        assert np.all(np.abs(got.astype(np.float64) - exact) <= bound)
        off = np.mean(got.view(np.uint16) != want.view(np.uint16))
        assert off <= 0.01, "act %d: %.4f of the outputs are not the correctly rounded value" % (act, off)


def _sparse_w4_pack(hip, orc, w):
    """Quantise to int4, pack for the row-skipping product and check the packed bytes: codes [F,C/2] (even c in the
    low nibble), then scales [F/128,C] fp16, then zero points [F/128,C]."""
    C, F = w.shape
    q, s, z = orc.quantize_w4(w)
    wt = hip.DeviceArray((hip.cmix_sparse_packed_bytes(hip.FMT_W4, C, F),), np.uint8)
    hip.cmix_sparse_pack_w4(C, F, dev(hip, q), dev(hip, s), dev(hip, z), wt)
    hip.device_sync()
    nib = np.empty((C, F), np.uint8)
    nib[:, 0::2] = q & 15
    nib[:, 1::2] = q >> 4
    nt = np.ascontiguousarray(nib.T)
    codes_t = (nt[:, 0::2] | (nt[:, 1::2] << 4)).astype(np.uint8)
    want = np.concatenate([codes_t.ravel(), np.ascontiguousarray(s.reshape(C, F // 128).T).view(np.uint8).ravel(),
                           np.ascontiguousarray(z.reshape(C, F // 128).T).ravel()])
    same = np.array_equal(wt.numpy(), want)
    assert same
    return q, s, z, wt


@pytest.mark.parametrize("fmt_name", ["w8", "f16", "w4"])
@pytest.mark.parametrize("C,F", [(768, 3072), (2560, 10240), (4096, 16384)])
def test_cmix_sparse_down_matches_dense_product_and_oracle(gpu, orc, C, F, fmt_name):
    """ffn.value of one token over the transposed copy, skipping rows with a zero activation: against the
    oracle's dense product of the same weights and against the dense GEMV on the GPU; edge patterns of the
    activation (none, one, all non-zero; a wavefront's 32 rows all zero); repeat calls bitwise equal."""
    hip = gpu
    rng = np.random.default_rng(C + F)
    w = (rng.standard_normal((C, F)) * 0.02).astype(np.float16)
    z, zd = None, None
    if fmt_name == "w4":
        fmt = hip.FMT_W4
        q, s, z, wt = _sparse_w4_pack(hip, orc, w)
        qd, sd, zd = dev(hip, q), dev(hip, s), dev(hip, z)
    else:
        if fmt_name == "w8":
            fmt = hip.FMT_W8
            q, s = orc.quantize_w8(w)
            qd, sd = dev(hip, q), dev(hip, s)
            wt = hip.DeviceArray((F, C), np.uint8)
            want_t = (q.T.astype(np.int16) + 128).astype(np.uint8)
        else:
            fmt = hip.FMT_F16
            q, s = w, None
            qd, sd = dev(hip, w), None
            wt = hip.DeviceArray((F, C), np.float16)
            want_t = np.ascontiguousarray(w.T)
        hip.cmix_sparse_pack(fmt, C, F, qd, wt)
        hip.device_sync()
        same = np.array_equal(wt.numpy().view(np.uint8), want_t.view(np.uint8))
        assert same
    ws = hip.DeviceArray.zeros((hip.cmix_sparse_workspace(C, F),), np.uint8)

    base = rng.standard_normal(F).astype(np.float16)
    patterns = {
        "half": base,
        "none": -np.abs(base),
        "one": np.where(np.arange(F) == F // 3, np.float16(1.5), np.float16(-1.0)).astype(np.float16),
        "all": (np.abs(base) + np.float16(0.01)).astype(np.float16),
        "gaps": np.where((np.arange(F) // 32) % 3 == 0, -np.abs(base), base).astype(np.float16),
        "minus_zero": np.where(np.arange(F) % 2 == 0, np.float16(-0.0), base).astype(np.float16),
    }
    for name, pre in patterns.items():
        act = orc.relu_square(pre.reshape(1, F))
        want = orc.gemv(fmt, act, q, s, z)
        out = hip.DeviceArray((1, C), np.float16)
        hip.cmix_sparse_down_relu_one(fmt, C, F, dev(hip, pre), wt, sd, ws, out)
        hip.device_sync()
        got = out.numpy()
        if name == "none":
            assert not got.any()
        else:
            err = rel_err(got.astype(np.float32), want.astype(np.float32))
            assert err <= F16_TOL, name
        dense = hip.DeviceArray((1, C), np.float16)
        hip.linear(fmt, 1, C, F, dev(hip, act), qd, sd, zd, dense)
        out2 = hip.DeviceArray((1, C), np.float16)
        hip.cmix_sparse_down_relu_one(fmt, C, F, dev(hip, pre), wt, sd, ws, out2)
        hip.device_sync()
        # two fp32 sums of the same exact products in different orders: at most an fp16 ulp apart at the output scale
        d = np.abs(got.astype(np.float32) - dense.numpy().astype(np.float32)).max()
        assert d <= 1e-3 * max(1e-6, np.abs(want.astype(np.float32)).max()), name
        same = np.array_equal(out2.numpy().view(np.uint16), got.view(np.uint16))
        assert same, name


@pytest.mark.parametrize("fmt_name", ["w8", "f16", "w4"])
def test_cmix_sparse_down_rows_matches_the_one_row_product(gpu, orc, fmt_name):
    """Several tokens per call: each row of the output is bitwise what the one-row call gives for that token, and
    matches the oracle's dense product."""
    hip = gpu
    C, F, rows = 768, 3072, 5
    rng = np.random.default_rng(17)
    w = (rng.standard_normal((C, F)) * 0.02).astype(np.float16)
    z = None
    if fmt_name == "w4":
        fmt = hip.FMT_W4
        q, s, z, wt = _sparse_w4_pack(hip, orc, w)
        sd = None
    elif fmt_name == "w8":
        fmt = hip.FMT_W8
        q, s = orc.quantize_w8(w)
        sd = dev(hip, s)
        wt = hip.DeviceArray((F, C), np.uint8)
    else:
        fmt = hip.FMT_F16
        q, s, sd = w, None, None
        wt = hip.DeviceArray((F, C), np.float16)
    if fmt_name != "w4":
        hip.cmix_sparse_pack(fmt, C, F, dev(hip, q), wt)
    pre = rng.standard_normal((rows, F)).astype(np.float16)
    pre[2] = -np.abs(pre[2])  # a token with no active row at all
    ws = hip.DeviceArray.zeros((hip.cmix_sparse_workspace(C, F, rows),), np.uint8)
    out = hip.DeviceArray((rows, C), np.float16)
    hip.cmix_sparse_down_relu_rows(fmt, rows, C, F, dev(hip, pre), wt, sd, ws, out)
    hip.device_sync()
    got = out.numpy()
    want = orc.gemv(fmt, orc.relu_square(pre), q, s, z)
    err = rel_err(got.astype(np.float32), want.astype(np.float32))
    assert err <= F16_TOL
    assert not got[2].any()
    ws1 = hip.DeviceArray.zeros((hip.cmix_sparse_workspace(C, F),), np.uint8)
    for r in range(rows):
        one = hip.DeviceArray((1, C), np.float16)
        hip.cmix_sparse_down_relu_one(fmt, C, F, dev(hip, pre[r]), wt, sd, ws1, one)
        hip.device_sync()
        same = np.array_equal(one.numpy().view(np.uint16)[0], got.view(np.uint16)[r])
        assert same, r
    with pytest.raises(hip.RwkvHipError):
        hip.cmix_sparse_down_relu_rows(fmt, 13, C, F, dev(hip, pre), wt, sd, ws, out)  # more rows than the path takes
    with pytest.raises(hip.RwkvHipError):
        hip.cmix_sparse_down_relu_rows(fmt, rows, C, F, dev(hip, pre), wt, sd, ws1, out)  # workspace of one row


@pytest.mark.parametrize("fmt_name", ["w8", "f16", "w4"])
@pytest.mark.parametrize("C,F,rows", [(768, 3072, 2), (2048, 8192, 3), (4096, 16384, 4)])
def test_cmix_sparse_down_shared_walk_matches_oracle_and_per_token_walks(gpu, orc, fmt_name, C, F, rows):
    """2..4 tokens in one walk over the union of their non-zero rows, at the three benchmark widths: against the
    oracle's dense product (the bar of the fp16 paths) and against one walk per token (equal up to the last bits of
    the fp32 sums: within an fp16 ulp of the output's scale after rounding, mostly identical); a token without any active row comes
    out as zeros; two calls give the same bits."""
    hip = gpu
    rng = np.random.default_rng(C + rows)
    w = (rng.standard_normal((C, F)) * 0.02).astype(np.float16)
    z = None
    if fmt_name == "w4":
        fmt = hip.FMT_W4
        q, s, z, wt = _sparse_w4_pack(hip, orc, w)
        sd = None
    elif fmt_name == "w8":
        fmt = hip.FMT_W8
        q, s = orc.quantize_w8(w)
        sd = dev(hip, s)
        wt = hip.DeviceArray((F, C), np.uint8)
    else:
        fmt = hip.FMT_F16
        q, s, sd = w, None, None
        wt = hip.DeviceArray((F, C), np.float16)
    if fmt_name != "w4":
        hip.cmix_sparse_pack(fmt, C, F, dev(hip, q), wt)
    pre = rng.standard_normal((rows, F)).astype(np.float16)
    pre[1, : F // 2] = -np.abs(pre[1, : F // 2])   # the tokens' masks differ in whole wavefront ranges too
    if rows >= 3:
        pre[2] = -np.abs(pre[2])                   # a token with no active row at all
    ws = hip.DeviceArray.zeros((hip.cmix_sparse_workspace(C, F, rows),), np.uint8)
    out = hip.DeviceArray((rows, C), np.float16)
    hip.cmix_sparse_down_relu_rows_shared(fmt, rows, C, F, dev(hip, pre), wt, sd, ws, out)
    hip.device_sync()
    got = out.numpy()
    want = orc.gemv(fmt, orc.relu_square(pre), q, s, z)
    assert rel_err(got.astype(np.float32), want.astype(np.float32)) <= F16_TOL
    if rows >= 3:
        assert not got[2].any()
    per_token = hip.DeviceArray((rows, C), np.float16)
    hip.cmix_sparse_down_relu_rows(fmt, rows, C, F, dev(hip, pre), wt, sd, ws, per_token)
    hip.device_sync()
    ref = per_token.numpy()
    same = float(np.mean(ref.view(np.uint16) == got.view(np.uint16)))
    assert same >= 0.9, same
    # (a sum that cancels to almost nothing can move by more than its own ulp: the bar is an ulp of the row's scale)
    assert rel_err(got.astype(np.float32), ref.astype(np.float32)) <= 2.0 ** -10
    again = hip.DeviceArray((rows, C), np.float16)
    hip.cmix_sparse_down_relu_rows_shared(fmt, rows, C, F, dev(hip, pre), wt, sd, ws, again)
    hip.device_sync()
    assert np.array_equal(again.numpy().view(np.uint16), got.view(np.uint16))
    with pytest.raises(hip.RwkvHipError):
        hip.cmix_sparse_down_relu_rows_shared(fmt, 5, C, F, dev(hip, pre), wt, sd, ws, out)   # more tokens than one walk takes


def test_cmix_sparse_rejects_bad_arguments(gpu):
    hip = gpu
    with pytest.raises(hip.RwkvHipError):
        hip.cmix_sparse_workspace(768, 3000)  # F not a multiple of 256
    with pytest.raises(hip.RwkvHipError):
        hip.cmix_sparse_workspace(100, 1024)  # C not a multiple of 16
    buf = hip.DeviceArray.zeros((1024,), np.uint8)
    with pytest.raises(hip.RwkvHipError):
        hip.cmix_sparse_down_relu_one(hip.FMT_W8, 256, 1024, buf, buf, buf, buf, buf)  # workspace too small
    with pytest.raises(hip.RwkvHipError):
        hip.cmix_sparse_pack(hip.FMT_W4, 256, 1024, buf, hip.DeviceArray.zeros((1024,), np.uint8))  # no int4 variant


def test_small_elementwise(gpu, orc):
    hip = gpu
    rng = np.random.default_rng(2)
    x = rng.standard_normal((4, 512)).astype(np.float16)
    vec = rng.standard_normal(512).astype(np.float16)
    out = hip.DeviceArray(x.shape, np.float16)
    hip.relu_square(x.size, dev(hip, x), out)
    hip.device_sync()
    same = np.array_equal(out.numpy().view(np.uint16), orc.relu_square(x).view(np.uint16))
    assert same
    hip.add_vec(4, 512, dev(hip, x), dev(hip, vec), out)
    hip.device_sync()
    same = np.array_equal(out.numpy().view(np.uint16), orc.add_vec(x, vec).view(np.uint16))
    assert same
    o32 = hip.DeviceArray(x.shape, np.float32)
    hip.f16_to_f32(x.size, dev(hip, x), o32)
    e = dev(hip, np.array([3, 9], np.int32))
    hip.advance_i32(2, 128, e)
    hip.device_sync()
    same = np.array_equal(o32.numpy(), x.astype(np.float32))
    assert same
    assert e.numpy().tolist() == [131, 137]


# ----------------------------------------------------------------------------- packed-weight MFMA GEMM
def _quant_parts(orc, hip, fmt, w):
    if fmt == hip.FMT_F16:
        return (w, None, None)
    if fmt == hip.FMT_W8:
        return orc.quantize_w8(w) + (None,)
    return orc.quantize_w4(w)


@pytest.mark.parametrize("fmt_name", ["f16", "w8", "w4"])
@pytest.mark.parametrize("M,N,K", [(16, 128, 512), (33, 96, 256), (64, 256, 1024), (128, 160, 2048), (200, 64, 768),
                                   (17, 4096, 256), (64, 128, 2560), (600, 256, 1024), (1030, 96, 512),
                                   (20, 96, 1024), (32, 4160, 512), (5, 64, 2048),
                                   (1030, 3872, 512), (3000, 2336, 256)])
def test_linear_packed_matches_oracle(gpu, orc, fmt_name, M, N, K):
    """Every tile variant (32-, 64- and 128-row tiles; one, two and four wavefront groups; 64-, 128- and 256-column
    blocks - the last two shapes take the 128 x 256 tile for int8 and fp16 weights, once split and once not;
    several row tiles), with and without K splits, chunk counts that are not a power of two, ragged M and column
    counts that are not a multiple of the column block."""
    hip = gpu
    if fmt_name == "w4" and K % 128:
        pytest.skip("W4 groups are 128 wide")
    rng = np.random.default_rng(M * 7 + N + K)
    fmt = {"f16": hip.FMT_F16, "w8": hip.FMT_W8, "w4": hip.FMT_W4}[fmt_name]
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float16)
    parts = _quant_parts(orc, hip, fmt, w)
    y_ref = orc.gemv(fmt, x, parts[0], parts[1], parts[2])
    dparts = [dev(hip, p) if p is not None else None for p in parts]
    packed = hip.DeviceArray(parts[0].shape, parts[0].dtype)
    hip.pack_weights(fmt, N, K, dparts[0], packed)
    ws = hip.DeviceArray((max(hip.linear_packed_workspace(M, N, K), 16),), np.uint8)
    y = hip.DeviceArray((M, N), np.float16)
    first = None
    for _ in range(2):
        y.fill0()
        hip.linear_packed(fmt, M, N, K, dev(hip, x), packed, dparts[1], dparts[2], y, ws)
        hip.device_sync()
        got = y.numpy()
        err = rel_err(got.astype(np.float32), y_ref.astype(np.float32))
        assert err <= F16_TOL
        if first is not None:   # split partials are summed in a fixed order: repeat calls agree bitwise
            same = np.array_equal(first.view(np.uint16), got.view(np.uint16))
            assert same
        first = got
    # relu^2 epilogue and fp32 output
    y32 = hip.DeviceArray((M, N), np.float32)
    hip.linear_packed(fmt, M, N, K, dev(hip, x), packed, dparts[1], dparts[2], y32, ws, out_f32=1)
    hip.linear_packed(fmt, M, N, K, dev(hip, x), packed, dparts[1], dparts[2], y, ws, epilogue=hip.EPI_RELU_SQUARE)
    hip.device_sync()
    got32 = y32.numpy()
    err = rel_err(got32, y_ref.astype(np.float32))
    assert err <= F16_TOL
    same = np.array_equal(got32, got32.astype(np.float16).astype(np.float32))
    assert same
    err = rel_err(y.numpy().astype(np.float32), orc.relu_square(y_ref).astype(np.float32))
    assert err <= 2 * F16_TOL


def test_pack_weights_is_the_documented_permutation(gpu):
    """Tile (band nt, k group kg) holds, for lane j + 32h, the KR consecutive k of row 32 nt + j starting at
    kg*G + h*KR, as 64 x 16-byte pieces (two pieces for fp16)."""
    hip = gpu
    rng = np.random.default_rng(4)
    N, K = 64, 512
    for fmt, dtype, per, G, pieces in ((hip.FMT_F16, np.float16, 8, 32, 2), (hip.FMT_W8, np.int8, 16, 32, 1),
                                       (hip.FMT_W4, np.uint8, 32, 64, 1)):
        cols = K if fmt != hip.FMT_W4 else K // 2
        if dtype == np.float16:
            src = rng.standard_normal((N, cols)).astype(dtype)
        else:
            src = rng.integers(-128 if dtype == np.int8 else 0, 127, (N, cols)).astype(dtype)
        packed = hip.DeviceArray(src.shape, src.dtype)
        hip.pack_weights(fmt, N, K, dev(hip, src), packed)
        hip.device_sync()
        got = packed.numpy().view(np.uint8).reshape(-1, 16)
        src_pieces = src.view(np.uint8).reshape(-1, 16)        # row-major 16-byte pieces
        KR = G // 2
        want = np.empty_like(got)
        p = 0
        for nt in range(N // 32):
            for kg in range(K // G):
                for i in range(pieces):
                    for lane in range(64):
                        row, h = nt * 32 + lane % 32, lane // 32
                        k = kg * G + h * KR + i * 8
                        want[p] = src_pieces[(row * K + k) // per]
                        p += 1
        same = np.array_equal(got, want)
        assert same


def test_linear_packed_rejects_bad_arguments(gpu):
    hip = gpu
    x = hip.DeviceArray((16, 256), np.float16)
    ws = hip.DeviceArray((8192,), np.uint8)
    with pytest.raises(hip.RwkvHipError, match="unsupported shape"):
        hip.linear_packed(hip.FMT_W8, 16, 48, 256, x, x, x, None, x, ws)      # N not a multiple of 32
    with pytest.raises(hip.RwkvHipError, match="unsupported shape"):
        hip.linear_packed(hip.FMT_W8, 16, 64, 320, x, x, x, None, x, ws)      # K not a multiple of 256
    with pytest.raises(hip.RwkvHipError, match="scale"):
        hip.linear_packed(hip.FMT_W8, 16, 64, 256, x, x, None, None, x, ws)
    with pytest.raises(hip.RwkvHipError, match="workspace"):
        hip.linear_packed(hip.FMT_F16, 16, 64, 4096, x, x, None, None, x, None)  # split K without a workspace


def test_wkv7_long_chunked_resume_through_host_slab_is_bitwise(gpu):
    """Benchmark configuration 4 at reduced size: fp16 r,w,k,v,a,b, fp32 state, sequence run in chunks of 128 with the state
    slab copied to the host and into a fresh device buffer at every quarter; outputs and final state must equal
    the single uninterrupted call bit for bit."""
    hip = gpu
    B, T, H = 1, 1024, 6
    C = H * 64
    t = wkv_inputs(B, T, H, seed=5, dtype=np.float16)
    dr, dw, dk, dv, da, db = [dev(hip, t[n]) for n in ("r", "w_raw", "k", "v", "a", "b")]
    s_full = hip.DeviceArray.zeros((B, H, 64, 64), np.float32)
    y_full = hip.DeviceArray((B, T, C), np.float16)
    hip.wkv7(B, T, C, H, hip.W_RAW_LOGIT, hip.IO_F16, s_full, dr, dw, dk, dv, da, db, y_full)
    hip.device_sync()

    state = hip.DeviceArray.zeros((B, H, 64, 64), np.float32)
    y = hip.DeviceArray((B, T, C), np.float16)
    for t0 in range(0, T, 128):
        if t0 and t0 % (T // 4) == 0:           # checkpoint: slab to the host, resume from a fresh allocation
            slab = state.numpy()
            state = hip.DeviceArray.from_numpy(slab)
        off = t0 * C
        views = [d.view(off, (1, 128, C)) for d in (dr, dw, dk, dv, da, db)]
        hip.wkv7(1, 128, C, H, hip.W_RAW_LOGIT, hip.IO_F16, state, views[0], views[1], views[2], views[3], views[4],
                 views[5], y.view(off, (1, 128, C)))
    hip.device_sync()
    same = np.array_equal(y.numpy().view(np.uint16), y_full.numpy().view(np.uint16))
    assert same
    same = np.array_equal(state.numpy().view(np.uint32), s_full.numpy().view(np.uint32))
    assert same
    finite = bool(np.isfinite(y.numpy().astype(np.float32)).all())
    assert finite


def test_wkv7_config4_full_size_chunked_resume_is_bitwise(gpu):
    """Benchmark configuration 4 at its full size: B = 16, T = 16384, H = 64, fp16 r,w,k,v,a,b (2.1 GB each), fp32
    state.  The rows are windows of one host-generated sequence with the configuration-0 distributions, copied on
    the device.  The sequence run as 128 chunks of 128 tokens, with the state slab taken to the host and resumed from
    a fresh device buffer every 4096 tokens, must give the outputs and the final state of the single uninterrupted
    call bit for bit; the outputs stay finite over the whole length."""
    hip = gpu
    B, T, H, chunk = 16, 16384, 64, 128
    C = H * 64
    seg = 4096
    n_win = B * (T // seg)
    base_T = seg + 64 * (n_win - 1)
    t = wkv_inputs(1, base_T, H, seed=11, dtype=np.float16)
    names = ("r", "w_raw", "k", "v", "a", "b")
    base = [dev(hip, t[n]) for n in names]
    del t
    ops = [hip.DeviceArray((B, T, C), np.float16) for _ in names]
    for b in range(B):
        for q in range(T // seg):
            start = 64 * (b * (T // seg) + q)
            for src, dst in zip(base, ops):
                dst.view((b * T + q * seg) * C, (seg, C)).copy_from(src.view(start * C, (seg, C)))
    for d in base:
        d.free()

    s_full = hip.DeviceArray.zeros((B, H, 64, 64), np.float32)
    y_full = hip.DeviceArray((B, T, C), np.float16)
    hip.wkv7(B, T, C, H, hip.W_RAW_LOGIT, hip.IO_F16, s_full, *ops, y_full)
    hip.device_sync()

    state = hip.DeviceArray.zeros((B, H, 64, 64), np.float32)
    y = hip.DeviceArray((B, T, C), np.float16)
    stage = [hip.DeviceArray((B, chunk, C), np.float16) for _ in names]
    y_stage = hip.DeviceArray((B, chunk, C), np.float16)
    for t0 in range(0, T, chunk):
        if t0 and t0 % seg == 0:                  # checkpoint: slab to the host, resume from a fresh allocation
            slab = state.numpy()
            state = hip.DeviceArray.from_numpy(slab)
        for b in range(B):
            for src, dst in zip(ops, stage):
                dst.view(b * chunk * C, (chunk, C)).copy_from(src.view((b * T + t0) * C, (chunk, C)))
        hip.wkv7(B, chunk, C, H, hip.W_RAW_LOGIT, hip.IO_F16, state, *stage, y_stage)
        for b in range(B):
            y.view((b * T + t0) * C, (chunk, C)).copy_from(y_stage.view(b * chunk * C, (chunk, C)))
    hip.device_sync()
    for b in range(B):
        got = y.view(b * T * C, (T, C)).numpy()
        same = np.array_equal(got.view(np.uint16), y_full.view(b * T * C, (T, C)).numpy().view(np.uint16))
        assert same, "batch row %d" % b
        finite = bool(np.isfinite(got.astype(np.float32)).all())
        assert finite, "batch row %d" % b
    same = np.array_equal(state.numpy().view(np.uint32), s_full.numpy().view(np.uint32))
    assert same
