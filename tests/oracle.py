"""ctypes wrapper of the CPU oracle (oracle/librwkv_oracle.so) with numpy in / numpy out.

Test infrastructure: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may use it.
fp16 tensors are numpy float16 arrays (passed as their uint16 bit patterns).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_DIR = os.path.join(os.path.dirname(_HERE), "oracle")
LIB_PATH = os.path.join(ORACLE_DIR, "librwkv_oracle.so")

FMT_F16, FMT_W8, FMT_W4 = 0, 1, 2

_lib = None


def build():
    subprocess.run(["make", "-C", ORACLE_DIR, "-s"], check=True)


def lib():
    global _lib
    if _lib is None:
        src_m = max(os.path.getmtime(os.path.join(ORACLE_DIR, f)) for f in ("rwkv_oracle.cpp", "rwkv_oracle.h"))
        if not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < src_m:
            build()
        L = ctypes.CDLL(LIB_PATH)
        L.orc_f16_to_f32.restype = ctypes.c_float
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_f32_to_f16.argtypes = [ctypes.c_float]
        L.orc_model_create.restype = ctypes.c_void_p
        L.orc_f64_to_f16.restype = ctypes.c_uint16
        L.orc_f64_to_f16.argtypes = [ctypes.c_double]
        L.orc_f16_fma.restype = ctypes.c_uint16
        L.orc_f16_fma.argtypes = [ctypes.c_uint16, ctypes.c_uint16, ctypes.c_uint16]
        L.orc_wkv16_rotator.restype = ctypes.c_float
        L.orc_wkv16_rotator.argtypes = [ctypes.c_int32]
        L.orc_wkv16_w_delta.restype = ctypes.c_uint16
        L.orc_wkv16_w_delta.argtypes = [ctypes.c_uint16, ctypes.c_void_p, ctypes.c_int, ctypes.c_int32]
        L.orc_sample_greedy_penalty.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float,
                                                ctypes.c_float, ctypes.c_float, ctypes.c_float]
        L.orc_sample_filter.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_int,
                                        ctypes.c_float, ctypes.c_void_p]
        _lib = L
    return _lib


def set_threads(n):
    lib().orc_set_threads(ctypes.c_int(n))


def _p(a):
    if a is None:
        return ctypes.c_void_p(0)
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def f32_to_f16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.float16)
    lib().orc_f32_to_f16_array(_p(x), _p(out), ctypes.c_int64(x.size))
    return out


def bf16_to_f16(bits, transpose=False):
    """bits: uint16 [rows, cols] of bf16 patterns -> float16 [rows, cols] (or [cols, rows])."""
    bits = _c(bits, np.uint16)
    rows, cols = bits.shape
    out = np.empty((cols, rows) if transpose else (rows, cols), np.float16)
    lib().orc_bf16_to_f16(rows, cols, int(bool(transpose)), _p(bits), _p(out))
    return out


def emb_ln0(emb_bits, w_bits, b_bits, eps=1e-5):
    """bf16 patterns (uint16) of the embedding [V,C] and ln0 weight / bias [C] -> float16 [V,C]."""
    emb_bits = _c(emb_bits, np.uint16)
    V, C = emb_bits.shape
    out = np.empty((V, C), np.float16)
    lib().orc_emb_ln0(V, C, _p(emb_bits), _p(_c(w_bits, np.uint16)), _p(_c(b_bits, np.uint16)), ctypes.c_float(eps), _p(out))
    return out


def f16_to_f32(x):
    x = _c(x, np.float16)
    out = np.empty(x.shape, np.float32)
    lib().orc_f16_to_f32_array(_p(x), _p(out), ctypes.c_int64(x.size))
    return out


def wkv7(state, r, w, k, v, a, b, H, w_mode=0):
    """state f32 [B,H,64,64] (updated in place); r..b [B,T,C] float32 or float16.  Returns y."""
    B, T, C = r.shape
    assert state.dtype == np.float32 and state.flags.c_contiguous
    if r.dtype == np.float16:
        args = [_c(t, np.float16) for t in (r, w, k, v, a, b)]
        y = np.empty((B, T, C), np.float16)
        fn = lib().orc_wkv7_f16
    else:
        args = [_c(t, np.float32) for t in (r, w, k, v, a, b)]
        y = np.empty((B, T, C), np.float32)
        fn = lib().orc_wkv7_f32
    fn(B, T, C, H, w_mode, _p(state), *[_p(t) for t in args], _p(y))
    return y


def wkv7_f16state(state, r, w, k, v, a, b, H, elapsed, w0=None):
    """state f16 [B,H,64,64] (updated in place); r..b f16 [B,T,C]; w raw decay logits; w0 f16 [C] or None;
    elapsed int32 [B] (not modified).  Returns y f16 [B,T,C]."""
    B, T, C = r.shape
    assert state.dtype == np.float16 and state.flags.c_contiguous
    args = [_c(t, np.float16) for t in (r, w, k, v, a, b)]
    w0c = None if w0 is None else _c(w0, np.float16)
    y = np.empty((B, T, C), np.float16)
    lib().orc_wkv7_f16state(B, T, C, H, _p(state), _p(args[0]), _p(args[1]), _p(w0c), _p(args[2]), _p(args[3]),
                            _p(args[4]), _p(args[5]), _p(y), _p(_c(elapsed, np.int32)))
    return y


def quantize_w8(w):
    w = _c(w, np.float16)
    N, K = w.shape
    q = np.empty((N, K), np.int8)
    s = np.empty((N,), np.float16)
    lib().orc_quantize_w8(N, K, _p(w), _p(q), _p(s))
    return q, s


def dequant_w8(q, s):
    N, K = q.shape
    w = np.empty((N, K), np.float16)
    lib().orc_dequant_w8(N, K, _p(_c(q, np.int8)), _p(_c(s, np.float16)), _p(w))
    return w


def quantize_w4(w):
    w = _c(w, np.float16)
    N, K = w.shape
    q = np.empty((N, K // 2), np.uint8)
    s = np.empty((N, K // 128), np.float16)
    z = np.empty((N, K // 128), np.uint8)
    lib().orc_quantize_w4(N, K, _p(w), _p(q), _p(s), _p(z))
    return q, s, z


def dequant_w4(q, s, z):
    N, K = q.shape[0], q.shape[1] * 2
    w = np.empty((N, K), np.float16)
    lib().orc_dequant_w4(N, K, _p(_c(q, np.uint8)), _p(_c(s, np.float16)), _p(_c(z, np.uint8)), _p(w))
    return w


def gemv(fmt, x, w, scale=None, zp=None, f32_out=False):
    """x f16 [M,K]; w per fmt ([N,K] f16 / int8, or packed [N,K/2]).  Returns y [M,N]."""
    x = _c(x, np.float16)
    M, K = x.shape
    N = w.shape[0]
    w = np.ascontiguousarray(w)
    if f32_out:
        y = np.empty((M, N), np.float32)
        lib().orc_gemv_any_f32(fmt, M, N, K, _p(x), _p(w), _p(scale), _p(zp), _p(y))
        return y
    y = np.empty((M, N), np.float16)
    if fmt == FMT_F16:
        lib().orc_gemv_f16(M, N, K, _p(x), _p(_c(w, np.float16)), _p(y))
    elif fmt == FMT_W8:
        lib().orc_gemv_w8(M, N, K, _p(x), _p(w), _p(scale), _p(y))
    else:
        lib().orc_gemv_w4(M, N, K, _p(x), _p(w), _p(scale), _p(zp), _p(y))
    return y


def layer_norm(x, w, b, eps=1e-5):
    x = _c(x, np.float16)
    rows, C = x.shape
    y = np.empty_like(x)
    lib().orc_layer_norm(rows, C, _p(x), _p(_c(w, np.float16)), _p(_c(b, np.float16)), _p(y), ctypes.c_float(eps))
    return y


def add_layer_norm(x, res, w, b, eps=1e-5):
    x = _c(x, np.float16)
    rows, C = x.shape
    xo, y = np.empty_like(x), np.empty_like(x)
    lib().orc_add_layer_norm(rows, C, _p(x), _p(_c(res, np.float16)), _p(_c(w, np.float16)), _p(_c(b, np.float16)),
                             _p(xo), _p(y), ctypes.c_float(eps))
    return xo, y


def add_last_layer_norm(x, res, w, b, B, T, eps=1e-5):
    x = _c(x, np.float16)
    C = x.shape[-1]
    y = np.empty((B, C), np.float16)
    lib().orc_add_last_layer_norm(B, T, C, _p(x), _p(_c(res, np.float16)), _p(_c(w, np.float16)), _p(_c(b, np.float16)),
                                  _p(y), ctypes.c_float(eps))
    return y


def _ptrs(arrs):
    arr = (ctypes.c_void_p * len(arrs))()
    for i, a in enumerate(arrs):
        arr[i] = a.ctypes.data
    return arr


def token_shift_mix(x, shift, mus, B, T):
    """x f16 [B*T,C]; shift f16 [B,C] updated in place.  Returns list of outputs."""
    x = _c(x, np.float16)
    C = x.shape[-1]
    mus = [_c(m, np.float16) for m in mus]
    outs = [np.empty_like(x) for _ in mus]
    lib().orc_token_shift_mix(B, T, C, len(mus), _p(x), _p(shift), _ptrs(mus), _ptrs(outs))
    return outs


def add_layer_norm_cmix_mix(x, res, shift, w, b, mu_k, eps=1e-5):
    x = _c(x, np.float16)
    rows, C = x.shape
    xo, mixed = np.empty_like(x), np.empty_like(x)
    lib().orc_add_layer_norm_cmix_mix(rows, C, _p(x), _p(_c(res, np.float16)), _p(shift), _p(_c(w, np.float16)),
                                      _p(_c(b, np.float16)), _p(_c(mu_k, np.float16)), _p(xo), _p(mixed),
                                      ctypes.c_float(eps))
    return xo, mixed


def add_layer_norm_tmix_mix6(x, res, shift, w, b, mus, eps=1e-5):
    x = _c(x, np.float16)
    rows, C = x.shape
    mus = [_c(m, np.float16) for m in mus]
    xo = np.empty_like(x)
    outs = [np.empty_like(x) for _ in range(6)]
    lib().orc_add_layer_norm_tmix_mix6(rows, C, _p(x), _p(_c(res, np.float16)), _p(shift), _p(_c(w, np.float16)),
                                       _p(_c(b, np.float16)), _ptrs(mus), _p(xo), _ptrs(outs), ctypes.c_float(eps))
    return xo, outs


def kk_a_gate(k, k_k, a0, a12, k_a, H):
    k = _c(k, np.float16)
    rows, C = k.shape
    nk, nkk, kka = np.empty_like(k), np.empty_like(k), np.empty_like(k)
    lib().orc_kk_a_gate(rows, C, H, _p(k), _p(_c(k_k, np.float16)), _p(_c(a0, np.float16)), _p(_c(a12, np.float16)),
                        _p(_c(k_a, np.float16)), _p(nk), _p(nkk), _p(kka))
    return nk, nkk, kka


def lnx_rkvres_xg(y, r, k, v, r_k, lnw, lnb, g, H):
    y = _c(y, np.float16)
    rows, C = y.shape
    out = np.empty_like(y)
    lib().orc_lnx_rkvres_xg(rows, C, H, _p(y), _p(_c(r, np.float16)), _p(_c(k, np.float16)), _p(_c(v, np.float16)),
                            _p(_c(r_k, np.float16)), _p(_c(lnw, np.float16)), _p(_c(lnb, np.float16)),
                            _p(_c(g, np.float16)), _p(out))
    return out


def vres_gate(v, v_first, v0, v12_f32):
    v = _c(v, np.float16)
    rows, C = v.shape
    out = np.empty_like(v)
    lib().orc_vres_gate(rows, C, _p(v), _p(_c(v_first, np.float16)), _p(_c(v0, np.float16)), _p(_c(v12_f32, np.float32)),
                        _p(out))
    return out


def relu_square(x):
    x = _c(x, np.float16)
    out = np.empty_like(x)
    lib().orc_relu_square(ctypes.c_int64(x.size), _p(x), _p(out))
    return out


def add_vec(x, vec):
    x = _c(x, np.float16)
    rows, C = x.shape
    out = np.empty_like(x)
    lib().orc_add_vec(rows, C, _p(x), _p(_c(vec, np.float16)), _p(out))
    return out


def lora(x, w1, w2, act):
    """x f16 [M,C]; w1 f16 [R,C]; w2 f16 [C,R].  Returns fp32 [M,C]."""
    x = _c(x, np.float16)
    M, C = x.shape
    R = w1.shape[0]
    out = np.empty((M, C), np.float32)
    lib().orc_lora(M, C, R, act, _p(x), _p(_c(w1, np.float16)), _p(_c(w2, np.float16)), _p(out))
    return out


def sample_greedy_penalty(logits, penalties, presence, frequency, decay, temperature=1.0):
    logits = _c(logits, np.float32)
    assert penalties.dtype == np.float32
    return lib().orc_sample_greedy_penalty(logits.size, _p(logits), _p(penalties), presence, frequency, decay,
                                           temperature)


def sample_filter(logits, penalties, temperature, top_k, top_p):
    logits = _c(logits, np.float32)
    probs = np.empty_like(logits)
    kept = lib().orc_sample_filter(logits.size, _p(logits), _p(penalties), temperature, top_k, top_p, _p(probs))
    return kept, probs


class Model:
    """Oracle model over numpy weights in the layout of rwkv_lightning_cuda_amd.model.synth_weights."""

    T_IDS = {"ln1_w": 10, "ln1_b": 11, "ln2_w": 12, "ln2_b": 13, "x_r": 14, "x_w": 15, "x_k": 16, "x_v": 17,
             "x_a": 18, "x_g": 19, "w0": 20, "a0": 21, "v0": 22, "k_k": 23, "k_a": 24, "r_k": 25, "lnx_w": 26,
             "lnx_b": 27, "ffn_x_k": 28, "w1": 40, "w2": 41, "a1": 42, "a2": 43, "g1": 44, "g2": 45, "v1": 46, "v2": 47}
    M_IDS = {"att_r": 0, "att_k": 1, "att_v": 2, "att_o": 3, "ffn_key": 4, "ffn_value": 5, "head": 6}

    def __init__(self, dims, weights, fmt=FMT_F16):
        self.dims = dims
        self.fmt = fmt
        self._keep = []
        L = lib()
        self.h = ctypes.c_void_p(L.orc_model_create(dims.L, dims.C, dims.H, dims.F, dims.V, dims.Rw, dims.Ra, dims.Rg,
                                                    dims.Rv))
        assert self.h
        self.quant = {}

        def keep(a):
            self._keep.append(a)
            return a

        def set_t(layer, tid, arr):
            assert L.orc_model_set_tensor(self.h, layer, tid, _p(keep(_c(arr, np.float16)))) == 0

        def set_m(layer, name, arr):
            arr = _c(arr, np.float16)
            if fmt == FMT_F16:
                parts = (keep(arr), None, None)
            elif fmt == FMT_W8:
                q, s = quantize_w8(arr)
                parts = (keep(q), keep(s), None)
            else:
                q, s, z = quantize_w4(arr)
                parts = (keep(q), keep(s), keep(z))
            self.quant[(layer, name)] = parts
            assert L.orc_model_set_matrix(self.h, layer, self.M_IDS[name], fmt, _p(parts[0]), _p(parts[1]),
                                          _p(parts[2])) == 0

        set_t(-1, 0, weights["emb_ln0"])
        set_t(-1, 1, weights["ln_out_w"])
        set_t(-1, 2, weights["ln_out_b"])
        set_m(-1, "head", weights["head"])
        for l, lw in enumerate(weights["layers"]):
            for name, arr in lw.items():
                if name in self.T_IDS:
                    set_t(l, self.T_IDS[name], arr)
                else:
                    set_m(l, name, arr)

    def new_state(self, B, wkv_fp16=False):
        d = self.dims
        return (np.zeros((d.L, 2, B, d.C), np.float16),
                np.zeros((d.L, B, d.H, 64, 64), np.float16 if wkv_fp16 else np.float32), np.zeros((B,), np.int32))

    def forward(self, tokens, state, trace=False):
        tokens = _c(tokens, np.int64)
        B, T = tokens.shape
        shift, wkv, elapsed = state
        logits = np.empty((B, self.dims.V), np.float32)
        tr = np.empty((self.dims.L, B * T, self.dims.C), np.float16) if trace else None
        fn = lib().orc_model_forward_f16state if wkv.dtype == np.float16 else lib().orc_model_forward
        rc = fn(self.h, _p(tokens), B, T, _p(shift), _p(wkv), _p(elapsed), _p(logits), _p(tr))
        if rc != 0:
            raise ValueError("orc_model_forward failed: %d" % rc)
        return (logits, tr) if trace else logits

    def __del__(self):
        try:
            lib().orc_model_destroy(self.h)
        except Exception:
            pass
