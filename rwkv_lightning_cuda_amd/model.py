"""Host-side model plumbing above the C ABI: shapes, synthetic weights, device upload with
quantise-on-load, state allocation and the forward / greedy-decode calls.

Mirrors the reference's ModelBackend surface (include/rwkv_server_backend.hpp:104-147):
create_state / forward_prefill / forward_decode, with the state layout of
src/rwkv7_fast_v4.cu:1373-1400 (shift f16 [L,2,B,C], wkv_state32 f32 [L,B,H,64,64], elapsed i32 [B]).
"""
import ctypes
from dataclasses import dataclass

import numpy as np

from . import hip

# (tensor id, shape key) of the per-layer fp16 vectors, in the order weights are generated
VEC_IDS = [
    ("ln1_w", hip.T_LN1_W), ("ln1_b", hip.T_LN1_B), ("ln2_w", hip.T_LN2_W), ("ln2_b", hip.T_LN2_B),
    ("x_r", hip.T_X_R), ("x_w", hip.T_X_W), ("x_k", hip.T_X_K), ("x_v", hip.T_X_V), ("x_a", hip.T_X_A),
    ("x_g", hip.T_X_G), ("w0", hip.T_W0), ("a0", hip.T_A0), ("v0", hip.T_V0), ("k_k", hip.T_K_K),
    ("k_a", hip.T_K_A), ("r_k", hip.T_R_K), ("lnx_w", hip.T_LNX_W), ("lnx_b", hip.T_LNX_B),
    ("ffn_x_k", hip.T_FFN_X_K),
]
LORA_IDS = [("w1", hip.T_W1, "Rw", 1), ("w2", hip.T_W2, "Rw", 2), ("a1", hip.T_A1, "Ra", 1), ("a2", hip.T_A2, "Ra", 2),
            ("g1", hip.T_G1, "Rg", 1), ("g2", hip.T_G2, "Rg", 2), ("v1", hip.T_V1, "Rv", 1), ("v2", hip.T_V2, "Rv", 2)]
MAT_IDS = [("att_r", hip.M_ATT_R), ("att_k", hip.M_ATT_K), ("att_v", hip.M_ATT_V), ("att_o", hip.M_ATT_O),
           ("ffn_key", hip.M_FFN_KEY), ("ffn_value", hip.M_FFN_VALUE)]


@dataclass(frozen=True)
class ModelDims:
    L: int
    C: int
    H: int
    F: int
    V: int
    Rw: int
    Ra: int
    Rg: int
    Rv: int

    def mat_shape(self, name):
        C, F, V = self.C, self.F, self.V
        return {"att_r": (C, C), "att_k": (C, C), "att_v": (C, C), "att_o": (C, C), "ffn_key": (F, C),
                "ffn_value": (C, F), "head": (V, C)}[name]


# Shapes of the benchmark configurations.  LoRA ranks (w, a, v, g): 0.1B as given there; the larger
# ones follow the upstream RWKV-7 convention.
PRESETS = {
    "0.1B": ModelDims(L=12, C=768, H=12, F=3072, V=65536, Rw=64, Ra=64, Rg=128, Rv=32),
    "1.5B": ModelDims(L=24, C=2048, H=32, F=8192, V=65536, Rw=96, Ra=96, Rg=256, Rv=64),
    "7.2B": ModelDims(L=32, C=4096, H=64, F=16384, V=65536, Rw=128, Ra=128, Rg=480, Rv=96),
}


def synth_weights(dims, seed, std=0.02):
    """Random-init fp16 weights ~ N(0, std) for every tensor (numpy, host).  LayerNorm / GroupNorm weights
    are 1 + N(0, std); the token-shift mixes are U(0,1); w0 is spread over the decay range."""
    rng = np.random.default_rng(seed)
    C = dims.C

    def nrm(*shape):
        return (rng.standard_normal(shape, dtype=np.float32) * std).astype(np.float16)

    w = {"emb_ln0": None, "layers": []}
    emb = rng.standard_normal((dims.V, C), dtype=np.float32) * std
    # ln0 applied to the embedding table, as the reference pre-computes at load time
    mu = emb.mean(axis=1, keepdims=True)
    var = ((emb - mu) ** 2).mean(axis=1, keepdims=True)
    ln0_w = 1.0 + rng.standard_normal(C, dtype=np.float32) * std
    ln0_b = rng.standard_normal(C, dtype=np.float32) * std
    w["emb_ln0"] = ((emb - mu) / np.sqrt(var + 1e-5) * ln0_w + ln0_b).astype(np.float16)
    w["ln_out_w"] = (1.0 + rng.standard_normal(C, dtype=np.float32) * std).astype(np.float16)
    w["ln_out_b"] = nrm(C)
    w["head"] = nrm(dims.V, C)
    for _ in range(dims.L):
        lw = {}
        for name, _id in VEC_IDS:
            if name in ("ln1_w", "ln2_w", "lnx_w"):
                lw[name] = (1.0 + rng.standard_normal(C, dtype=np.float32) * std).astype(np.float16)
            elif name.startswith("x_") or name == "ffn_x_k":
                lw[name] = rng.uniform(0.0, 1.0, C).astype(np.float16)
            elif name == "w0":
                lw[name] = rng.uniform(-6.0, 1.0, C).astype(np.float16)
            elif name in ("k_k", "k_a"):
                lw[name] = (1.0 + rng.standard_normal(C, dtype=np.float32) * 0.1).astype(np.float16)
            else:
                lw[name] = nrm(C)
        for name, _id, rk, which in LORA_IDS:
            R = getattr(dims, rk)
            # scaled up from N(0, std) so the low-rank paths contribute visibly to the activations
            shape = (R, C) if which == 1 else (C, R)
            lw[name] = (rng.standard_normal(shape, dtype=np.float32) * (std * 4)).astype(np.float16)
        for name, _id in MAT_IDS:
            lw[name] = nrm(*dims.mat_shape(name))
        w["layers"].append(lw)
    return w


class DeviceMatrix:
    """A [N,K] weight matrix on the device in one of the three formats."""

    def __init__(self, fmt, N, K, data, scale=None, zp=None):
        self.fmt, self.N, self.K, self.data, self.scale, self.zp = fmt, N, K, data, scale, zp

    @classmethod
    def from_f16_device(cls, fmt, N, K, w_dev):
        """Quantise-on-load from an fp16 device tensor (kept as is for FMT_F16)."""
        if fmt == hip.FMT_F16:
            return cls(fmt, N, K, w_dev)
        if fmt == hip.FMT_W8:
            q = hip.DeviceArray((N, K), np.int8)
            s = hip.DeviceArray((N,), np.float16)
            hip.quantize_w8(N, K, w_dev, q, s)
            return cls(fmt, N, K, q, s)
        q = hip.DeviceArray((N, K // 2), np.uint8)
        s = hip.DeviceArray((N, K // 128), np.float16)
        z = hip.DeviceArray((N, K // 128), np.uint8)
        hip.quantize_w4(N, K, w_dev, q, s, z)
        return cls(fmt, N, K, q, s, z)


class HipModel:
    """Owns the device weights and the rwkv_hip_model handle."""

    def __init__(self, dims, fmt=hip.FMT_F16):
        self.dims, self.fmt = dims, fmt
        self._keep = []
        h = ctypes.c_void_p(0)
        hip.check(hip.load().rwkv_hip_model_create(ctypes.byref(h), dims.L, dims.C, dims.H, dims.F, dims.V, dims.Rw,
                                                   dims.Ra, dims.Rg, dims.Rv))
        self.handle = h
        self.mats = {}

    def set_tensor(self, layer, tid, dev):
        self._keep.append(dev)
        hip.check(hip.load().rwkv_hip_model_set_tensor(self.handle, ctypes.c_int(layer), ctypes.c_int(tid), hip._p(dev)))

    def set_matrix(self, layer, mid, mat):
        self._keep.append(mat)
        self.mats[(layer, mid)] = mat
        hip.check(hip.load().rwkv_hip_model_set_matrix(self.handle, ctypes.c_int(layer), ctypes.c_int(mid),
                                                       ctypes.c_int(mat.fmt), hip._p(mat.data), hip._p(mat.scale),
                                                       hip._p(mat.zp)))

    @classmethod
    def from_host_weights(cls, dims, weights, fmt=hip.FMT_F16):
        """Uploads numpy weights (synth_weights layout); the seven big matrices are quantised on the device."""
        m = cls(dims, fmt)
        m.set_tensor(-1, hip.T_EMB_LN0, hip.DeviceArray.from_numpy(weights["emb_ln0"]))
        m.set_tensor(-1, hip.T_LN_OUT_W, hip.DeviceArray.from_numpy(weights["ln_out_w"]))
        m.set_tensor(-1, hip.T_LN_OUT_B, hip.DeviceArray.from_numpy(weights["ln_out_b"]))
        N, K = dims.mat_shape("head")
        m.set_matrix(-1, hip.M_HEAD, DeviceMatrix.from_f16_device(fmt, N, K, hip.DeviceArray.from_numpy(weights["head"])))
        for l, lw in enumerate(weights["layers"]):
            for name, tid in VEC_IDS:
                m.set_tensor(l, tid, hip.DeviceArray.from_numpy(lw[name]))
            for name, tid, _rk, _which in LORA_IDS:
                m.set_tensor(l, tid, hip.DeviceArray.from_numpy(lw[name]))
            for name, mid in MAT_IDS:
                N, K = dims.mat_shape(name)
                m.set_matrix(l, mid, DeviceMatrix.from_f16_device(fmt, N, K, hip.DeviceArray.from_numpy(lw[name])))
        hip.device_sync()
        return m

    @classmethod
    def random_on_device(cls, dims, fmt, seed=0, std=0.02):
        """Random-init weights generated on the GPU (no host copy): N(0, std) matrices quantised on load."""
        m = cls(dims, fmt)
        C = dims.C
        ctr = [seed * 1000003 + 1]

        def fill(shape, mean=0.0, s=std):
            d = hip.DeviceArray(shape, np.float16)
            ctr[0] += 1
            hip.fill_normal_f16(int(np.prod(shape)), ctr[0], mean, s, d)
            return d

        def matrix(name):
            N, K = dims.mat_shape(name)
            w16 = fill((N, K))
            mat = DeviceMatrix.from_f16_device(fmt, N, K, w16)
            if fmt != hip.FMT_F16:
                hip.device_sync()
                w16.free()
            return mat

        # a real table has ln0 applied: rows are roughly unit variance
        m.set_tensor(-1, hip.T_EMB_LN0, fill((dims.V, C), 0.0, 1.0))
        m.set_tensor(-1, hip.T_LN_OUT_W, fill((C,), 1.0))
        m.set_tensor(-1, hip.T_LN_OUT_B, fill((C,)))
        m.set_matrix(-1, hip.M_HEAD, matrix("head"))
        for l in range(dims.L):
            for name, tid in VEC_IDS:
                if name in ("ln1_w", "ln2_w", "lnx_w", "k_k", "k_a"):
                    m.set_tensor(l, tid, fill((C,), 1.0))
                elif name.startswith("x_") or name == "ffn_x_k":
                    m.set_tensor(l, tid, fill((C,), 0.5, 0.15))
                elif name == "w0":
                    m.set_tensor(l, tid, fill((C,), -2.0, 1.5))
                else:
                    m.set_tensor(l, tid, fill((C,)))
            for name, tid, rk, which in LORA_IDS:
                R = getattr(dims, rk)
                m.set_tensor(l, tid, fill((R, C) if which == 1 else (C, R), 0.0, std * 4))
            for name, mid in MAT_IDS:
                m.set_matrix(l, mid, matrix(name))
        hip.device_sync()
        return m

    def weight_bytes(self):
        n = ctypes.c_uint64(0)
        hip.check(hip.load().rwkv_hip_model_weight_bytes(self.handle, ctypes.byref(n)))
        return n.value

    def close(self):
        if self.handle:
            hip.load().rwkv_hip_model_destroy(self.handle)
            self.handle = None


class State:
    """Generation state on the device (GenerationState, include/rwkv_server_backend.hpp:45-58, wkv32 mode)."""

    def __init__(self, dims, B, wkv_fp16=False):
        self.B = B
        self.wkv_fp16 = wkv_fp16
        self.shift = hip.DeviceArray.zeros((dims.L, 2, B, dims.C), np.float16)
        self.wkv = hip.DeviceArray.zeros((dims.L, B, dims.H, 64, 64), np.float16 if wkv_fp16 else np.float32)
        self.elapsed = hip.DeviceArray.zeros((B,), np.int32)


class Session:
    def __init__(self, model):
        self.model = model
        h = ctypes.c_void_p(0)
        hip.check(hip.load().rwkv_hip_session_create(ctypes.byref(h), model.handle))
        self.handle = h
        self._trace = None

    @property
    def stream(self):
        s = ctypes.c_void_p(0)
        hip.check(hip.load().rwkv_hip_session_stream(self.handle, ctypes.byref(s)))
        return s.value

    def set_graph(self, on):
        hip.check(hip.load().rwkv_hip_session_set_graph(self.handle, ctypes.c_int(1 if on else 0)))

    def set_trace(self, dev):
        self._trace = dev
        hip.check(hip.load().rwkv_hip_session_set_trace(self.handle, hip._p(dev)))

    DEBUG_IDS = ["x", "xx", "xr", "xw", "xk", "xv", "xa", "xg", "r", "k", "v", "v_first", "w12", "a12", "g", "hw", "ha",
                 "hg", "hv", "k2", "nkk", "kka", "y", "y2", "att", "x1", "ln2", "mixed", "act", "cm", "r32", "d32", "k32",
                 "a32", "b32"]

    def debug_buffer(self, name, shape):
        """Host copy of one of the session's activation buffers (what the last layer of the last forward call
        left there): a parity tap for tests."""
        idx = self.DEBUG_IDS.index(name)
        p = ctypes.c_void_p(0)
        hip.check(hip.load().rwkv_hip_session_debug_buffer(self.handle, ctypes.c_int(idx), ctypes.byref(p)))
        dtype = np.float32 if name.endswith("32") else np.float16
        out = np.empty(shape, dtype)
        hip.check(hip.load().rwkv_hip_memcpy_d2h(out.ctypes.data_as(ctypes.c_void_p), p, ctypes.c_size_t(out.nbytes)))
        return out

    def set_fused_ln(self, on):
        """Decode steps fold LayerNorm + token shift into the linear launches: True always, False never, None (the
        default of a new session) for one or two rows of at most 4096 channels."""
        hip.check(hip.load().rwkv_hip_session_set_fused_ln(self.handle, ctypes.c_int(-1 if on is None else 1 if on else 0)))

    def set_tmix_rows(self, rows):
        """Decode steps' single-launch time-mix core: 1, 2 or 4 batch rows per block (always that launch), 0 never
        (the row-tiled kernels instead), None (the default of a new session) by batch size.  1, 2 and 4 give the same
        bits."""
        hip.check(hip.load().rwkv_hip_session_set_tmix_rows(self.handle, ctypes.c_int(-1 if rows is None else int(rows))))

    def set_wkv_fp16(self, on):
        """The state's WKV tensor is fp16 and the recurrence runs in fp16 (the reference's use_wkv32 == false)."""
        hip.check(hip.load().rwkv_hip_session_set_wkv_fp16(self.handle, ctypes.c_int(1 if on else 0)))

    def set_sparse_ffn(self, max_rows):
        """Decode steps of up to max_rows rows (0..12; True = 1, False = 0) read only the ffn.value rows with a
        non-zero activation (default 4; two to four rows share one walk over the rows any of them needs)."""
        hip.check(hip.load().rwkv_hip_session_set_sparse_ffn(self.handle, ctypes.c_int(int(max_rows))))

    def set_profile(self, mode):
        """0/False off; 1/True one event pair per linear launch; 2 passes launch the linear kernels only, back to
        back, one event pair per pass (state and logits are garbage afterwards)."""
        hip.check(hip.load().rwkv_hip_session_set_profile(self.handle, ctypes.c_int(int(mode))))

    def read_profile(self):
        """(launches, total_ms) of the event-bracketed linear launches since the last read."""
        n, ms = ctypes.c_int64(0), ctypes.c_double(0)
        hip.check(hip.load().rwkv_hip_session_read_profile(self.handle, ctypes.byref(n), ctypes.byref(ms)))
        return n.value, ms.value

    def forward(self, tokens, state, logits, sync=True):
        """tokens: int array [B,T].  Updates state in place, writes logits f32 [B,V] (last token per row)."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int64)
        B, T = tokens.shape
        if B != state.B:
            raise ValueError("state batch size mismatch")  # src/rwkv7_fast_v4.cu:1057-1059
        self.set_wkv_fp16(state.wkv_fp16)
        hip.check(hip.load().rwkv_hip_forward(self.handle, tokens.ctypes.data_as(ctypes.c_void_p), ctypes.c_int(B),
                                              ctypes.c_int(T), hip._p(state.shift), hip._p(state.wkv),
                                              hip._p(state.elapsed), hip._p(logits), ctypes.c_int(1 if sync else 0)))

    def decode_greedy(self, first_tokens, steps, state, logits):
        first = np.ascontiguousarray(first_tokens, dtype=np.int64)
        B = first.shape[0]
        self.set_wkv_fp16(state.wkv_fp16)
        out = np.zeros((steps, B), dtype=np.int32)
        hip.check(hip.load().rwkv_hip_decode_greedy(self.handle, first.ctypes.data_as(ctypes.c_void_p), ctypes.c_int(B),
                                                    ctypes.c_int(steps), hip._p(state.shift), hip._p(state.wkv),
                                                    hip._p(state.elapsed), hip._p(logits),
                                                    out.ctypes.data_as(ctypes.c_void_p)))
        return out

    def close(self):
        if self.handle:
            hip.load().rwkv_hip_session_destroy(self.handle)
            self.handle = None
