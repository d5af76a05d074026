"""ctypes binding of the C ABI in include/rwkv_hip.h (librwkv_hip.so).

No torch involved: device memory comes from rwkv_hip_malloc and moves through numpy arrays.
Every call raises RwkvHipError with the library's message on a non-zero return code.  There is
no CPU fallback: if the library is missing, loading raises.
"""
import ctypes
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "librwkv_hip.so")

FMT_F16, FMT_W8, FMT_W4 = 0, 1, 2
W_RAW_LOGIT, W_DECAY = 0, 1
IO_F16, IO_F32 = 0, 1
ACT_NONE, ACT_TANH, ACT_SIGMOID = 0, 1, 2
EPI_NONE, EPI_RELU_SQUARE = 0, 1

# tensor / matrix ids (rwkv_hip.h)
T_EMB_LN0, T_LN_OUT_W, T_LN_OUT_B = 0, 1, 2
(T_LN1_W, T_LN1_B, T_LN2_W, T_LN2_B, T_X_R, T_X_W, T_X_K, T_X_V, T_X_A, T_X_G, T_W0, T_A0, T_V0, T_K_K, T_K_A,
 T_R_K, T_LNX_W, T_LNX_B, T_FFN_X_K) = range(10, 29)
T_W1, T_W2, T_A1, T_A2, T_G1, T_G2, T_V1, T_V2 = range(40, 48)
M_ATT_R, M_ATT_K, M_ATT_V, M_ATT_O, M_FFN_KEY, M_FFN_VALUE, M_HEAD = range(7)

# every symbol include/rwkv_hip.h declares; checked at load time and by the CPU test-suite
EXPORTS = [
    "rwkv_hip_last_error", "rwkv_hip_device_count", "rwkv_hip_device_name", "rwkv_hip_malloc", "rwkv_hip_free",
    "rwkv_hip_malloc_recycled", "rwkv_hip_free_recycled", "rwkv_hip_recycle_trim", "rwkv_hip_graph_capture_count",
    "rwkv_hip_host_alloc", "rwkv_hip_host_free", "rwkv_hip_memcpy_h2d", "rwkv_hip_memcpy_d2h", "rwkv_hip_memcpy_d2d",
    "rwkv_hip_memcpy_h2d_async", "rwkv_hip_memcpy_d2h_async", "rwkv_hip_memcpy_d2d_async", "rwkv_hip_memset",
    "rwkv_hip_mem_info", "rwkv_hip_stream_create", "rwkv_hip_stream_destroy", "rwkv_hip_stream_sync",
    "rwkv_hip_device_sync", "rwkv_hip_event_create", "rwkv_hip_event_destroy", "rwkv_hip_event_record",
    "rwkv_hip_event_sync", "rwkv_hip_stream_wait_event",
    "rwkv_hip_event_elapsed_ms", "rwkv_hip_measure_launch_chain", "rwkv_hip_wkv7", "rwkv_hip_wkv7_f16state", "rwkv_hip_quantize_w8", "rwkv_hip_dequant_w8",
    "rwkv_hip_quantize_w4", "rwkv_hip_dequant_w4", "rwkv_hip_bf16_to_f16", "rwkv_hip_bf16_to_f16_transpose",
    "rwkv_hip_emb_ln0_bf16_to_f16", "rwkv_hip_fill_normal_f16", "rwkv_hip_linear",
    "rwkv_hip_pack_weights", "rwkv_hip_linear_packed_workspace", "rwkv_hip_linear_packed", "rwkv_hip_lora_in", "rwkv_hip_lora_out",
    "rwkv_hip_cmix_sparse_pack", "rwkv_hip_cmix_sparse_pack_w4", "rwkv_hip_cmix_sparse_packed_bytes",
    "rwkv_hip_cmix_sparse_workspace", "rwkv_hip_cmix_sparse_down_relu_one",
    "rwkv_hip_cmix_sparse_down_relu_rows", "rwkv_hip_cmix_sparse_down_relu_rows_static",
    "rwkv_hip_cmix_sparse_down_relu_rows_shared",
    "rwkv_hip_session_set_sparse_ffn", "rwkv_hip_session_set_fused_ln", "rwkv_hip_session_set_tmix_rows", "rwkv_hip_session_set_wkv_fp16",
    "rwkv_hip_layer_norm", "rwkv_hip_add_layer_norm", "rwkv_hip_add_last_layer_norm", "rwkv_hip_token_shift_mix",
    "rwkv_hip_add_layer_norm_cmix_mix", "rwkv_hip_add_layer_norm_tmix_mix6", "rwkv_hip_kk_a_gate",
    "rwkv_hip_lnx_rkvres_xg", "rwkv_hip_relu_square", "rwkv_hip_add_vec", "rwkv_hip_f16_to_f32",
    "rwkv_hip_advance_i32", "rwkv_hip_sample", "rwkv_hip_argmax", "rwkv_hip_model_create", "rwkv_hip_model_destroy",
    "rwkv_hip_model_set_tensor", "rwkv_hip_model_set_matrix", "rwkv_hip_model_weight_bytes",
    "rwkv_hip_session_debug_buffer",
    "rwkv_hip_session_create", "rwkv_hip_session_destroy", "rwkv_hip_session_stream", "rwkv_hip_session_set_graph",
    "rwkv_hip_session_set_trace", "rwkv_hip_session_set_profile", "rwkv_hip_session_read_profile", "rwkv_hip_forward", "rwkv_hip_decode_greedy",
]


class RwkvHipError(RuntimeError):
    pass


_lib = None


def load():
    """Loads librwkv_hip.so (raises if it has not been built) and returns the ctypes handle."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RwkvHipError(
            "%s not found: build it with `python -m rwkv_lightning_cuda_amd.build` (there is no CPU fallback)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    missing = [s for s in EXPORTS if not hasattr(lib, s)]
    if missing:
        raise RwkvHipError("librwkv_hip.so lacks symbols: %s" % ", ".join(missing))
    lib.rwkv_hip_last_error.restype = ctypes.c_char_p
    _lib = lib
    return lib


def _p(x):
    """Device pointer of a DeviceArray / int / None as c_void_p."""
    if x is None:
        return ctypes.c_void_p(0)
    if isinstance(x, DeviceArray):
        return ctypes.c_void_p(x.ptr)
    return ctypes.c_void_p(int(x))


def check(rc):
    if rc != 0:
        raise RwkvHipError("rwkv_hip error %d: %s" % (rc, load().rwkv_hip_last_error().decode()))


def device_count():
    n = ctypes.c_int(0)
    check(load().rwkv_hip_device_count(ctypes.byref(n)))
    return n.value


def device_name():
    buf = ctypes.create_string_buffer(256)
    check(load().rwkv_hip_device_name(buf, ctypes.c_size_t(256)))
    return buf.value.decode()


def device_sync():
    check(load().rwkv_hip_device_sync())


def mem_info():
    f, t = ctypes.c_size_t(0), ctypes.c_size_t(0)
    check(load().rwkv_hip_mem_info(ctypes.byref(f), ctypes.byref(t)))
    return f.value, t.value


class DeviceArray:
    """A device allocation with a numpy dtype and shape.  fp16 tensors use dtype float16."""

    def __init__(self, shape, dtype):
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = ctypes.c_void_p(0)
        check(load().rwkv_hip_malloc(ctypes.byref(p), ctypes.c_size_t(self.nbytes)))
        self.ptr = p.value or 0
        self._owner = True

    @classmethod
    def from_numpy(cls, arr):
        arr = np.ascontiguousarray(arr)
        d = cls(arr.shape, arr.dtype)
        d.upload(arr)
        return d

    @classmethod
    def zeros(cls, shape, dtype):
        d = cls(shape, dtype)
        d.fill0()
        return d

    def fill0(self):
        if self.nbytes:
            check(load().rwkv_hip_memset(_p(self), 0, ctypes.c_size_t(self.nbytes)))

    def upload(self, arr):
        arr = np.ascontiguousarray(arr, dtype=self.dtype)
        assert arr.nbytes == self.nbytes, (arr.shape, self.shape)
        if self.nbytes:
            check(load().rwkv_hip_memcpy_h2d(_p(self), arr.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(self.nbytes)))

    def numpy(self):
        out = np.empty(self.shape, dtype=self.dtype)
        if self.nbytes:
            check(load().rwkv_hip_memcpy_d2h(out.ctypes.data_as(ctypes.c_void_p), _p(self), ctypes.c_size_t(self.nbytes)))
        return out

    def copy_from(self, other):
        assert other.nbytes == self.nbytes
        check(load().rwkv_hip_memcpy_d2d(_p(self), _p(other), ctypes.c_size_t(self.nbytes)))

    def view(self, offset_elems, shape, dtype=None):
        """A non-owning sub-array starting offset_elems elements in."""
        v = object.__new__(DeviceArray)
        v.dtype = np.dtype(dtype) if dtype is not None else self.dtype
        v.shape = tuple(shape)
        v.nbytes = int(np.prod(v.shape, dtype=np.int64)) * v.dtype.itemsize
        v.ptr = self.ptr + offset_elems * self.dtype.itemsize
        v._owner = False
        v._base = self
        return v

    def free(self):
        if getattr(self, "_owner", False) and self.ptr:
            load().rwkv_hip_free(ctypes.c_void_p(self.ptr))
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _i(x):
    return ctypes.c_int(int(x))


def _ptr_array(items):
    arr = (ctypes.c_void_p * len(items))()
    for i, it in enumerate(items):
        arr[i] = it.ptr if isinstance(it, DeviceArray) else int(it)
    return arr


# ---- ops --------------------------------------------------------------------------------------------
def wkv7(B, T, C, H, w_mode, io, state, r, w, k, v, a, b, y, stream=None):
    check(load().rwkv_hip_wkv7(_p(stream), _i(B), _i(T), _i(C), _i(H), _i(w_mode), _i(io), _p(state), _p(r), _p(w),
                               _p(k), _p(v), _p(a), _p(b), _p(y)))


def wkv7_f16state(B, T, C, H, state, r, w, k, v, a, b, y, elapsed, w0=None, stream=None):
    """The recurrence with an fp16 state [B,H,64,64]; w raw decay logits, w0 [C] or None, elapsed int32 [B]."""
    check(load().rwkv_hip_wkv7_f16state(_p(stream), _i(B), _i(T), _i(C), _i(H), _p(state), _p(r), _p(w), _p(w0), _p(k),
                                        _p(v), _p(a), _p(b), _p(y), _p(elapsed)))


def bf16_to_f16(n, src, dst, stream=None):
    check(load().rwkv_hip_bf16_to_f16(_p(stream), ctypes.c_int64(n), _p(src), _p(dst)))


def bf16_to_f16_transpose(rows, cols, src, dst, stream=None):
    check(load().rwkv_hip_bf16_to_f16_transpose(_p(stream), _i(rows), _i(cols), _p(src), _p(dst)))


def emb_ln0_bf16_to_f16(V, C, emb, weight, bias, eps, out, stream=None):
    check(load().rwkv_hip_emb_ln0_bf16_to_f16(_p(stream), _i(V), _i(C), _p(emb), _p(weight), _p(bias),
                                              ctypes.c_float(eps), _p(out)))


def quantize_w8(N, K, w, q, scale, stream=None):
    check(load().rwkv_hip_quantize_w8(_p(stream), _i(N), _i(K), _p(w), _p(q), _p(scale)))


def dequant_w8(N, K, q, scale, w, stream=None):
    check(load().rwkv_hip_dequant_w8(_p(stream), _i(N), _i(K), _p(q), _p(scale), _p(w)))


def quantize_w4(N, K, w, q, scale, zp, stream=None):
    check(load().rwkv_hip_quantize_w4(_p(stream), _i(N), _i(K), _p(w), _p(q), _p(scale), _p(zp)))


def dequant_w4(N, K, q, scale, zp, w, stream=None):
    check(load().rwkv_hip_dequant_w4(_p(stream), _i(N), _i(K), _p(q), _p(scale), _p(zp), _p(w)))


def fill_normal_f16(n, seed, mean, std, out, stream=None):
    check(load().rwkv_hip_fill_normal_f16(_p(stream), ctypes.c_int64(n), ctypes.c_uint64(seed), ctypes.c_float(mean),
                                          ctypes.c_float(std), _p(out)))


def linear(fmt, M, N, K, x, w, scale, zp, y, epilogue=EPI_NONE, out_f32=0, stream=None):
    check(load().rwkv_hip_linear(_p(stream), _i(fmt), _i(M), _i(N), _i(K), _p(x), _p(w), _p(scale), _p(zp),
                                 _i(epilogue), _i(out_f32), _p(y)))


def pack_weights(fmt, N, K, w, packed, stream=None):
    check(load().rwkv_hip_pack_weights(_p(stream), _i(fmt), _i(N), _i(K), _p(w), _p(packed)))


def linear_packed_workspace(M, N, K):
    n = ctypes.c_size_t(0)
    check(load().rwkv_hip_linear_packed_workspace(_i(M), _i(N), _i(K), ctypes.byref(n)))
    return n.value


def linear_packed(fmt, M, N, K, x, packed, scale, zp, y, workspace, epilogue=EPI_NONE, out_f32=0, stream=None):
    check(load().rwkv_hip_linear_packed(_p(stream), _i(fmt), _i(M), _i(N), _i(K), _p(x), _p(packed), _p(scale), _p(zp),
                                        _i(epilogue), _i(out_f32), _p(y), _p(workspace),
                                        ctypes.c_size_t(workspace.nbytes if workspace is not None else 0)))


def lora_in(M, C, R, x, w1, h, stream=None):
    check(load().rwkv_hip_lora_in(_p(stream), _i(M), _i(C), _i(R), _p(x), _p(w1), _p(h)))


def cmix_sparse_pack(fmt, C, F, w, wt, stream=None):
    check(load().rwkv_hip_cmix_sparse_pack(_p(stream), _i(fmt), _i(C), _i(F), _p(w), _p(wt)))


def cmix_sparse_pack_w4(C, F, q, scale, zp, wt, stream=None):
    check(load().rwkv_hip_cmix_sparse_pack_w4(_p(stream), _i(C), _i(F), _p(q), _p(scale), _p(zp), _p(wt)))


def cmix_sparse_packed_bytes(fmt, C, F):
    n = ctypes.c_size_t(0)
    check(load().rwkv_hip_cmix_sparse_packed_bytes(_i(fmt), _i(C), _i(F), ctypes.byref(n)))
    return n.value


def cmix_sparse_workspace(C, F, rows=1):
    n = ctypes.c_size_t(0)
    check(load().rwkv_hip_cmix_sparse_workspace(_i(rows), _i(C), _i(F), ctypes.byref(n)))
    return n.value


def cmix_sparse_down_relu_one(fmt, C, F, preact, wt, scale, workspace, out, stream=None):
    check(load().rwkv_hip_cmix_sparse_down_relu_one(_p(stream), _i(fmt), _i(C), _i(F), _p(preact), _p(wt), _p(scale),
                                                    _p(workspace), ctypes.c_size_t(workspace.nbytes), _p(out)))


def cmix_sparse_down_relu_rows(fmt, rows, C, F, preact, wt, scale, workspace, out, stream=None):
    check(load().rwkv_hip_cmix_sparse_down_relu_rows(_p(stream), _i(fmt), _i(rows), _i(C), _i(F), _p(preact), _p(wt),
                                                     _p(scale), _p(workspace), ctypes.c_size_t(workspace.nbytes), _p(out)))


def cmix_sparse_down_relu_rows_shared(fmt, rows, C, F, preact, wt, scale, workspace, out, stream=None):
    """2..4 tokens in one walk over the rows that are non-zero for any of them."""
    check(load().rwkv_hip_cmix_sparse_down_relu_rows_shared(_p(stream), _i(fmt), _i(rows), _i(C), _i(F), _p(preact),
                                                            _p(wt), _p(scale), _p(workspace),
                                                            ctypes.c_size_t(workspace.nbytes), _p(out)))


def measure_launch_chain(links, blocks=1, threads=64, use_graph=True, reps=20):
    """Microseconds per link of a chain of dependent launches of a near-empty kernel."""
    us = ctypes.c_float(0)
    check(load().rwkv_hip_measure_launch_chain(_i(links), _i(blocks), _i(threads), _i(1 if use_graph else 0), _i(reps),
                                               ctypes.byref(us)))
    return us.value


def cmix_sparse_down_relu_rows_static(fmt, rows, C, F, preact, wt, scale, out, stream=None):
    """The product above with the partial rows in the library's built-in scratch array: allocates nothing."""
    check(load().rwkv_hip_cmix_sparse_down_relu_rows_static(_p(stream), _i(fmt), _i(rows), _i(C), _i(F), _p(preact),
                                                            _p(wt), _p(scale), _p(out)))


def lora_out(M, C, R, act, h, w2, out, bias=None, vres=0, v=None, v_first=None, stream=None):
    check(load().rwkv_hip_lora_out(_p(stream), _i(M), _i(C), _i(R), _i(act), _p(h), _p(w2), _p(bias), _i(vres), _p(v),
                                   _p(v_first), _p(out)))


def layer_norm(rows, C, x, w, b, y, eps=1e-5, stream=None):
    check(load().rwkv_hip_layer_norm(_p(stream), _i(rows), _i(C), _p(x), _p(w), _p(b), _p(y), ctypes.c_float(eps)))


def add_layer_norm(rows, C, x, res, w, b, x_out, y, eps=1e-5, stream=None):
    check(load().rwkv_hip_add_layer_norm(_p(stream), _i(rows), _i(C), _p(x), _p(res), _p(w), _p(b), _p(x_out), _p(y),
                                         ctypes.c_float(eps)))


def add_last_layer_norm(B, T, C, x, res, w, b, y, eps=1e-5, stream=None):
    check(load().rwkv_hip_add_last_layer_norm(_p(stream), _i(B), _i(T), _i(C), _p(x), _p(res), _p(w), _p(b), _p(y),
                                              ctypes.c_float(eps)))


def token_shift_mix(B, T, C, x, shift, mus, outs, stream=None):
    check(load().rwkv_hip_token_shift_mix(_p(stream), _i(B), _i(T), _i(C), _i(len(mus)), _p(x), _p(shift),
                                          _ptr_array(mus), _ptr_array(outs)))


def add_layer_norm_cmix_mix(rows, C, x, res, shift, w, b, mu_k, x_out, mixed, eps=1e-5, stream=None):
    check(load().rwkv_hip_add_layer_norm_cmix_mix(_p(stream), _i(rows), _i(C), _p(x), _p(res), _p(shift), _p(w), _p(b),
                                                  _p(mu_k), _p(x_out), _p(mixed), ctypes.c_float(eps)))


def add_layer_norm_tmix_mix6(rows, C, x, res, shift, w, b, mus, x_out, outs, eps=1e-5, stream=None):
    check(load().rwkv_hip_add_layer_norm_tmix_mix6(_p(stream), _i(rows), _i(C), _p(x), _p(res), _p(shift), _p(w), _p(b),
                                                   _ptr_array(mus), _p(x_out), _ptr_array(outs), ctypes.c_float(eps)))


def kk_a_gate(rows, C, H, k, k_k, a0, a12, k_a, new_k, neg_kk, kka, stream=None):
    check(load().rwkv_hip_kk_a_gate(_p(stream), _i(rows), _i(C), _i(H), _p(k), _p(k_k), _p(a0), _p(a12), _p(k_a),
                                    _p(new_k), _p(neg_kk), _p(kka)))


def lnx_rkvres_xg(rows, C, H, y, r, k, v, r_k, lnw, lnb, g, out, stream=None):
    check(load().rwkv_hip_lnx_rkvres_xg(_p(stream), _i(rows), _i(C), _i(H), _p(y), _p(r), _p(k), _p(v), _p(r_k),
                                        _p(lnw), _p(lnb), _p(g), _p(out)))


def relu_square(n, x, out, stream=None):
    check(load().rwkv_hip_relu_square(_p(stream), ctypes.c_int64(n), _p(x), _p(out)))


def add_vec(rows, C, x, vec, out, stream=None):
    check(load().rwkv_hip_add_vec(_p(stream), _i(rows), _i(C), _p(x), _p(vec), _p(out)))


def f16_to_f32(n, src, dst, stream=None):
    check(load().rwkv_hip_f16_to_f32(_p(stream), ctypes.c_int64(n), _p(src), _p(dst)))


def advance_i32(n, amount, x, stream=None):
    check(load().rwkv_hip_advance_i32(_p(stream), _i(n), _i(amount), _p(x)))


def sample(B, V, logits, penalties, probs, out, presence=0.0, frequency=0.0, decay=1.0, temperature=1.0, top_k=0,
           top_p=1.0, seed=0, step=0, stream=None):
    check(load().rwkv_hip_sample(_p(stream), _i(B), _i(V), _p(logits), _p(penalties), _p(probs), _p(out),
                                 ctypes.c_double(presence), ctypes.c_double(frequency), ctypes.c_double(decay),
                                 ctypes.c_double(temperature), _i(top_k), ctypes.c_double(top_p),
                                 ctypes.c_uint64(seed), ctypes.c_uint64(step)))


def argmax(B, V, logits, out, stream=None):
    check(load().rwkv_hip_argmax(_p(stream), _i(B), _i(V), _p(logits), _p(out)))


class Event:
    def __init__(self):
        p = ctypes.c_void_p(0)
        check(load().rwkv_hip_event_create(ctypes.byref(p)))
        self.ptr = p.value

    def record(self, stream=None):
        check(load().rwkv_hip_event_record(ctypes.c_void_p(self.ptr), _p(stream)))

    def elapsed_ms(self, stop):
        ms = ctypes.c_float(0)
        check(load().rwkv_hip_event_elapsed_ms(ctypes.c_void_p(self.ptr), ctypes.c_void_p(stop.ptr), ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            load().rwkv_hip_event_destroy(ctypes.c_void_p(self.ptr))
        except Exception:
            pass
