"""The entry point that allocates nothing (rwkv_hip_cmix_sparse_down_relu_rows_static) against the entry point it is
a variant of (rwkv_hip_cmix_sparse_down_relu_rows, partial rows in a caller's workspace): same kernels, so the
outputs must be bit-identical - on two calls in a row, the second smaller than the first (the built-in scratch
array keeps the first call's partial rows), and once more after the array has been used for another format."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _case(hip, orc, fmt, rows, C, F, seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((C, F)).astype(np.float32) * 0.05).astype(np.float16)
    pre = (rng.standard_normal((rows, F)).astype(np.float32)).astype(np.float16)   # about half the activations are zero
    dev = hip.DeviceArray.from_numpy
    scale = None
    if fmt == hip.FMT_F16:
        wt = hip.DeviceArray((C * F,), np.float16)
        hip.cmix_sparse_pack(fmt, C, F, dev(w), wt)
    elif fmt == hip.FMT_W8:
        q, s = orc.quantize_w8(w)
        scale = dev(s)
        wt = hip.DeviceArray((C * F,), np.int8)
        hip.cmix_sparse_pack(fmt, C, F, dev(q), wt)
    else:
        q, s, z = orc.quantize_w4(w)
        wt = hip.DeviceArray((hip.cmix_sparse_packed_bytes(hip.FMT_W4, C, F),), np.uint8)
        hip.cmix_sparse_pack_w4(C, F, dev(q), dev(s), dev(z), wt)
    ws = hip.DeviceArray.zeros((hip.cmix_sparse_workspace(C, F, rows),), np.uint8)
    want = hip.DeviceArray.zeros((rows, C), np.float16)
    got = hip.DeviceArray.zeros((rows, C), np.float16)
    pre_d = dev(pre)
    hip.cmix_sparse_down_relu_rows(fmt, rows, C, F, pre_d, wt, scale, ws, want)
    hip.cmix_sparse_down_relu_rows_static(fmt, rows, C, F, pre_d, wt, scale, got)
    hip.device_sync()
    w_, g_ = want.numpy(), got.numpy()
    assert np.abs(w_.astype(np.float32)).max() > 0
    same = np.array_equal(w_.view(np.uint16), g_.view(np.uint16))
    assert same, "fmt %d rows %d C %d F %d" % (fmt, rows, C, F)


def test_static_scratch_entry_point_matches_the_workspace_entry_point(gpu, orc):
    hip = gpu
    # two calls in a row, the second with a smaller input (fewer rows, narrower, shorter)
    _case(hip, orc, hip.FMT_W8, 5, 2048, 4096, seed=1)
    _case(hip, orc, hip.FMT_W8, 2, 1024, 1024, seed=2)
    # other formats reuse the same array
    _case(hip, orc, hip.FMT_F16, 3, 512, 2048, seed=3)
    _case(hip, orc, hip.FMT_W4, 1, 1024, 1024, seed=4)
    _case(hip, orc, hip.FMT_W8, 1, 4096, 16384, seed=5)   # the 7.2B shape's one-row step


def test_static_scratch_entry_point_rejects_what_does_not_fit(gpu):
    hip = gpu
    x = hip.DeviceArray.zeros((64,), np.float16)
    # 12 rows x (32768 / 256) x 8192 x 4 bytes = 48 MiB of partial rows > 16 MiB
    with pytest.raises(hip.RwkvHipError, match="built-in scratch holds"):
        hip.cmix_sparse_down_relu_rows_static(hip.FMT_W8, 12, 8192, 32768, x, x, x, x)
    with pytest.raises(hip.RwkvHipError, match="rows"):
        hip.cmix_sparse_down_relu_rows_static(hip.FMT_W8, 13, 1024, 1024, x, x, x, x)
    with pytest.raises(hip.RwkvHipError, match="unsupported"):
        hip.cmix_sparse_down_relu_rows_static(hip.FMT_W8, 1, 1000, 1000, x, x, x, x)
