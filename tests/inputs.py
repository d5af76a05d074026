"""Seeded synthetic inputs shared by the CPU and GPU tests (shapes and distributions of the configs)."""
import numpy as np


def wkv_inputs(B, T, H, seed, dtype=np.float32):
    """Config-0 distributions: r,k,v ~ N(0,1); decay = exp(-exp(x)), x ~ U(-6,-0.5); kk = k/||k|| per head;
    a = -kk; b = kk * sigmoid(U(-3,3)).  Returns dict with both the decay and the equivalent raw logit."""
    rng = np.random.default_rng(seed)
    C = H * 64
    r = rng.standard_normal((B, T, C)).astype(np.float32)
    k = rng.standard_normal((B, T, C)).astype(np.float32)
    v = rng.standard_normal((B, T, C)).astype(np.float32)
    x = rng.uniform(-6.0, -0.5, (B, T, C))
    decay = np.exp(-np.exp(x)).astype(np.float32)
    # raw logit with exp(-e^-1/2 * sigmoid(w)) == decay  <=>  sigmoid(w) = exp(x + 1/2)
    s = np.exp(x + 0.5)
    w_raw = np.log(s / (1.0 - s)).astype(np.float32)
    kh = k.reshape(B, T, H, 64)
    kk = (kh / np.linalg.norm(kh, axis=-1, keepdims=True)).reshape(B, T, C).astype(np.float32)
    a = -kk
    b = (kk * (1.0 / (1.0 + np.exp(-rng.uniform(-3.0, 3.0, (B, T, C)))))).astype(np.float32)
    out = dict(r=r, k=k, v=v, decay=decay, w_raw=w_raw, a=a, b=b)
    return {n: t.astype(dtype) for n, t in out.items()}


def pattern_value(index, scale, bias):
    """The deterministic input pattern of the reference's kernel test (test/cuda_non4096_kernels_test.cpp:20-24)."""
    index = np.asarray(index)
    return (np.sin((index % 97).astype(np.float32) * np.float32(0.173)) * np.float32(scale)
            + np.cos((index % 53).astype(np.float32) * np.float32(0.071)) * np.float32(scale * 0.5)
            + np.float32(bias)).astype(np.float32)
