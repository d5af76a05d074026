"""MI355X (gfx950) RWKV-7 inference kernels behind a C ABI, with a thin ctypes/numpy host layer.

  hip    -- ctypes binding of include/rwkv_hip.h (librwkv_hip.so); no CPU fallback
  model  -- model shapes, synthetic weights, device upload with quantise-on-load, sessions
  build  -- builds librwkv_hip.so in-tree with hipcc
"""
__all__ = ["hip", "model", "build"]
