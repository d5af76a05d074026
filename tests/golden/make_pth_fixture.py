"""Writes a small RWKV-7-shaped checkpoint with torch.save and, beside it, a manifest of what went in.

    python tests/golden/make_pth_fixture.py [out.pth [out.manifest]]      (default: tests/golden/rwkv7_tiny.*)

The checkpoint is what the checkpoint reader has to understand: a zip written by torch.save (stored members, 64-byte
aligned), bf16 tensors under the x070 names, an OrderedDict carrying `_metadata` (a BUILD opcode), two tensors that
are views into one storage at different offsets, one non-contiguous tensor, and one tensor of special values
(subnormals, infinities, a NaN, signed zeros, magnitudes beyond fp16).  The manifest holds, per tensor in state-dict
order, name, shape, stride, storage offset and the bf16 bit patterns in logical order - taken from the tensors
themselves, not from the file.

    manifest := "PTHM" u32 count { u32 len, name, u32 rank, i64 shape[rank], i64 stride[rank], u64 offset, u64 n, u16 bits[n] }
"""
import collections
import os
import struct
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def tiny_dims():
    return dict(L=2, C=64, H=1, F=128, V=32, Rw=16, Ra=16, Rg=16, Rv=16)


def state_dict(dims, seed=1234):
    """name -> bf16 tensor, in the order an RWKV-7 (x070) checkpoint lists them."""
    g = torch.Generator().manual_seed(seed)
    L, C, H, F, V = dims["L"], dims["C"], dims["H"], dims["F"], dims["V"]

    def normal(shape, mean=0.0, std=0.02):
        return (torch.randn(shape, generator=g) * std + mean).to(torch.bfloat16)

    sd = collections.OrderedDict()
    sd["emb.weight"] = normal((V, C), 0.0, 1.0)
    for l in range(L):
        p = "blocks.%d." % l
        if l == 0:
            sd[p + "ln0.weight"] = normal((C,), 1.0, 0.05)
            sd[p + "ln0.bias"] = normal((C,), 0.0, 0.05)
        for n in ("ln1", "ln2"):
            sd[p + n + ".weight"] = normal((C,), 1.0, 0.02)
            sd[p + n + ".bias"] = normal((C,), 0.0, 0.02)
        for n in ("x_r", "x_w", "x_k", "x_v", "x_a", "x_g"):
            sd[p + "att." + n] = normal((1, 1, C), 0.5, 0.15)
        sd[p + "att.w0"] = normal((1, 1, C), -2.0, 1.5)
        sd[p + "att.w1"] = normal((C, dims["Rw"]), 0.0, 0.08)
        sd[p + "att.w2"] = normal((dims["Rw"], C), 0.0, 0.08)
        sd[p + "att.a0"] = normal((1, 1, C), 0.0, 0.02)
        sd[p + "att.a1"] = normal((C, dims["Ra"]), 0.0, 0.08)
        sd[p + "att.a2"] = normal((dims["Ra"], C), 0.0, 0.08)
        sd[p + "att.v0"] = normal((1, 1, C), 0.0, 0.02)
        sd[p + "att.v1"] = normal((C, dims["Rv"]), 0.0, 0.08)
        sd[p + "att.v2"] = normal((dims["Rv"], C), 0.0, 0.08)
        sd[p + "att.g1"] = normal((C, dims["Rg"]), 0.0, 0.08)
        sd[p + "att.g2"] = normal((dims["Rg"], C), 0.0, 0.08)
        sd[p + "att.k_k"] = normal((1, 1, C), 1.0, 0.02)
        sd[p + "att.k_a"] = normal((1, 1, C), 1.0, 0.02)
        sd[p + "att.r_k"] = normal((H, C // H), 0.0, 0.02)
        for n in ("receptance", "key", "value", "output"):
            sd[p + "att." + n + ".weight"] = normal((C, C))
        sd[p + "att.ln_x.weight"] = normal((C,), 1.0, 0.02)
        sd[p + "att.ln_x.bias"] = normal((C,), 0.0, 0.02)
        sd[p + "ffn.x_k"] = normal((1, 1, C), 0.5, 0.15)
        sd[p + "ffn.key.weight"] = normal((F, C))
        sd[p + "ffn.value.weight"] = normal((C, F))
    sd["ln_out.weight"] = normal((C,), 1.0, 0.02)
    sd["ln_out.bias"] = normal((C,), 0.0, 0.02)
    sd["head.weight"] = normal((V, C))
    return sd


def reader_stress_entries():
    """Extra tensors that exercise the reader (not part of a model): shared storage, strides, special values."""
    base = torch.arange(48, dtype=torch.float32).to(torch.bfloat16)
    special = torch.tensor([0.0, -0.0, 1.0, -1.0, 65504.0, 65536.0, -1.0e6, float("inf"), float("-inf"), float("nan"),
                            2.0 ** -14, 2.0 ** -15, 3 * 2.0 ** -25, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -24, 1.0e-30,
                            -(2.0 ** -20)], dtype=torch.float32).to(torch.bfloat16)
    extra = collections.OrderedDict()
    extra["stress.view_head"] = base[:16].view(4, 4)
    extra["stress.view_tail"] = base[20:44].view(2, 3, 4)          # same storage, offset 20
    extra["stress.transposed"] = torch.arange(24, dtype=torch.float32).to(torch.bfloat16).view(4, 6).t()  # strides (1, 6)
    extra["stress.special"] = special
    extra["stress.empty"] = torch.zeros((0, 5), dtype=torch.bfloat16)
    extra["stress.scalar"] = torch.tensor(3.25, dtype=torch.bfloat16)
    return extra


def bits_in_logical_order(t):
    return t.contiguous().view(torch.int16).numpy().astype(np.uint16).reshape(-1)


def write_manifest(path, sd):
    with open(path, "wb") as f:
        f.write(b"PTHM")
        f.write(struct.pack("<I", len(sd)))
        for name, t in sd.items():
            nm = name.encode()
            f.write(struct.pack("<I", len(nm)) + nm)
            f.write(struct.pack("<I", t.dim()))
            f.write(struct.pack("<%dq" % t.dim(), *t.shape))
            f.write(struct.pack("<%dq" % t.dim(), *t.stride()))
            bits = bits_in_logical_order(t)
            f.write(struct.pack("<QQ", t.storage_offset(), bits.size))
            f.write(bits.astype("<u2").tobytes())


def write_checkpoint(pth_path, manifest_path, sd, with_metadata=True):
    out = collections.OrderedDict(sd)
    if with_metadata:   # what nn.Module.state_dict() attaches: pickled with a BUILD opcode
        out._metadata = collections.OrderedDict([("", {"version": 1}), ("blocks.0", {"version": 1})])
    torch.save(out, pth_path)
    write_manifest(manifest_path, sd)


def load_rate_dims(layers=4):
    """The 7.2B shape cut to a few layers: full-size embedding, head and per-layer tensors (0.43 GB a layer + 1.07 GB),
    for timing the checkpoint loader - ModelBackend prints the rate it reached."""
    return dict(L=layers, C=4096, H=64, F=16384, V=65536, Rw=128, Ra=128, Rg=480, Rv=96)


def main():
    if len(sys.argv) > 2 and sys.argv[1] == "--load-rate":
        # python make_pth_fixture.py --load-rate OUT.pth [LAYERS]: no manifest, no stress entries
        sd = state_dict(load_rate_dims(int(sys.argv[3]) if len(sys.argv) > 3 else 4), seed=3)
        torch.save(sd, sys.argv[2])
        print("wrote %s (%.2f GB)" % (sys.argv[2], os.path.getsize(sys.argv[2]) / 1e9))
        return
    pth = sys.argv[1] if len(sys.argv) > 1 else os.path.join(HERE, "rwkv7_tiny.pth")
    manifest = sys.argv[2] if len(sys.argv) > 2 else os.path.join(HERE, "rwkv7_tiny.manifest")
    sd = state_dict(tiny_dims())
    sd.update(reader_stress_entries())
    write_checkpoint(pth, manifest, sd)
    print("wrote %s (%d bytes) and %s (%d tensors), torch %s" % (pth, os.path.getsize(pth), manifest, len(sd), torch.__version__))


if __name__ == "__main__":
    main()
