"""Writes tests/golden/*.npz: inputs and outputs of the REFERENCE CPU backend.

Run where oracle/_ref/libiom_ref.so has been built from the reference's own
sources (`make -C oracle ref`):

    python tests/golden/make_golden.py

Every fixture holds raw leaf bit patterns only (inputs in logical row-major
order, view recipes as plain tuples, outputs as the owner's logical content
and its raw tiled storage).  The reference is driven through its public
Device / TensorView / DeviceOps API; nothing of its source is stored.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [os.path.join(ROOT, "oracle"), os.path.join(ROOT, "tests")]

import datagen  # noqa: E402
import iomo  # noqa: E402
from iomo import DT_BF16, DT_F32, DT_I32  # noqa: E402

BITS = {DT_BF16: 16, DT_F32: 32, DT_I32: 32}


def apply(view, steps):
    for name, args in steps:
        view = getattr(view, name)(*args)
    return view


def directed_bits(dtype):
    """Special encodings every elementwise op must get right."""
    if dtype == DT_I32:
        return np.array([0, 1, 0xFFFFFFFF, 0x80000000, 0x7FFFFFFF, 3, 0x00100000, 0xFFF00000],
                        np.uint32)
    if dtype == DT_F32:
        return np.array([0, 0x80000000, 0x3F800000, 0xBF800000, 0x7F800000, 0xFF800000,
                         0x7FC00000, 0xFFC12345, 0x7F7FFFFF, 0xFF7FFFFF, 0x00000001, 0x80000001,
                         0x007FFFFF, 0x00800000, 0x3F000000, 0x40000000, 0x1FFFFFFF, 0x20000000,
                         0x33800000, 0x4B000001], np.uint32)
    return np.array([0, 0x8000, 0x3F80, 0xBF80, 0x7F80, 0xFF80, 0x7FC0, 0xFFFF, 0x7F7F, 0xFF7F,
                     0x0001, 0x8001, 0x007F, 0x0080, 0x3F00, 0x4000, 0x1FC0, 0x2000, 0x1F81,
                     0x3F81, 0x4301, 0x0040], np.uint16)


def main():
    ref = iomo.ref_backend()
    out = {}
    manifest = []

    # --- binary: directed cross product and hashed views -----------------------
    for dtype in (DT_I32, DT_F32, DT_BF16):
        d = directed_bits(dtype)
        n = d.size
        A = np.repeat(d, n).reshape(1, n, n)
        B = np.tile(d, n).reshape(1, n, n)
        for op in (0, 1, 2):
            ta, tb, to = (ref.tensor(dtype, (1, n, n)) for _ in range(3))
            ta.view().from_host(A)
            tb.view().from_host(B)
            assert ref.binary(op, ta.view(), tb.view(), to.view()) > 0
            key = f"binary_directed_dt{dtype}_op{op}"
            out[key + "_a"], out[key + "_b"] = A, B
            out[key + "_y"] = to.view().to_host()
            manifest.append({"kind": "binary_directed", "key": key, "dtype": dtype, "op": op,
                             "dims": [1, n, n]})
    view_cases = [
        ((2, 1, 33), [], (1, 17, 1), [], (2, 17, 33), []),
        ((3, 32, 48), [], (1, 48), [], (3, 32, 48), []),
        ((6, 20, 35), [("slice", (0, 1, 3, 2))], (3, 20, 35), [], (3, 20, 35), []),
        ((4, 3, 16, 32), [("permute", ([1, 0],))], (3, 4, 16, 32), [], (3, 4, 16, 32), []),
        ((4, 3, 16, 32), [("select", (0, 2))], (1, 16, 32), [], (5, 3, 16, 32), [("select", (0, 4))]),
    ]
    for ci, (ld, ls, rd, rs, od, os_) in enumerate(view_cases):
        for dtype in (DT_I32, DT_F32, DT_BF16):
            for op in (0, 1, 2):
                A = datagen.pattern_bits(BITS[dtype], int(np.prod(ld)), 0x100 + ci).reshape(ld)
                B = datagen.pattern_bits(BITS[dtype], int(np.prod(rd)), 0x200 + ci).reshape(rd)
                O = datagen.pattern_bits(BITS[dtype], int(np.prod(od)), 0x300 + ci).reshape(od)
                ta, tb, to = ref.tensor(dtype, ld), ref.tensor(dtype, rd), ref.tensor(dtype, od)
                ta.view().from_host(A)
                tb.view().from_host(B)
                to.view().from_host(O)
                assert ref.binary(op, apply(ta.view(), ls), apply(tb.view(), rs),
                                  apply(to.view(), os_)) > 0
                key = f"binary_view{ci}_dt{dtype}_op{op}"
                out[key + "_y"] = to.view().to_host()
                manifest.append({"kind": "binary_view", "key": key, "dtype": dtype, "op": op,
                                 "lhs": [list(ld), ls, 0x100 + ci],
                                 "rhs": [list(rd), rs, 0x200 + ci],
                                 "out": [list(od), os_, 0x300 + ci]})

    # --- rmsnorm / silu --------------------------------------------------------
    for dtype in (DT_BF16, DT_F32):
        for (R, F) in ((17, 33), (4, 2048), (16, 256)):
            x = datagen.normal_f32(R * F, 0, 1, 7)
            x = x.reshape(R, F)
            x[1] *= 50
            w = datagen.uniform_f32(F, 0.5, 1.5, 8)
            if dtype == DT_BF16:
                xl, wl = datagen.bf16_rne(x), datagen.bf16_rne(w)
            else:
                xl, wl = x.view(np.uint32), w.view(np.uint32)
            tx, tw, to = ref.tensor(dtype, (R, F)), ref.tensor(dtype, (1, F)), ref.tensor(dtype, (R, F))
            tx.view().from_host(xl)
            tw.view().from_host(wl.reshape(1, F))
            assert ref.rmsnorm(tx.view(), tw.view(), to.view(), 1e-5) > 0
            key = f"rmsnorm_dt{dtype}_{R}x{F}"
            out[key + "_x"], out[key + "_w"], out[key + "_y"] = xl, wl, to.view().to_host()
            manifest.append({"kind": "rmsnorm", "key": key, "dtype": dtype, "dims": [R, F],
                             "eps": 1e-5})
        # SiLU: every BF16 encoding; a hashed + directed sample for F32
        if dtype == DT_BF16:
            xl = np.arange(65536, dtype=np.uint16).reshape(256, 256)
        else:
            xs = np.concatenate([
                datagen.pattern_bits(32, 16 * 1024 - 64, 9),
                np.linspace(-110, 90, 64).astype(np.float32).view(np.uint32)])
            xl = xs.reshape(64, 256)
        tx, to = ref.tensor(dtype, xl.shape), ref.tensor(dtype, xl.shape)
        tx.view().from_host(xl)
        assert ref.silu(tx.view(), to.view()) > 0
        key = f"silu_dt{dtype}"
        out[key + "_x"], out[key + "_y"] = xl, to.view().to_host()
        manifest.append({"kind": "silu", "key": key, "dtype": dtype, "dims": list(xl.shape)})

    ref.close()
    np.savez_compressed(os.path.join(HERE, "reference_cpu_vectors.npz"), **out)
    with open(os.path.join(HERE, "reference_cpu_vectors.json"), "w") as f:
        json.dump(manifest, f, indent=0)
    print("wrote", len(manifest), "cases")


if __name__ == "__main__":
    main()
