"""Loader for tests/golden/reference_cpu_vectors.*: the reference CPU backend's
outputs on fixed inputs (written by tests/golden/make_golden.py)."""
import json
import os

import numpy as np

import datagen

HERE = os.path.dirname(os.path.abspath(__file__))
_NPZ = None


def manifest():
    with open(os.path.join(HERE, "golden", "reference_cpu_vectors.json")) as f:
        return json.load(f)


def arrays():
    global _NPZ
    if _NPZ is None:
        _NPZ = np.load(os.path.join(HERE, "golden", "reference_cpu_vectors.npz"))
    return _NPZ


def bits_of(dtype):
    return 16 if dtype == 20 else 32


def steps_of(raw):
    return [(name, tuple(args)) for name, args in raw]


def operand(spec, dtype):
    dims, steps, salt = spec
    n = int(np.prod(dims))
    return tuple(dims), steps_of(steps), datagen.pattern_bits(bits_of(dtype), n, salt).reshape(dims)


def apply(view, steps):
    for name, args in steps:
        view = getattr(view, name)(*args)
    return view


def case_id(case):
    return case["key"]
