"""Writes tests/golden/sdpa_reference_cases.json: the reference's fixed attention fixtures.

The reference keeps its attention fixtures as code (sdpa_reference_cases,
test/backend/backend_conformance_sdpa_reference.hpp:1267-1299) together with an
independent evaluator (evaluate, :988) and the acceptance rule (matches, :1232-1259).
Run where oracle/_ref/libiom_ref.so has been built (`make -C oracle ref`):

    python tests/golden/make_sdpa_golden.py

Per case the file holds the shape parameters, the raw BF16 bits of q [B..,Hq,R,D] and
k, v [B..,Hkv,C,D] in logical row-major order, and the evaluator's output
[B..,R,Hq*D] as raw bits plus value class (0 finite, 1 +0, 2 -0, 3 +inf, 4 -inf, 5 NaN).
It also records, for a spread of (actual, expected) pairs, what the reference's
acceptance rule answers, so the rule restated in the tests is pinned too.
"""
import ctypes as C
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [os.path.join(ROOT, "oracle"), os.path.join(ROOT, "tests")]

import iomo  # noqa: E402


def main():
    lib = iomo.bind_iomc(iomo._load(iomo.REF_PATH))
    U16P, U8P = C.POINTER(C.c_uint16), C.POINTER(C.c_uint8)
    cases = []
    for index in range(lib.iomc_sdpa_case_count()):
        info = (C.c_uint64 * 17)()
        label = C.create_string_buffer(256)
        assert lib.iomc_sdpa_case_info(index, info, label, 256) == 0
        lead = [int(info[2 + i]) for i in range(int(info[1]))]
        hq, hkv, R, D, cap, a, L = (int(info[i]) for i in range(6, 13))
        q = np.zeros(int(info[14]), np.uint16)
        k = np.zeros(int(info[15]), np.uint16)
        v = np.zeros(int(info[16]), np.uint16)
        assert lib.iomc_sdpa_case_data(index, q.ctypes.data_as(U16P), k.ctypes.data_as(U16P),
                                       v.ctypes.data_as(U16P)) == 0
        n_out = int(np.prod(lead, dtype=np.int64)) * R * hq * D if lead else R * hq * D
        bits = np.zeros(n_out, np.uint16)
        classes = np.zeros(n_out, np.uint8)
        got = lib.iomc_sdpa_case_expected(index, bits.ctypes.data_as(U16P), classes.ctypes.data_as(U8P), n_out)
        assert got == n_out, (label.value, got, n_out)
        cases.append({
            "label": label.value.decode(), "kind": int(info[0]), "leading": lead,
            "Hq": hq, "Hkv": hkv, "R": R, "D": D, "C": cap, "a": a, "L": L,
            "padding_salt": int(info[13]),
            "q": q.tolist(), "k": k.tolist(), "v": v.tolist(),
            "expected_bits": bits.tolist(), "expected_class": classes.tolist(),
        })
    # the acceptance rule on a grid of pairs around a few reference values
    rule = []
    for expected in (0x3F80, 0x3C00, 0x3A00, 0x3800, 0x0080, 0xBF80, 0x4120, 0x7F7F, 0x0001):
        for delta in range(-6, 7):
            actual = (expected + delta) & 0xFFFF
            rule.append([actual, expected, 0, int(lib.iomc_sdpa_matches(actual, expected, 0))])
    for actual, expected, cls in ((0x0000, 0x0000, 1), (0x8000, 0x0000, 1), (0x8000, 0x8000, 2), (0x7FC0, 0x7FC0, 5),
                                  (0xFFC1, 0x7FC0, 5), (0x7F80, 0x7F80, 3), (0xFF80, 0x7F80, 3), (0x3F80, 0x7FC0, 5),
                                  (0x0000, 0x0001, 0), (0x3F80, 0x0000, 1)):
        rule.append([actual, expected, cls, int(lib.iomc_sdpa_matches(actual, expected, cls))])
    path = os.path.join(HERE, "sdpa_reference_cases.json")
    with open(path, "w") as f:
        json.dump({"cases": cases, "matches": rule}, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes,", len(cases), "cases")


if __name__ == "__main__":
    main()
