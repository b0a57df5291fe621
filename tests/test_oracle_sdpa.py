"""The CPU oracle's attention (iomo_sdpa) against the reference's own fixtures and backend.

* tests/golden/sdpa_reference_cases.json holds the reference's fixed attention fixtures,
  the values its independent evaluator expects and answers of its acceptance rule
  (test/backend/backend_conformance_sdpa_reference.hpp:988,1232-1299), written by
  tests/golden/make_sdpa_golden.py.
* Where oracle/_ref is built, the oracle is also compared bit for bit with the reference's
  compiled CPU backend (src/cpu/sdpa.cpp) on seeded shapes.
"""
import json
import os

import numpy as np
import pytest

import datagen
import iomo
from iomo import DT_BF16, DT_F32

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "sdpa_reference_cases.json")) as f:
    GOLDEN = json.load(f)
CASES = GOLDEN["cases"]


def bf16_class(bits):
    """0 finite, 1 +0, 2 -0, 3 +inf, 4 -inf, 5 NaN."""
    mag = bits & 0x7FFF
    if mag > 0x7F80:
        return 5
    if mag == 0x7F80:
        return 4 if bits & 0x8000 else 3
    if mag == 0:
        return 2 if bits & 0x8000 else 1
    return 0


def ordered(bits):
    return -(bits & 0x7FFF) if bits & 0x8000 else (bits & 0x7FFF)


def matches(actual, expected_bits, expected_class):
    """test/backend/backend_conformance_sdpa_reference.hpp:1232-1259 for BF16."""
    if bf16_class(actual) != expected_class:
        return False
    if expected_class != 0:
        return True
    if abs(ordered(actual) - ordered(expected_bits)) <= 2:
        return True
    a = datagen.bf16_to_f32(np.array([actual], np.uint16))[0]
    r = datagen.bf16_to_f32(np.array([expected_bits], np.uint16))[0]
    ulp = abs(np.nextafter(r, np.float32(np.inf)) - r)
    return abs(np.float32(a) - np.float32(r)) <= max(np.float32(2) * ulp, np.float32(2.0 ** -10))


def all_match(got, case):
    got = np.asarray(got).reshape(-1)
    return [i for i, (g, e, c) in enumerate(zip(got, case["expected_bits"], case["expected_class"]))
            if not matches(int(g), e, c)]


def test_acceptance_rule_restated_like_the_reference():
    for actual, expected, cls, answer in GOLDEN["matches"]:
        assert matches(actual, expected, cls) == bool(answer), (hex(actual), hex(expected), cls)


def shapes(case):
    lead = tuple(case["leading"])
    return (lead + (case["Hq"], case["R"], case["D"]), lead + (case["Hkv"], case["C"], case["D"]),
            lead + (case["R"], case["Hq"] * case["D"]))


def host_operands(case, fill=0x5A):
    qd, kd, od = shapes(case)
    q = iomo.HostTensor(DT_BF16, qd, fill=fill)
    k = iomo.HostTensor(DT_BF16, kd, fill=fill)
    v = iomo.HostTensor(DT_BF16, kd, fill=fill)
    o = iomo.HostTensor(DT_BF16, od, fill=fill)
    q.view().from_logical(np.array(case["q"], np.uint16).reshape(qd))
    k.view().from_logical(np.array(case["k"], np.uint16).reshape(kd))
    v.view().from_logical(np.array(case["v"], np.uint16).reshape(kd))
    return q, k, v, o


@pytest.mark.parametrize("index", range(len(CASES)), ids=[c["label"].replace(" ", "_") for c in CASES])
def test_oracle_on_the_reference_fixtures(index):
    case = CASES[index]
    for fill in (0x5A, 0xFF):          # 0xFF fills padding and the cache tail with NaN patterns
        q, k, v, o = host_operands(case, fill)
        assert iomo.sdpa(q.view(), k.view(), v.view(), o.view(), case["a"], case["L"]) == 0
        got = o.view().to_logical().reshape(-1)
        assert all_match(got, case) == []
    exact = int(np.sum(got == np.array(case["expected_bits"], np.uint16)))
    print(case["label"], "bit-equal to the independent evaluator:", exact, "of", got.size)


def random_case(seed, lead, Hq, Hkv, R, D, C, a, L):
    n = int(np.prod(lead)) if lead else 1
    q = datagen.bf16_rne(datagen.normal_f32(n * Hq * R * D, 0, 1, seed)).tolist()
    k = datagen.bf16_rne(datagen.normal_f32(n * Hkv * C * D, 0, 1, seed + 1)).tolist()
    v = datagen.bf16_rne(datagen.normal_f32(n * Hkv * C * D, 0, 2, seed + 2)).tolist()
    return {"leading": list(lead), "Hq": Hq, "Hkv": Hkv, "R": R, "D": D, "C": C, "a": a, "L": L,
            "q": q, "k": k, "v": v}


RANDOM = [((), 2, 1, 5, 8, 12, 3, 9), ((2,), 4, 2, 17, 16, 40, 20, 37), ((2, 2), 4, 1, 3, 33, 20, 0, 2),
          ((), 8, 2, 1, 64, 70, 69, 70), ((3,), 2, 2, 16, 5, 16, 0, 16)]


def test_tail_future_and_padding_do_not_matter():
    case = random_case(5, (2,), 4, 2, 6, 16, 24, 4, 8)
    outs = []
    for variant in range(3):
        c = dict(case)
        k = np.array(case["k"], np.uint16).reshape(2, 2, 24, 16).copy()
        v = np.array(case["v"], np.uint16).reshape(2, 2, 24, 16).copy()
        if variant >= 1:
            k[:, :, 8:, :] = 0x7FC0        # cache tail [L, C)
            v[:, :, 8:, :] = 0x7F80
        if variant == 2:
            c["R"] = 3                      # rows 0..2 see tokens 0..4+r; tokens 7.. are future for all
            c["q"] = np.array(case["q"], np.uint16).reshape(2, 4, 6, 16)[:, :, :3].reshape(-1).tolist()
            k[:, :, 7, :] = 0xFF80
            v[:, :, 7, :] = 0x7FC1
        c["k"], c["v"] = k.reshape(-1).tolist(), v.reshape(-1).tolist()
        q_, k_, v_, o_ = host_operands(c, fill=0x5A if variant == 0 else 0xFF)
        assert iomo.sdpa(q_.view(), k_.view(), v_.view(), o_.view(), c["a"], c["L"]) == 0
        outs.append(o_.view().to_logical())
    assert np.array_equal(outs[0], outs[1])
    assert np.array_equal(outs[0][:, :3], outs[2])


def test_incremental_rows_equal_the_full_recomputation():
    case = random_case(9, (), 4, 2, 7, 8, 7, 0, 7)
    q, k, v, o = host_operands(case)
    assert iomo.sdpa(q.view(), k.view(), v.view(), o.view(), 0, 7) == 0
    full = o.view().to_logical()
    for r in range(7):
        c = dict(case)
        c["R"] = 1
        c["q"] = np.array(case["q"], np.uint16).reshape(4, 7, 8)[:, r:r + 1].reshape(-1).tolist()
        q1, k1, v1, o1 = host_operands(c)
        assert iomo.sdpa(q1.view(), k1.view(), v1.view(), o1.view(), r, r + 1) == 0
        assert np.array_equal(o1.view().to_logical()[0], full[r])


def test_uniform_scores_average_v():
    """q = 0 makes every visible probability 1/n: out = mean of the visible V rows, computed
    as the sequential binary32 sum of bf16(1/n) * v."""
    Hq, R, D, C, a, L = 2, 4, 4, 9, 3, 6
    case = random_case(13, (), Hq, 1, R, D, C, a, L)
    case["q"] = [0] * (Hq * R * D)
    q, k, v, o = host_operands(case)
    assert iomo.sdpa(q.view(), k.view(), v.view(), o.view(), a, L) == 0
    got = o.view().to_logical()
    vv = datagen.bf16_to_f32(np.array(case["v"], np.uint16)).reshape(C, D)
    for r in range(R):
        n = min(L, a + r + 1)
        p = datagen.bf16_to_f32(datagen.bf16_rne(np.array([np.float32(1) / np.float32(n)], np.float32)))[0]
        acc = np.zeros(D, np.float32)
        for t in range(n):
            acc = (acc + np.float32(p) * vv[t]).astype(np.float32)
        want = datagen.bf16_rne(acc)
        for h in range(Hq):
            assert np.array_equal(got[r, h * D:(h + 1) * D], want)


def test_rejections():
    case = random_case(3, (), 4, 2, 3, 8, 10, 2, 5)
    q, k, v, o = host_operands(case)
    for a, L in ((2, 0), (2, 11), (10, 5), (8, 5)):
        assert iomo.sdpa(q.view(), k.view(), v.view(), o.view(), a, L) == -1, (a, L)
    bad = iomo.HostTensor(DT_BF16, (3, 4 * 8 + 1))
    assert iomo.sdpa(q.view(), k.view(), v.view(), bad.view(), 2, 5) == -1
    k3 = iomo.HostTensor(DT_BF16, (3, 10, 8))
    assert iomo.sdpa(q.view(), k3.view(), k3.view(), o.view(), 2, 5) == -1       # Hq % Hkv != 0
    qf, kf, of = (iomo.HostTensor(DT_F32, d) for d in ((4, 3, 8), (2, 10, 8), (3, 32)))
    assert iomo.sdpa(qf.view(), kf.view(), kf.view(), of.view(), 2, 5) == -2


# ---- against the reference's compiled CPU backend -------------------------------------

@pytest.fixture(scope="module")
def ref():
    if not iomo.ref_available():
        pytest.skip("oracle/_ref/libiom_ref.so not built (needs the reference sources)")
    b = iomo.ref_backend()
    yield b
    b.close()


@pytest.mark.parametrize("spec", RANDOM, ids=[str(i) for i in range(len(RANDOM))])
def test_bit_exact_with_the_reference_cpu_backend(ref, spec):
    lead, Hq, Hkv, R, D, C, a, L = spec
    case = random_case(21 + R, lead, Hq, Hkv, R, D, C, a, L)
    # a few operands that exercise the flush and the special rows
    kk = np.array(case["k"], np.uint16)
    kk[1] = 0x0040          # subnormal
    kk[2] = 0x8001
    case["k"] = kk.tolist()
    qd, kd, od = shapes(case)
    q, k, v, o = host_operands(case)
    rq, rk, rv, ro = (ref.tensor(DT_BF16, d) for d in (qd, kd, kd, od))
    rq.view().from_host(np.array(case["q"], np.uint16).reshape(qd))
    rk.view().from_host(np.array(case["k"], np.uint16).reshape(kd))
    rv.view().from_host(np.array(case["v"], np.uint16).reshape(kd))
    tok = ref.sdpa(rq.view(), rk.view(), rv.view(), ro.view(), a, L)
    assert tok > 0, (tok, ref.error())
    assert iomo.sdpa(q.view(), k.view(), v.view(), o.view(), a, L) == 0
    assert np.array_equal(ro.view().to_host(), o.view().to_logical())


@pytest.mark.parametrize("index", range(len(CASES)), ids=[c["label"].replace(" ", "_") for c in CASES])
def test_reference_cpu_backend_and_oracle_agree_on_the_fixtures(ref, index):
    case = CASES[index]
    qd, kd, od = shapes(case)
    q, k, v, o = host_operands(case)
    rq, rk, rv, ro = (ref.tensor(DT_BF16, d) for d in (qd, kd, kd, od))
    rq.view().from_host(np.array(case["q"], np.uint16).reshape(qd))
    rk.view().from_host(np.array(case["k"], np.uint16).reshape(kd))
    rv.view().from_host(np.array(case["v"], np.uint16).reshape(kd))
    tok = ref.sdpa(rq.view(), rk.view(), rv.view(), ro.view(), case["a"], case["L"])
    assert tok > 0, (tok, ref.error())
    assert iomo.sdpa(q.view(), k.view(), v.view(), o.view(), case["a"], case["L"]) == 0
    want, got = ro.view().to_host().reshape(-1), o.view().to_logical().reshape(-1)
    nan = (want & 0x7FFF) > 0x7F80
    assert np.array_equal(nan, (got & 0x7FFF) > 0x7F80)
    assert np.array_equal(want[~nan], got[~nan])
