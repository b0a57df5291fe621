"""Bit-for-bit check of the C restatement against the reference's own CPU
backend, compiled from its sources into oracle/_ref (skipped where that
library was not built).  The reference is driven through its public
Device / TensorView / DeviceOps API exactly as its conformance drivers do.
"""
import numpy as np
import pytest

import datagen
import iomo
from iomo import DT_BF16, DT_F32, DT_I32, OP_ADD, OP_DIV, OP_MUL, OP_SUB

BITS = {DT_BF16: 16, DT_F32: 32, DT_I32: 32}


def both(ref, dtype, dims, salt=None, values=None, fill=None):
    """Create the same owner on the reference backend and in the oracle."""
    rt = ref.tensor(dtype, dims)
    ht = iomo.HostTensor(dtype, dims, fill=fill)
    if salt is not None:
        values = datagen.pattern_bits(BITS[dtype], int(np.prod(dims)), salt).reshape(dims)
    if values is not None:
        rt.view().from_host(values)
        ht.view().from_logical(values)
    return rt, ht


def apply(view, steps):
    for name, args in steps:
        view = getattr(view, name)(*args)
    return view


BINARY_CASES = [
    # (lhs owner dims, lhs view steps, rhs owner dims, rhs steps, out owner dims, out steps)
    ((2, 17, 33), [], (2, 17, 33), [], (2, 17, 33), []),
    ((1, 17, 33), [], (1, 17, 33), [], (1, 17, 33), []),
    ((2, 1, 33), [], (1, 17, 1), [], (2, 17, 33), []),              # row+column broadcast
    ((3, 32, 48), [], (1, 48), [], (3, 32, 48), []),                # row vector, lower rank
    ((3, 32, 48), [], (32, 1), [], (3, 32, 48), []),                # column vector
    ((1, 1), [], (2, 2, 16, 16), [], (2, 2, 16, 16), []),           # scalar broadcast
    ((6, 20, 35), [("slice", (0, 1, 3, 2))], (3, 20, 35), [], (3, 20, 35), []),
    ((4, 3, 16, 32), [("permute", ([1, 0],))], (3, 4, 16, 32), [], (3, 4, 16, 32), []),
    ((4, 3, 16, 32), [("select", (0, 2))], (1, 16, 32), [], (5, 3, 16, 32), [("select", (0, 4))]),
    ((2, 6, 16, 16), [("reshape_leading", ([3, 4],))], (4, 16, 16), [], (3, 4, 16, 16), []),
    ((2, 1, 16, 16), [], (1, 5, 16, 16), [], (2, 5, 16, 16), []),   # leading broadcast both sides
]


@pytest.mark.parametrize("dtype", [DT_I32, DT_F32, DT_BF16])
@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
@pytest.mark.parametrize("case", range(len(BINARY_CASES)))
def test_binary_bit_exact(ref, dtype, op, case):
    if op == OP_DIV and dtype == DT_I32:
        pytest.skip("integer division is refused; see test_division_of_integer_leaves_is_refused")
    ld, ls, rd, rs, od, os_ = BINARY_CASES[case]
    rl, hl = both(ref, dtype, ld, salt=0x100 + case)
    rr, hr = both(ref, dtype, rd, salt=0x200 + case)
    ro, ho = both(ref, dtype, od, salt=0x300 + case)   # prior content must survive outside the view
    tok = ref.binary(op, apply(rl.view(), ls), apply(rr.view(), rs), apply(ro.view(), os_))
    assert tok > 0, ref.error()
    for ieee in (False, True):
        _, ho2 = both(ref, dtype, od, salt=0x300 + case)
        assert iomo.binary(op, apply(hl.view(), ls), apply(hr.view(), rs),
                           apply(ho2.view(), os_), ieee) == 0
        assert np.array_equal(ro.view().to_host(), ho2.view().to_logical())
        assert np.array_equal(ro.view().raw_storage().view(ho2.storage.dtype), ho2.storage)


@pytest.mark.parametrize("dtype", [DT_I32, DT_F32, DT_BF16])
@pytest.mark.parametrize("which", ["lhs", "rhs", "both"])
def test_binary_exact_alias(ref, dtype, which):
    dims = (2, 17, 33)
    ra, ha = both(ref, dtype, dims, salt=1)
    rb, hb = both(ref, dtype, dims, salt=2)
    if which == "lhs":
        tok = ref.binary(OP_ADD, ra.view(), rb.view(), ra.view())
        rc = iomo.binary(OP_ADD, ha.view(), hb.view(), ha.view())
    elif which == "rhs":
        tok = ref.binary(OP_SUB, rb.view(), ra.view(), ra.view())
        rc = iomo.binary(OP_SUB, hb.view(), ha.view(), ha.view())
    else:
        tok = ref.binary(OP_MUL, ra.view(), ra.view(), ra.view())
        rc = iomo.binary(OP_MUL, ha.view(), ha.view(), ha.view())
    assert tok > 0 and rc == 0
    assert np.array_equal(ra.view().to_host(), ha.view().to_logical())


def test_division_of_integer_leaves_is_refused(ref):
    a, ha = both(ref, DT_I32, (2, 16, 16), salt=1)
    b, hb = both(ref, DT_I32, (2, 16, 16), salt=2)
    o, ho = both(ref, DT_I32, (2, 16, 16), salt=3)
    assert ref.binary(OP_DIV, a.view(), b.view(), o.view()) < 0
    assert iomo.binary(OP_DIV, ha.view(), hb.view(), ho.view()) == -2
    assert np.array_equal(o.view().to_host(), ho.view().to_logical())      # untouched


def test_reference_rejects_what_the_oracle_rejects(ref):
    a, ha = both(ref, DT_F32, (2, 16, 16), salt=1)
    b, hb = both(ref, DT_F32, (3, 16, 16), salt=2)
    o, ho = both(ref, DT_F32, (2, 16, 16), salt=3)
    assert ref.binary(OP_ADD, a.view(), b.view(), o.view()) == -1
    assert iomo.binary(OP_ADD, ha.view(), hb.view(), ho.view()) == -1


def float_values(dtype, dims, salt, kind):
    n = int(np.prod(dims))
    if kind == "bits":
        return datagen.pattern_bits(BITS[dtype], n, salt).reshape(dims)
    v = datagen.normal_f32(n, 0, 1, salt)
    if kind == "outliers":
        v = v.reshape(-1, dims[-1])
        v[::7] *= 50
        v = v.reshape(-1)
    if dtype == DT_BF16:
        return datagen.bf16_rne(v).reshape(dims)
    return v.view(np.uint32).reshape(dims)


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32])
@pytest.mark.parametrize("dims,steps", [
    ((1, 1), []), ((15, 16), []), ((17, 33), []), ((16, 31), []), ((3, 5, 130), []),
    ((2, 3, 17, 64), [("permute", ([1, 0],))]),
    ((6, 16, 48), [("slice", (0, 0, 3, 2))]),
    ((40, 2048), []),
])
@pytest.mark.parametrize("kind", ["normal", "outliers", "bits"])
def test_rmsnorm_bit_exact(ref, dtype, dims, steps, kind):
    rx, hx = both(ref, dtype, dims, values=float_values(dtype, dims, 31, kind))
    F = dims[-1]
    w = datagen.uniform_f32(F, 0.5, 1.5, 32)
    wl = (datagen.bf16_rne(w) if dtype == DT_BF16 else w.view(np.uint32)).reshape(1, F)
    rw, hw = both(ref, dtype, (1, F), values=wl)
    vx, vhx = apply(rx.view(), steps), apply(hx.view(), steps)
    odims = vhx.dims
    ro, ho = both(ref, dtype, odims, salt=99, fill=None)
    tok = ref.rmsnorm(vx, rw.view(), ro.view(), 1e-5)
    assert tok > 0, ref.error()
    assert iomo.rmsnorm(vhx, hw.view(), ho.view(), 1e-5) == 0
    assert np.array_equal(ro.view().to_host(), ho.view().to_logical())
    assert np.array_equal(ro.view().raw_storage().view(ho.storage.dtype), ho.storage)


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32])
@pytest.mark.parametrize("dims,steps", [
    ((17, 33), []), ((3, 16, 48), []), ((4, 2, 16, 16), [("permute", ([1, 0],))]), ((64, 512), []),
])
@pytest.mark.parametrize("kind", ["normal", "bits"])
def test_silu_bit_exact(ref, dtype, dims, steps, kind):
    rx, hx = both(ref, dtype, dims, values=float_values(dtype, dims, 41, kind))
    vx, vhx = apply(rx.view(), steps), apply(hx.view(), steps)
    ro, ho = both(ref, dtype, vhx.dims, salt=98)
    tok = ref.silu(vx, ro.view())
    assert tok > 0, ref.error()
    assert iomo.silu(vhx, ho.view()) == 0
    assert np.array_equal(ro.view().to_host(), ho.view().to_logical())
    assert np.array_equal(ro.view().raw_storage().view(ho.storage.dtype), ho.storage)


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32, DT_I32])
@pytest.mark.parametrize("sd,ss,dd,ds", [
    ((2, 17, 33), [], (2, 17, 33), []),
    ((6, 20, 35), [("slice", (0, 1, 3, 2))], (3, 20, 35), []),
    ((4, 3, 16, 32), [("permute", ([1, 0],))], (3, 4, 16, 32), []),
    ((3, 16, 16), [], (5, 3, 16, 16), [("select", (0, 1))]),
])
def test_copy_bit_exact(ref, dtype, sd, ss, dd, ds):
    rs_, hs = both(ref, dtype, sd, salt=51)
    rd_, hd = both(ref, dtype, dd, salt=52)
    tok = ref.copy(apply(rs_.view(), ss), apply(rd_.view(), ds))
    assert tok > 0, ref.error()
    assert iomo.copy(apply(hs.view(), ss), apply(hd.view(), ds)) == 0
    assert np.array_equal(rd_.view().raw_storage().view(hd.storage.dtype), hd.storage)


# ---- softmax stage, reached through the public sdpa with identity K and V ----

def sdpa_probabilities(ref, scores_bf16_times8, a, L, C=64):
    """Run the reference's sdpa with Hq=Hkv=1, D=C=64, K=V=I.

    q[r,t] = 8*score[r,t] (exact in BF16 for the chosen scores), so
    dot(q[r],k[t]) / sqrt(64) = score[r,t] exactly, and out[r,d] = P[r,d]
    for d < visible(r) (src/cpu/sdpa.cpp:186-203,317-336).
    """
    R = scores_bf16_times8.shape[0]
    D = C
    eye = np.zeros((C, D), np.uint16)
    eye[np.arange(C), np.arange(C)] = 0x3F80
    q = ref.tensor(DT_BF16, (1, R, D))
    k = ref.tensor(DT_BF16, (1, C, D))
    v = ref.tensor(DT_BF16, (1, C, D))
    o = ref.tensor(DT_BF16, (R, D))
    q.view().from_host(scores_bf16_times8.reshape(1, R, D))
    k.view().from_host(eye.reshape(1, C, D))
    v.view().from_host(eye.reshape(1, C, D))
    tok = ref.sdpa(q.view(), k.view(), v.view(), o.view(), a, L)
    assert tok > 0, (tok, ref.error())
    return o.view().to_host()


def test_softmax_stage_matches_reference_sdpa(ref):
    C, L, a = 64, 40, 10
    R = 33
    raw = datagen.normal_f32(R * C, 0, 3, 61).reshape(R, C)
    # Infinite or NaN scores cannot be fed this way (inf*0 in the other dot products
    # poisons the whole row); those rows are pinned by the reference's own special-row
    # vectors in test_oracle_kats.py.  Finite extremes can.
    raw[3, 2] = -200.0
    raw[4, :] = -300.0
    raw[4, 12] = 0.5
    raw[8, 1] = -60.0
    raw[8, 0] = 20.0
    raw[9, :] = 1000.0
    raw[11, :] = 0.0
    q_bits = datagen.bf16_rne(raw * 8.0)
    scores = (datagen.bf16_to_f32(q_bits.reshape(-1)) / np.float32(8.0)).reshape(R, C)
    got = sdpa_probabilities(ref, q_bits, a, L, C)
    want = iomo.softmax(scores.reshape(1, 1, R, C), a=a, L=L)[0, 0]
    for r in range(R):
        vis = min(L, a + r + 1)
        w = want[r, :vis].copy()
        if np.all(w == 0x7FC0):
            assert np.all(got[r] == 0x7FC0)        # NaN rows poison the whole output row
            continue
        # the PV stage flushes subnormal probabilities and stores -0 as +0
        w[(w & 0x7F80) == 0] = 0
        assert np.array_equal(got[r, :vis], w), r
        assert np.all(got[r, vis:] == 0)
