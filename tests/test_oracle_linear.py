"""Linear projection of the C restatement against the reference CPU backend compiled into
oracle/_ref (bit for bit: the scalar recurrence with the same fused multiply-add), on the
contract's fixture shapes (docs/BACKEND_CONTRACT/linear-projections.md:307-330), and against
exact integer / float64 evaluations that do not involve the reference."""
import numpy as np
import pytest

import datagen
import iomo
from iomo import DT_BF16, DT_F32, DT_F64, FLOAT_LEAVES, INTEGER_LEAVES, LEAF_BITS, LEAF_NAME, NUMERIC_LEAVES

names = lambda ds: [LEAF_NAME[d] for d in ds]
FMT = {13: (2, 1, 1), 14: (2, 3, 1), 15: (3, 2, 3), 16: (4, 3, 7), 17: (5, 2, 15), 19: (5, 10, 15),
       20: (8, 7, 127), 21: (8, 23, 127), 22: (11, 52, 1023)}


def small_values(dtype, count, salt):
    """Raw encodings of moderate finite values (no NaN / infinity, sums stay in range)."""
    bits = LEAF_BITS[dtype]
    v = datagen.pattern_bits(bits, count, salt)
    if dtype in INTEGER_LEAVES or dtype in (13, 14, 15):
        return v
    ebits, fbits, bias = FMT[dtype]
    exp = (v.astype(np.uint64) >> np.uint64(fbits)) & np.uint64((1 << ebits) - 1)
    exp = exp % np.uint64(5) + np.uint64(bias - 3)
    cleared = v.astype(np.uint64) & ~np.uint64(((1 << ebits) - 1) << fbits)
    return (cleared | (exp << np.uint64(fbits))).astype(v.dtype)


def both(ref, dtype, dims, values=None, salt=None):
    rt, ht = ref.tensor(dtype, dims), iomo.HostTensor(dtype, dims)
    if salt is not None:
        values = datagen.pattern_bits(LEAF_BITS[dtype], int(np.prod(dims)), salt).reshape(dims)
    if values is not None:
        rt.view().from_host(values)
        ht.view().from_logical(values)
    return rt, ht


def same_storage(rt, ht):
    return np.array_equal(rt.view().raw_storage(), ht.storage.view(np.uint8))


FIXTURES = [
    # x dims, w dims, s, R, head_planar, H, D
    ((19, 3), (10, 3), 2, 17, False, 1, 10), ((19, 3), (10, 3), 2, 16, False, 1, 10),
    ((19, 3), (10, 3), 2, 15, True, 2, 5), ((19, 3), (10, 3), 2, 1, True, 2, 5),
    ((2, 3, 20, 65), (33, 65), 3, 17, False, 1, 33), ((2, 3, 20, 65), (34, 65), 0, 20, True, 2, 17),
    ((7, 48), (100, 48), 6, 1, False, 1, 100),                       # LM head: last row only
]


@pytest.mark.parametrize("dtype", NUMERIC_LEAVES, ids=names(NUMERIC_LEAVES))
@pytest.mark.parametrize("case", range(len(FIXTURES)))
def test_linear_bit_exact(ref, dtype, case):
    xd, wd, s, R, hp, H, D = FIXTURES[case]
    rx, hx = both(ref, dtype, xd, values=small_values(dtype, int(np.prod(xd)), 1 + case).reshape(xd))
    rw, hw = both(ref, dtype, wd, values=small_values(dtype, int(np.prod(wd)), 11 + case).reshape(wd))
    od = xd[:-2] + ((H, R, D) if hp else (R, D))
    ro, ho = both(ref, dtype, od, salt=21 + case)
    assert ref.linear(rx.view(), rw.view(), ro.view(), s, R, hp, H, D) > 0, ref.error()
    assert iomo.linear(hx.view(), hw.view(), ho.view(), s, R, hp, H, D) == 0
    assert same_storage(ro, ho)


def test_linear_views(ref):
    xd, wd = (4, 2, 20, 40), (3, 24, 40)
    rx, hx = both(ref, DT_BF16, xd, values=small_values(DT_BF16, int(np.prod(xd)), 5).reshape(xd))
    rw, hw = both(ref, DT_BF16, wd, values=small_values(DT_BF16, int(np.prod(wd)), 6).reshape(wd))
    ro, ho = both(ref, DT_BF16, (2, 4, 3, 9, 8), salt=7)
    xv = lambda t: t.view().permute([1, 0])                       # [2,4,20,40]
    wv = lambda t: t.view().select(0, 1)                          # [24,40]
    assert ref.linear(xv(rx), wv(rw), ro.view(), 5, 9, True, 3, 8) > 0, ref.error()
    assert iomo.linear(xv(hx), wv(hw), ho.view(), 5, 9, True, 3, 8) == 0
    assert same_storage(ro, ho)


def test_linear_rejections(ref):
    rx, hx = both(ref, DT_F32, (19, 3), salt=1)
    rw, hw = both(ref, DT_F32, (10, 3), salt=2)
    ro, ho = both(ref, DT_F32, (17, 10))
    rh, hh = both(ref, DT_F32, (2, 17, 5))
    for args in ((2, 18, False, 1, 10), (20, 1, False, 1, 10), (2, 0, False, 1, 10), (2, 17, False, 2, 5),
                 (2, 17, False, 1, 9)):
        assert ref.linear(rx.view(), rw.view(), ro.view(), *args) == -1, args
        assert iomo.linear(hx.view(), hw.view(), ho.view(), *args) == -1, args
    assert ref.linear(rx.view(), rw.view(), rh.view(), 2, 17, True, 2, 6) == -1
    assert iomo.linear(hx.view(), hw.view(), hh.view(), 2, 17, True, 2, 6) == -1
    assert ref.linear(rx.view(), rw.view(), rh.view(), 2, 17, True, 5, 2) == -1   # out shape is [2,17,5]
    assert iomo.linear(hx.view(), hw.view(), hh.view(), 2, 17, True, 5, 2) == -1
    for dtype in (iomo.DT_BOOL, iomo.DT_F8_E8M0):
        a, ha = both(ref, dtype, (19, 3))
        b, hb = both(ref, dtype, (10, 3))
        o, ho2 = both(ref, dtype, (17, 10))
        assert ref.linear(a.view(), b.view(), o.view(), 2, 17, False, 1, 10) == -2
        assert iomo.linear(ha.view(), hb.view(), ho2.view(), 2, 17, False, 1, 10) == -2


@pytest.mark.parametrize("dtype", [iomo.DT_I8, iomo.DT_U16, iomo.DT_I32, iomo.DT_U64], ids=["I8", "U16", "I32", "U64"])
def test_linear_integers_against_exact_arithmetic(dtype):
    T, I, O = 9, 65, 21
    bits = LEAF_BITS[dtype]
    x = datagen.pattern_bits(bits, T * I, 3).reshape(T, I)
    w = datagen.pattern_bits(bits, O * I, 4).reshape(O, I)
    hx, hw, ho = iomo.HostTensor(dtype, (T, I)), iomo.HostTensor(dtype, (O, I)), iomo.HostTensor(dtype, (T, O))
    hx.view().from_logical(x)
    hw.view().from_logical(w)
    assert iomo.linear(hx.view(), hw.view(), ho.view(), 0, T, False, 1, O) == 0
    exact = [[sum(int(a) * int(b) for a, b in zip(x[r], w[o])) % (1 << bits) for o in range(O)] for r in range(T)]
    assert np.array_equal(ho.view().to_logical().astype(np.uint64), np.array(exact, dtype=np.uint64))


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32, DT_F64], ids=["BF16", "F32", "F64"])
def test_linear_floats_against_float64(dtype):
    """The contract's own thresholds (linear-projections.md:334-341)."""
    T, I, O = 9, 65, 21
    x64 = datagen.normal_f32(T * I, 0, 1, 5).astype(np.float64).reshape(T, I)
    w64 = datagen.normal_f32(O * I, 0, 1, 6).astype(np.float64).reshape(O, I)
    if dtype == DT_BF16:
        xr, wr = datagen.bf16_rne(x64.astype(np.float32)), datagen.bf16_rne(w64.astype(np.float32))
        x64, w64 = datagen.bf16_to_f32(xr).astype(np.float64), datagen.bf16_to_f32(wr).astype(np.float64)
    elif dtype == DT_F32:
        xr, wr = x64.astype(np.float32).view(np.uint32), w64.astype(np.float32).view(np.uint32)
    else:
        xr, wr = x64.view(np.uint64), w64.view(np.uint64)
    hx, hw, ho = iomo.HostTensor(dtype, (T, I)), iomo.HostTensor(dtype, (O, I)), iomo.HostTensor(dtype, (T, O))
    hx.view().from_logical(xr.reshape(T, I))
    hw.view().from_logical(wr.reshape(O, I))
    assert iomo.linear(hx.view(), hw.view(), ho.view(), 0, T, False, 1, O) == 0
    got = ho.view().to_logical()
    ref = x64.reshape(T, I) @ w64.reshape(O, I).T
    if dtype == DT_BF16:
        g = datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(T, O)
        q = datagen.bf16_to_f32(datagen.bf16_rne(ref.astype(np.float32).reshape(-1))).astype(np.float64).reshape(T, O)
        ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(q), 1e-30))) - 7)
        assert (np.abs(g - q) <= np.maximum(np.maximum(ulp, 2.0 ** -7), 2.0 ** -6 * np.abs(q))).all()
    elif dtype == DT_F32:
        assert (np.abs(got.view(np.float32).astype(np.float64) - ref) <= 1e-5 + 1e-5 * np.abs(ref)).all()
    else:
        assert (np.abs(got.view(np.float64) - ref) <= 1e-12 + 1e-12 * np.abs(ref)).all()
