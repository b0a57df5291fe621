"""cache_append, embedding and rope of the C restatement against the reference CPU
backend compiled into oracle/_ref (bit for bit: same compiler flags, same libm), plus
checks that do not depend on the reference."""
import numpy as np
import pytest

import datagen
import iomo
from iomo import (ALL_LEAVES, DT_BF16, DT_F16, DT_F32, DT_F64, DT_I16, DT_I32, DT_I64, DT_I8, DT_U2,
                  DT_U32, DT_U4, DT_U8, FLOAT_LEAVES, INTEGER_LEAVES, LEAF_BITS, LEAF_NAME)

names = lambda ds: [LEAF_NAME[d] for d in ds]


def pattern(dtype, count, salt):
    v = datagen.pattern_bits(LEAF_BITS[dtype], count, salt)
    return v & 1 if dtype == iomo.DT_BOOL else v


def both(ref, dtype, dims, salt=None, values=None):
    rt, ht = ref.tensor(dtype, dims), iomo.HostTensor(dtype, dims)
    if salt is not None:
        values = pattern(dtype, int(np.prod(dims)), salt).reshape(dims)
    if values is not None:
        rt.view().from_host(values)
        ht.view().from_logical(values)
    return rt, ht


def same_storage(rt, ht):
    return np.array_equal(rt.view().raw_storage(), ht.storage.view(np.uint8))


# -- cache append -------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ALL_LEAVES, ids=names(ALL_LEAVES))
@pytest.mark.parametrize("shape", [((2, 3, 5, 40), (2, 3, 37, 40), 0), ((2, 3, 5, 40), (2, 3, 37, 40), 32),
                                   ((4, 1, 64), (4, 20, 64), 19), ((1, 2, 17, 7), (1, 2, 17, 7), 0)])
def test_cache_append_bit_exact(ref, dtype, shape):
    sd, dd, a = shape
    rs, hs = both(ref, dtype, sd, salt=3)
    rd, hd = both(ref, dtype, dd, salt=4)
    assert ref.cache_append(rs.view(), rd.view(), a) > 0, ref.error()
    assert iomo.cache_append(hs.view(), hd.view(), a) == 0
    assert same_storage(rd, hd)
    # closed form: rows a..a+R of every plane are the source, everything else untouched
    before = pattern(dtype, int(np.prod(dd)), 4).reshape(dd)
    want = before.copy()
    want[..., a:a + sd[-2], :] = pattern(dtype, int(np.prod(sd)), 3).reshape(sd)
    assert np.array_equal(hd.view().to_logical(), want)


def test_cache_append_views_and_rejections(ref):
    rs, hs = both(ref, DT_BF16, (4, 2, 3, 32), salt=5)
    rd, hd = both(ref, DT_BF16, (2, 4, 40, 32), salt=6)
    sv = lambda t: t.view().slice(0, 0, 2, 2).permute([1, 0])     # [2,2,3,32]
    dv = lambda t: t.view().slice(1, 1, 2, 2).permute([1, 0])     # [2,2,40,32]
    assert ref.cache_append(sv(rs), dv(rd), 37) > 0, ref.error()
    assert iomo.cache_append(sv(hs), dv(hd), 37) == 0
    assert same_storage(rd, hd)
    for a in (38, 41, 1 << 40):                                      # rows exceed the capacity
        assert ref.cache_append(sv(rs), dv(rd), a) == -1
        assert iomo.cache_append(sv(hs), dv(hd), a) == -1
    r2, h2 = both(ref, DT_BF16, (2, 2, 3, 48), salt=7)                # feature extents differ
    assert ref.cache_append(r2.view(), dv(rd), 0) == -1
    assert iomo.cache_append(h2.view(), dv(hd), 0) == -1
    assert ref.cache_append(dv(rd), dv(rd), 0) == -1                  # same owner
    assert iomo.cache_append(dv(hd), dv(hd), 0) == -1


# -- embedding ----------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ALL_LEAVES, ids=names(ALL_LEAVES))
def test_embedding_every_payload_leaf(ref, dtype):
    V, F, R = 37, 40, 9
    rt, ht = both(ref, dtype, (V, F), salt=11)
    ids = (datagen.pattern_bits(32, 2 * 3 * R, 12) % V).reshape(2, 3, 1, R)
    ri, hi = both(ref, DT_I32, (2, 3, 1, R), values=ids)
    ro, ho = both(ref, dtype, (2, 3, R, F), salt=13)
    token, waited = ref.embedding(rt.view(), ri.view(), ro.view())
    assert token > 0 and waited == 0, ref.error()
    assert iomo.embedding(ht.view(), hi.view(), ho.view()) == 0
    assert same_storage(ro, ho)
    table = pattern(dtype, V * F, 11).reshape(V, F)
    assert np.array_equal(ho.view().to_logical(), table[ids.reshape(2, 3, R)])   # numpy fancy indexing


@pytest.mark.parametrize("index_dtype", INTEGER_LEAVES, ids=names(INTEGER_LEAVES))
def test_embedding_every_index_leaf(ref, index_dtype):
    bits = LEAF_BITS[index_dtype]
    signed = index_dtype in (iomo.DT_I2, iomo.DT_I4, DT_I8, DT_I16, DT_I32, DT_I64)
    top = (1 << (bits - 1 if signed else bits)) - 1
    V = min(top + 1, 50)
    R = 21
    rt, ht = both(ref, DT_BF16, (V, 16), salt=21)
    ids = (datagen.pattern_bits(32, 2 * R, 22) % V).astype(iomo.NP_OF[index_dtype]).reshape(2, 1, R)
    ri, hi = both(ref, index_dtype, (2, 1, R), values=ids)
    ro, ho = both(ref, DT_BF16, (2, R, 16))
    token, waited = ref.embedding(rt.view(), ri.view(), ro.view())
    assert token > 0 and waited == 0, ref.error()
    assert iomo.embedding(ht.view(), hi.view(), ho.view()) == 0
    assert same_storage(ro, ho)
    # one invalid id: the largest value of the leaf (negative when signed, else >= V if V is smaller)
    bad = ids.copy()
    bad[1, 0, R - 1] = (1 << bits) - 1 if bits < 64 else np.uint64(0xFFFFFFFFFFFFFFFF)
    if signed or (1 << bits) - 1 >= V:
        ri2, hi2 = both(ref, index_dtype, (2, 1, R), values=bad)
        token, waited = ref.embedding(rt.view(), ri2.view(), ro.view())
        assert token > 0 and waited == -1          # accepted, then the deferred InvalidArgument
        assert iomo.embedding(ht.view(), hi2.view(), ho.view()) == -1


def test_embedding_views(ref):
    V, F, R = 20, 33, 5
    rt, ht = both(ref, DT_F32, (3, V, F), salt=31)                 # table = plane 2 of a rank-3 owner
    ids = (datagen.pattern_bits(32, 4 * 2 * R, 32) % V).reshape(4, 2, 1, R)
    ri, hi = both(ref, DT_U8, (4, 2, 1, R), values=ids.astype(np.uint8))
    ro, ho = both(ref, DT_F32, (2, 6, R, F), salt=33)
    iv = lambda t: t.view().slice(0, 1, 2, 2).permute([1, 0])      # [2,2,1,R]
    ov = lambda t: t.view().slice(1, 0, 2, 3).permute([1, 0])      # [2,2,R,F]
    token, waited = ref.embedding(rt.view().select(0, 2), iv(ri), ov(ro))
    assert token > 0 and waited == 0, ref.error()
    assert iomo.embedding(ht.view().select(0, 2), iv(hi), ov(ho)) == 0
    assert same_storage(ro, ho)


# -- rope ---------------------------------------------------------------------------

def finite_values(dtype, count, salt):
    bits = LEAF_BITS[dtype]
    v = datagen.pattern_bits(bits, count, salt)
    ebits, fbits = {13: (2, 1), 14: (2, 3), 15: (3, 2), 16: (4, 3), 17: (5, 2), 19: (5, 10),
                    20: (8, 7), 21: (8, 23), 22: (11, 52)}[dtype]
    if dtype in (13, 14, 15):
        return v
    top = (1 << ebits) - 1
    exp = (v.astype(np.uint64) >> np.uint64(fbits)) & np.uint64(top)
    if dtype in (20, 21, 22):
        bias = (1 << (ebits - 1)) - 1
        exp = exp % np.uint64(17) + np.uint64(bias - 8)
    else:
        exp = np.where(exp == top, np.uint64(top - 1), exp)
    cleared = v.astype(np.uint64) & ~np.uint64(top << fbits)
    return (cleared | (exp << np.uint64(fbits))).astype(v.dtype)


@pytest.mark.parametrize("dtype", FLOAT_LEAVES, ids=names(FLOAT_LEAVES))
@pytest.mark.parametrize("a", [0, 1, 511])
def test_rope_every_float_leaf_bit_exact(ref, dtype, a):
    dims = (2, 3, 5, 40)
    rx, hx = both(ref, dtype, dims, values=finite_values(dtype, int(np.prod(dims)), 41).reshape(dims))
    ro, ho = both(ref, dtype, dims, salt=42)
    assert ref.rope(rx.view(), ro.view(), a, 10000.0) > 0, ref.error()
    assert iomo.rope(hx.view(), ho.view(), a, 10000.0) == 0
    assert same_storage(ro, ho)


def test_rope_every_bf16_encoding_and_views(ref):
    dims = (4, 2, 16, 128)
    vals = np.arange(int(np.prod(dims)), dtype=np.uint32).astype(np.uint16).reshape(dims) * 4 + 3
    rx, hx = both(ref, DT_BF16, dims, values=vals)
    ro, ho = both(ref, DT_BF16, (2, 4, 16, 128), salt=44)
    xv = lambda t: t.view().permute([1, 0])
    assert ref.rope(xv(rx), ro.view(), 7, 500000.0) > 0, ref.error()
    assert iomo.rope(xv(hx), ho.view(), 7, 500000.0) == 0
    assert same_storage(ro, ho)


@pytest.mark.parametrize("dtype", [DT_F32, DT_F64])
def test_rope_against_float64_and_rotation_invariants(dtype):
    """No reference involved: the rotation preserves the norm of every pair, position 0 is
    the identity, and the result agrees with a float64 evaluation."""
    H, R, D, a, theta = 2, 9, 64, 3, 10000.0
    x = datagen.normal_f32(H * R * D, 0, 1, 51).astype(np.float64).reshape(1, H, R, D)
    raw = (x.astype(np.float32).view(np.uint32) if dtype == DT_F32 else x.view(np.uint64))
    hx, ho = iomo.HostTensor(dtype, (1, H, R, D)), iomo.HostTensor(dtype, (1, H, R, D))
    hx.view().from_logical(raw)
    assert iomo.rope(hx.view(), ho.view(), a, theta) == 0
    got = ho.view().to_logical()
    got = got.view(np.float32).astype(np.float64) if dtype == DT_F32 else got.view(np.float64)
    xs = x.astype(np.float32).astype(np.float64) if dtype == DT_F32 else x
    c = np.arange(D // 2)
    ang = (a + np.arange(R))[:, None] * theta ** (-2.0 * c / D)[None, :]
    x1, x2 = xs[..., :D // 2], xs[..., D // 2:]
    want = np.concatenate([x1 * np.cos(ang) - x2 * np.sin(ang), x2 * np.cos(ang) + x1 * np.sin(ang)], -1)
    tol = 2e-5 if dtype == DT_F32 else 1e-12          # binary32 pow/angle error grows with the position
    assert np.abs(got - want).max() <= tol * 8
    g1, g2 = got[..., :D // 2], got[..., D // 2:]
    assert np.abs((g1 * g1 + g2 * g2) - (x1 * x1 + x2 * x2)).max() <= 1e-5
    assert iomo.rope(hx.view(), ho.view(), 0, theta) == 0
    assert np.array_equal(ho.view().to_logical()[0, :, 0, :], raw[0, :, 0, :])       # position 0: raw copy


def test_rope_rejections(ref):
    rx, hx = both(ref, DT_F32, (2, 4, 16), salt=1)
    ro, ho = both(ref, DT_F32, (2, 4, 16))
    r3, h3 = both(ref, DT_F32, (2, 4, 15))
    for args in ((0, 0.5), (0, float("inf")), (1 << 24, 10000.0)):
        assert ref.rope(rx.view(), ro.view(), *args) == -1
        assert iomo.rope(hx.view(), ho.view(), *args) == -1
    assert ref.rope(r3.view(), r3.view(), 0, 10000.0) == -1
    assert iomo.rope(h3.view(), h3.view(), 0, 10000.0) == -1
    assert ref.rope(rx.view(), rx.view(), 0, 10000.0) == -1       # output overlaps input
    assert iomo.rope(hx.view(), hx.view(), 0, 10000.0) == -1
    ri, hi = both(ref, DT_I32, (2, 4, 16))
    rj, hj = both(ref, DT_I32, (2, 4, 16))
    assert ref.rope(ri.view(), rj.view(), 0, 10000.0) == -2
    assert iomo.rope(hi.view(), hj.view(), 0, 10000.0) == -2
