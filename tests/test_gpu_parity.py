"""GPU parity: the HIP path, called through the C ABI (include/iomx.h), against
the CPU oracle on the same seeded inputs, and against the committed vectors of
the reference CPU backend.

Bars (written where they are applied):
  elementwise I32/F32/BF16      bit-exact, including untouched tile padding
  RMSNorm                       BF16 <= 1 ulp, F32 relative error <= 1e-5,
                                special classes (NaN / signed zero) exact
  SiLU                          BF16 <= 1 ulp against the CPU oracle; F32 <= 4 ulp
                                against the exact value, the reference's own
                                ceiling for every backend
                                (test/backend/backend_conformance_silu.hpp:492-494,
                                docs/BACKEND_CONTRACT/silu-activation.md:160-162),
                                and so <= 8 ulp against the CPU oracle
  softmax stage                 <= 1 BF16 ulp, masked entries exactly +0,
                                special rows exact
"""
import ctypes as C

import numpy as np
import pytest

import datagen
import golden_cases as gc
import iomo
from iom_amd import iomx
from iomo import DT_BF16, DT_F32, DT_I32, DT_U32, OP_ADD, OP_DIV, OP_MUL, OP_SUB

pytestmark = pytest.mark.gpu

BITS = {DT_BF16: 16, DT_F32: 32, DT_I32: 32, DT_U32: 32}


@pytest.fixture(scope="module", autouse=True)
def _device():
    assert iomx.device_count() >= 1, "no HIP device visible"
    iomx.check(iomx.lib().iomx_set_device(0))
    props = iomx.device_props(0)
    print("device:", props.name.decode(), props.compute_units, "CUs", flush=True)
    yield


def apply(view, steps):
    for name, args in steps:
        view = getattr(view, name)(*args)
    return view


def pair(dtype, dims, salt=None, values=None, fill=0x5A):
    """The same owner in device memory and in the oracle's host memory, padding
    poisoned with `fill` on both sides."""
    dt = iomx.DeviceTensor(dtype, dims, fill=fill)
    ht = iomo.HostTensor(dtype, dims, fill=fill)
    if salt is not None:
        values = datagen.pattern_bits(BITS[dtype], int(np.prod(dims)), salt).reshape(dims)
    if values is not None:
        dt.view().from_host(values)
        ht.view().from_logical(values)
    return dt, ht


def ordered(bits, width):
    bits = bits.astype(np.int64)
    sign = 1 << (width - 1)
    return np.where(bits & sign, (~bits) & ((1 << width) - 1), bits | sign)


def ulp_distance(a, b, width):
    return np.abs(ordered(a, width) - ordered(b, width))


def kernel_name():
    return iomx.last_launch().kernel.decode()


# ------------------------------------------------------------- self tests ----

def test_hardware_bf16_conversion_is_rne_for_every_binary32_encoding():
    bad = C.c_uint64(123)
    iomx.check(iomx.probe_lib().iomx_selftest_bf16_convert(C.byref(bad), None))
    assert bad.value == 0


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32])
@pytest.mark.parametrize("dims,steps", [
    ((20, 35), []), ((2, 3, 17, 33), []), ((3, 16, 48), []), ((1, 1), []),
    ((6, 20, 35), [("slice", (0, 1, 3, 2))]),
    ((4, 3, 16, 32), [("permute", ([1, 0],))]),
    ((5, 3, 16, 24), [("select", (0, 4))]),
    ((2, 64, 256), []),
])
def test_scatter_gather_match_the_closed_form_layout(dtype, dims, steps):
    dt, ht = pair(dtype, dims, salt=0xA0)
    dv, hv = apply(dt.view(), steps), apply(ht.view(), steps)
    vals = datagen.pattern_bits(BITS[dtype], hv.logical_count, 0xA1).reshape(hv.dims)
    dv.from_host(vals)
    hv.from_logical(vals)
    assert np.array_equal(dt.raw(), ht.storage)            # includes poisoned padding
    assert np.array_equal(dv.to_host(), vals)
    dt.free()


# ----------------------------------------------------------------- binary ----

BINARY_CASES = [
    # lhs owner dims, lhs steps, rhs owner dims, rhs steps, out owner dims, out steps, kernel family
    ((2, 17, 33), [], (2, 17, 33), [], (2, 17, 33), [], "binary_padded"),
    ((1, 17, 33), [], (1, 17, 33), [], (1, 17, 33), [], "binary_padded"),
    ((2, 1, 33), [], (1, 17, 1), [], (2, 17, 33), [], "binary_general"),
    ((3, 32, 48), [], (1, 48), [], (3, 32, 48), [], "binary_rowvec"),
    ((1, 48), [], (3, 32, 48), [], (3, 32, 48), [], "binary_rowvec"),
    ((3, 32, 48), [], (32, 1), [], (3, 32, 48), [], "binary_padded"),
    ((3, 1), [], (5, 3, 19), [], (5, 3, 19), [], "binary_padded"),
    ((4, 3, 35, 1), [("permute", ([1, 0],))], (3, 4, 35, 50), [], (3, 4, 35, 50), [], "binary_padded"),
    ((2, 40, 64), [], (2, 1, 1), [], (2, 40, 64), [], "binary_padded"),
    ((1, 1), [], (2, 2, 16, 16), [], (2, 2, 16, 16), [], "binary_padded"),
    ((6, 20, 35), [("slice", (0, 1, 3, 2))], (3, 20, 35), [], (3, 20, 35), [], "binary_padded"),
    ((3, 40, 4100), [], (1, 4100), [], (3, 40, 4100), [], "binary_padded"),
    ((1, 52), [], (4, 3, 21, 52), [("permute", ([1, 0],))], (3, 4, 21, 52), [], "binary_padded"),
    ((5, 500, 272), [], (5, 500, 272), [], (5, 500, 272), [], "binary_padded"),
    ((6, 32, 64), [("slice", (0, 1, 3, 2))], (3, 32, 64), [], (3, 32, 64), [], "binary_planes"),
    ((4, 3, 16, 32), [("permute", ([1, 0],))], (3, 4, 16, 32), [], (3, 4, 16, 32), [], "binary_planes"),
    ((4, 3, 16, 32), [("select", (0, 2))], (1, 16, 32), [], (5, 3, 16, 32), [("select", (0, 4))],
     "binary_planes"),
    ((2, 6, 16, 16), [("reshape_leading", ([3, 4],))], (4, 16, 16), [], (3, 4, 16, 16), [],
     "binary_planes"),
    ((2, 1, 16, 16), [], (1, 5, 16, 16), [], (2, 5, 16, 16), [], "binary_planes"),
    ((5, 64, 256), [], (5, 64, 256), [], (5, 64, 256), [], "binary_planes"),
    ((7, 3, 48, 80), [], (3, 1, 80), [], (7, 3, 48, 80), [], "binary_rowvec"),
    ((4, 160, 4112), [], (1, 4112), [], (4, 160, 4112), [], "binary_rowvec"),
    ((2, 16, 16), [], (1, 16), [], (2, 16, 16), [], "binary_rowvec"),
    # a row vector against planes of a single band: the lane's chunk of the vector must still be
    # found where the launch has no band axis (one plane; two strided leading axes)
    ((16, 64), [], (1, 64), [], (16, 64), [], "binary_rowvec"),
    ((1, 64), [], (16, 64), [], (16, 64), [], "binary_rowvec"),
    ((4, 6, 16, 32), [("slice", (0, 0, 2, 2)), ("slice", (1, 1, 2, 2))], (2, 2, 1, 32), [],
     (2, 2, 16, 32), [], "binary_rowvec"),
    ((1, 3, 16, 48), [("slice", (1, 0, 2, 2))], (5, 2, 1, 48), [("slice", (0, 2, 2, 1))],
     (4, 3, 16, 48), [("slice", (0, 0, 2, 2)), ("slice", (1, 0, 2, 2))], "binary_rowvec"),
]


@pytest.mark.parametrize("dtype", [DT_I32, DT_F32, DT_BF16])
@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
@pytest.mark.parametrize("case", range(len(BINARY_CASES)))
def test_binary_bit_exact_against_oracle(dtype, op, case):
    if op == OP_DIV and dtype == DT_I32:
        pytest.skip("division is defined on the floating leaves only")
    ld, ls, rd, rs, od, os_, family = BINARY_CASES[case]
    dl, hl = pair(dtype, ld, salt=0x100 + case)
    dr, hr = pair(dtype, rd, salt=0x200 + case)
    do, ho = pair(dtype, od, salt=0x300 + case)
    rc = iomx.binary(op, apply(dl.view(), ls), apply(dr.view(), rs), apply(do.view(), os_))
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    assert kernel_name() == family
    big = int(np.prod(od)) > 200000
    assert iomo.binary(op, apply(hl.view(), ls), apply(hr.view(), rs), apply(ho.view(), os_),
                       ieee=big) == 0
    got = do.raw()
    assert np.array_equal(got, ho.storage), f"{np.count_nonzero(got != ho.storage)} raw words differ"
    for t in (dl, dr, do):
        t.free()


@pytest.mark.parametrize("dtype", [DT_I32, DT_F32, DT_BF16])
@pytest.mark.parametrize("dims", [(2, 17, 33), (3, 32, 64)])
@pytest.mark.parametrize("which", ["lhs", "rhs", "both"])
def test_binary_exact_alias(dtype, dims, which):
    da, ha = pair(dtype, dims, salt=1)
    db, hb = pair(dtype, dims, salt=2)
    if which == "lhs":
        rc = iomx.binary(OP_ADD, da.view(), db.view(), da.view())
        iomo.binary(OP_ADD, ha.view(), hb.view(), ha.view())
    elif which == "rhs":
        rc = iomx.binary(OP_SUB, db.view(), da.view(), da.view())
        iomo.binary(OP_SUB, hb.view(), ha.view(), ha.view())
    else:
        rc = iomx.binary(OP_MUL, da.view(), da.view(), da.view())
        iomo.binary(OP_MUL, ha.view(), ha.view(), ha.view())
    assert rc == 0
    assert np.array_equal(da.raw(), ha.storage)
    da.free()
    db.free()


def test_binary_rejections_match_the_reference_rules():
    a = iomx.DeviceTensor(DT_F32, (2, 16, 16))
    b = iomx.DeviceTensor(DT_F32, (3, 16, 16))
    o = iomx.DeviceTensor(DT_F32, (2, 16, 16))
    big = iomx.DeviceTensor(DT_F32, (4, 16, 16))
    assert iomx.binary(OP_ADD, a.view(), b.view(), o.view()) == -1          # not broadcastable
    assert iomx.binary(OP_ADD, a.view(), a.view(), b.view()) == -1          # wrong output shape
    assert iomx.binary(7, a.view(), a.view(), o.view()) == -1               # unknown operation
    # integer division is refused, but only after the shape checks (device_ops_binary.cpp:121-176)
    for dtype in (DT_I32, DT_U32, 1, 5, 12):
        i = iomx.DeviceTensor(dtype, (2, 16, 16))
        j = iomx.DeviceTensor(dtype, (3, 16, 16))
        assert iomx.binary(OP_DIV, i.view(), i.view(), i.view()) == -2
        assert iomx.binary(OP_DIV, i.view(), j.view(), i.view()) == -1
        i.free()
        j.free()
    for code in (0, 18, 23, -1):         # BOOL, F8_E8M0: no arithmetic; unknown leaf codes
        assert iomx.lib().iomx_launch_binary(OP_ADD, code, C.byref(a.view().cview()),
                                             C.byref(a.view().cview()), C.byref(o.view().cview()),
                                             None) == -2
    # an input sharing the output's storage through a different window is forbidden
    assert iomx.binary(OP_ADD, big.view().slice(0, 0, 2), a.view(), big.view().slice(0, 1, 2)) == -1
    for t in (a, b, o, big):
        t.free()


@pytest.mark.parametrize("dtype,op", [(DT_F32, OP_ADD), (DT_I32, OP_ADD), (DT_BF16, OP_ADD),
                                      (DT_BF16, OP_MUL), (DT_F32, OP_MUL), (DT_I32, OP_MUL),
                                      (DT_F32, OP_SUB), (DT_BF16, OP_SUB),
                                      (DT_F32, OP_DIV), (DT_BF16, OP_DIV)])
def test_binary_directed_encodings_cross_product(dtype, op):
    """Every special encoding against every other, F32/BF16 through the codec oracle."""
    if dtype == DT_I32:
        d = np.array([0, 1, 0xFFFFFFFF, 0x80000000, 0x7FFFFFFF, 3, 0x00100000, 0xFFF00000], np.uint32)
    elif dtype == DT_F32:
        base = np.array([0, 0x3F800000, 0x7F800000, 0x7FC00000, 0x7F7FFFFF, 0x00000001, 0x007FFFFF,
                         0x00800000, 0x3F000000, 0x40000000, 0x1FFFFFFF, 0x20000000, 0x33800000,
                         0x4B000001, 0x7FA00001, 0x00400000, 0x5F000000, 0x1F800000], np.uint32)
        d = np.concatenate([base, base | 0x80000000])
    else:
        base = np.array([0, 0x3F80, 0x7F80, 0x7FC0, 0x7F7F, 0x0001, 0x007F, 0x0080, 0x3F00, 0x4000,
                         0x1FC0, 0x2000, 0x1F81, 0x3F81, 0x4301, 0x0040, 0x7FA1, 0x5F00, 0x1F80,
                         0x2001, 0x207F], np.uint16)
        d = np.concatenate([base, base | 0x8000])
    n = d.size
    A = np.repeat(d, n).reshape(1, n, n)
    B = np.tile(d, n).reshape(1, n, n)
    da, ha = pair(dtype, (1, n, n), values=A)
    db, hb = pair(dtype, (1, n, n), values=B)
    do, ho = pair(dtype, (1, n, n), salt=9)
    assert iomx.binary(op, da.view(), db.view(), do.view()) == 0
    assert iomo.binary(op, ha.view(), hb.view(), ho.view()) == 0
    assert np.array_equal(do.raw(), ho.storage)
    for t in (da, db, do):
        t.free()


def test_bf16_every_encoding_against_a_spread_of_partners():
    """All 65536 BF16 values as lhs, against 48 partners chosen across the exponent
    range (includes the subnormal product and quotient bands), bit-exact for all four ops."""
    partners = np.array([0x0000, 0x8000, 0x0001, 0x807F, 0x0080, 0x00FF, 0x0100, 0x1F80, 0x2000,
                         0x2041, 0x3000, 0x3F80, 0xBF80, 0x3F81, 0x3FFF, 0x4000, 0x4049, 0x5F00,
                         0x7F00, 0x7F7F, 0xFF7F, 0x7F80, 0xFF80, 0x7FC0, 0x1001, 0x9001, 0x0800,
                         0x0440, 0x3E80, 0x4080, 0x1F01, 0x1F7F, 0x2080, 0x1E80, 0x0F80, 0x1000,
                         0x2F80, 0x3780, 0x4780, 0x5780, 0x6780, 0x7780, 0x0780, 0x0380, 0x0180,
                         0x00C0, 0x0060, 0x0003], np.uint16)
    rows = partners.size * 16            # 768 rows of 4096 lhs values = 16 partners... 48 x 65536
    A = np.tile(np.arange(65536, dtype=np.uint16), partners.size).reshape(1, rows, 4096)
    B = np.repeat(partners, 65536).reshape(1, rows, 4096)
    da, ha = pair(DT_BF16, A.shape, values=A)
    db, hb = pair(DT_BF16, B.shape, values=B)
    do, ho = pair(DT_BF16, A.shape)
    for op in (OP_ADD, OP_MUL, OP_SUB, OP_DIV):
        assert iomx.binary(op, da.view(), db.view(), do.view()) == 0
        assert iomo.binary(op, ha.view(), hb.view(), ho.view(), ieee=True) == 0
        got = do.raw()
        assert np.array_equal(got, ho.storage), (op, np.count_nonzero(got != ho.storage))
    # the fast element rule used above is itself pinned to the codec on a sample
    idx = np.arange(0, A.size, 1021)
    Lr = iomo.lib()
    a_flat, b_flat = A.reshape(-1), B.reshape(-1)
    for i in idx[:3000]:
        for op in (OP_MUL, OP_DIV):
            assert Lr.iomo_scalar_binary(op, DT_BF16, int(a_flat[i]), int(b_flat[i])) == \
                Lr.iomo_scalar_binary_ieee(op, DT_BF16, int(a_flat[i]), int(b_flat[i]))
    for t in (da, db, do):
        t.free()


# ---------------------------------------------------------------- RMSNorm ----

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


def assert_float_close(got, want, dtype, what, bf16_ulp=1, f32_rel=1e-5, f32_ulp=None):
    """NaN class, zero sign and infinities exact; the rest within the stated bar."""
    got = got.reshape(-1)
    want = want.reshape(-1)
    if dtype == DT_BF16:
        g, w = datagen.bf16_to_f32(got), datagen.bf16_to_f32(want)
    else:
        g, w = got.view(np.float32), want.view(np.float32)
    gn, wn = np.isnan(g), np.isnan(w)
    assert np.array_equal(gn, wn), f"{what}: NaN positions differ"
    nan_bits = 0x7FC0 if dtype == DT_BF16 else 0x7FC00000
    assert np.all(got[gn] == nan_bits), f"{what}: NaN is not the positive canonical encoding"
    special = wn | np.isinf(w) | (w == 0)
    assert np.array_equal(got[special & ~wn], want[special & ~wn]), f"{what}: zero/inf class differs"
    rest = ~special
    if dtype == DT_BF16:
        d = ulp_distance(got[rest], want[rest], 16)
        assert d.size == 0 or d.max() <= bf16_ulp, f"{what}: {d.max()} BF16 ulp"
    elif f32_ulp is not None:
        d = ulp_distance(got[rest], want[rest], 32)
        assert d.size == 0 or d.max() <= f32_ulp, f"{what}: {d.max()} F32 ulp"
    else:
        with np.errstate(all="ignore"):
            rel = np.abs(g[rest].astype(np.float64) - w[rest]) / np.abs(w[rest].astype(np.float64))
        # results in the subnormal range are compared by ulp instead
        tiny = np.abs(w[rest]) < 1e-37
        d = ulp_distance(got[rest][tiny], want[rest][tiny], 32)
        assert rel[~tiny].size == 0 or rel[~tiny].max() <= f32_rel, f"{what}: rel {rel[~tiny].max()}"
        assert d.size == 0 or d.max() <= 64


def silu_exact_f32_bits(x_bits):
    """x*sigmoid(x) evaluated in binary64 and rounded once to binary32."""
    x = x_bits.reshape(-1).view(np.float32).astype(np.float64)
    with np.errstate(all="ignore"):
        y = np.where(x < -700.0, x * np.exp(x), x / (1.0 + np.exp(-x)))
        y = np.where(np.isneginf(x), -0.0, y)
        y = np.where(x == 0, x, y)
        return y.astype(np.float32).view(np.uint32)


RMS_CASES = [
    ((1, 1), [], "rmsnorm_generic"), ((15, 16), [], "rmsnorm_band"), ((17, 33), [], "rmsnorm_generic"),
    ((16, 31), [], "rmsnorm_generic"), ((3, 5, 130), [], "rmsnorm_generic"),
    ((2, 3, 17, 64), [("permute", ([1, 0],))], "rmsnorm_band"),
    ((6, 16, 48), [("slice", (0, 0, 3, 2))], "rmsnorm_band"),
    ((40, 2048), [], "rmsnorm_split"), ((33, 256), [], "rmsnorm_band"), ((16, 512), [], "rmsnorm_band"),
    ((2, 20, 1024), [], None), ((48, 4096), [], "rmsnorm_split"), ((20, 5632), [], None),
    ((16, 8192), [], None), ((16, 16384), [], "rmsnorm_split"), ((4, 40000), [], None),
    # wide rows cut into 2..8 parts per band, with tail rows and strided planes
    ((35, 32768), [], "rmsnorm_split"), ((3, 19, 16384), [("slice", (0, 0, 2, 2))], "rmsnorm_split"),
    ((2, 2, 33, 8192), [("permute", ([1, 0],))], None), ((2, 65536), [], None),
]


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32])
@pytest.mark.parametrize("case", range(len(RMS_CASES)))
@pytest.mark.parametrize("kind", ["normal", "outliers", "bits"])
def test_rmsnorm_against_oracle(dtype, case, kind):
    dims, steps, family = RMS_CASES[case]
    dx, hx = pair(dtype, dims, values=float_values(dtype, dims, 31 + case, kind))
    F = dims[-1]
    w = datagen.uniform_f32(F, 0.5, 1.5, 32)
    wl = (datagen.bf16_rne(w) if dtype == DT_BF16 else w.view(np.uint32)).reshape(1, F)
    dw, hw = pair(dtype, (1, F), values=wl)
    dvx, hvx = apply(dx.view(), steps), apply(hx.view(), steps)
    do, ho = pair(dtype, hvx.dims, salt=99)
    rc = iomx.rmsnorm(dvx, dw.view(), do.view(), 1e-5)
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    if family:
        assert kernel_name() == family
    assert iomo.rmsnorm(hvx, hw.view(), ho.view(), 1e-5) == 0
    got, want = do.view().to_host(), ho.view().to_logical()
    if kind == "bits":
        # rows of raw hash bits are NaN/inf rows almost surely: the class must match
        assert_float_close(got, want, dtype, "rmsnorm bits", bf16_ulp=1, f32_rel=1e-5)
    else:
        assert_float_close(got, want, dtype, "rmsnorm", bf16_ulp=1, f32_rel=1e-5)
    # padding of the output owner untouched
    pad = iomo.tile_plane(np.ones(hvx.dims, ho.storage.dtype)) == 0
    assert np.array_equal(do.raw()[pad], ho.storage[pad])
    for t in (dx, dw, do):
        t.free()


def test_rmsnorm_all_ones_closed_form_and_special_rows():
    feats = 64
    rows = np.ones((20, feats), np.float32)
    rows[1, 5] = np.nan
    rows[2, :] = -2.0
    rows[2, 7] = np.inf
    rows[3, :] = 0.0
    rows[3, 3] = -0.0
    dx, hx = pair(DT_F32, rows.shape, values=rows.view(np.uint32))
    dw, hw = pair(DT_F32, (1, feats), values=np.ones((1, feats), np.float32).view(np.uint32))
    do, ho = pair(DT_F32, rows.shape)
    assert iomx.rmsnorm(dx.view(), dw.view(), do.view(), 1e-5) == 0
    assert iomo.rmsnorm(hx.view(), hw.view(), ho.view(), 1e-5) == 0
    got = do.view().to_host()
    assert np.array_equal(got, ho.view().to_logical())     # exact here: every sum is exact
    inv = np.float32(1.0) / np.sqrt(np.float32(1.0) + np.float32(1e-5))
    assert np.all(got[0].view(np.float32) == inv)
    assert np.all(got[1] == 0x7FC00000)
    assert got[2, 7] == 0x7FC00000 and got[2, 0] == 0x80000000
    assert got[3, 3] == 0x80000000 and got[3, 0] == 0
    for t in (dx, dw, do):
        t.free()


def test_rmsnorm_rejections():
    x = iomx.DeviceTensor(DT_F32, (4, 32))
    o = iomx.DeviceTensor(DT_F32, (4, 32))
    w = iomx.DeviceTensor(DT_F32, (1, 32))
    wb = iomx.DeviceTensor(DT_F32, (2, 32))
    assert iomx.rmsnorm(x.view(), wb.view(), o.view(), 1e-5) == -1
    assert iomx.rmsnorm(x.view(), w.view(), x.view(), 1e-5) == -1
    assert iomx.rmsnorm(x.view(), w.view(), o.view(), -1.0) == -1
    assert iomx.rmsnorm(x.view(), w.view(), o.view(), float("nan")) == -1
    assert iomx.rmsnorm(x.view(), w.view(), o.view(), float("inf")) == -1
    xi, oi, wi = (iomx.DeviceTensor(DT_I32, d) for d in ((4, 32), (4, 32), (1, 32)))
    assert iomx.rmsnorm(xi.view(), wi.view(), oi.view(), 1e-5) == -2
    for t in (x, o, w, wb, xi, oi, wi):
        t.free()


# ------------------------------------------------------------ SiLU / copy ----

@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32])
@pytest.mark.parametrize("dims,steps,family", [
    ((17, 33), [], "silu_padded"), ((3, 16, 48), [], "silu_planes"),
    ((4, 2, 16, 16), [("permute", ([1, 0],))], "silu_planes"), ((64, 5632), [], "silu_planes"),
])
@pytest.mark.parametrize("kind", ["normal", "bits"])
def test_silu_against_oracle(dtype, dims, steps, family, kind):
    dx, hx = pair(dtype, dims, values=float_values(dtype, dims, 41, kind))
    dvx, hvx = apply(dx.view(), steps), apply(hx.view(), steps)
    do, ho = pair(dtype, hvx.dims, salt=98)
    rc = iomx.silu(dvx, do.view())
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    assert kernel_name() == family
    assert iomo.silu(hvx, ho.view()) == 0
    got = do.view().to_host()
    assert_float_close(got, ho.view().to_logical(), dtype, "silu", bf16_ulp=1, f32_ulp=8)
    if dtype == DT_F32:
        assert_float_close(got, silu_exact_f32_bits(hvx.to_logical()), dtype, "silu vs exact",
                           f32_ulp=4)
    pad = iomo.tile_plane(np.ones(hvx.dims, ho.storage.dtype)) == 0
    assert np.array_equal(do.raw()[pad], ho.storage[pad])
    dx.free()
    do.free()


def test_silu_every_bf16_encoding():
    x = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    dx, hx = pair(DT_BF16, x.shape, values=x)
    do, ho = pair(DT_BF16, x.shape)
    assert iomx.silu(dx.view(), do.view()) == 0
    assert iomo.silu(hx.view(), ho.view()) == 0
    got, want = do.view().to_host(), ho.view().to_logical()
    assert_float_close(got, want, DT_BF16, "silu all bf16", bf16_ulp=1)
    print("silu bf16: exact matches", int((got == want).sum()), "of 65536", flush=True)
    dx.free()
    do.free()


def test_silu_f32_tails_and_specials():
    xs = np.array([-104.0, -103.9, -90.0, -88.0, -87.0, -20.0, -1e-30, 1e-30, 88.0, 100.0, 3e38,
                   -3e38, np.inf, -np.inf, 0.0, -0.0, np.nan, -1.0, 1.0, 0.5, -0.5, -17.0, -40.0,
                   -150.0, -208.0, -300.0], np.float32)
    x = np.zeros((16, 16), np.float32)
    x.reshape(-1)[:xs.size] = xs
    dx, hx = pair(DT_F32, x.shape, values=x.view(np.uint32))
    do, ho = pair(DT_F32, x.shape)
    assert iomx.silu(dx.view(), do.view()) == 0
    assert iomo.silu(hx.view(), ho.view()) == 0
    got, want = do.view().to_host(), ho.view().to_logical()
    assert_float_close(got, want, DT_F32, "silu tails", f32_ulp=8)
    assert_float_close(got, silu_exact_f32_bits(x.view(np.uint32)), DT_F32, "silu tails vs exact",
                       f32_ulp=4)
    t = got.reshape(-1)[0]
    assert t & 0x80000000 and t & 0x7FFFFFFF          # -104 keeps a nonzero negative tail
    dx.free()
    do.free()


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32])
@pytest.mark.parametrize("dims", [(3, 16, 48), (17, 33), (64, 5632)])
def test_fused_silu_mul_equals_the_two_operation_sequence(dtype, dims):
    g = iomx.DeviceTensor(dtype, dims)
    u = iomx.DeviceTensor(dtype, dims)
    g.view().from_host(float_values(dtype, dims, 71, "normal"))
    u.view().from_host(float_values(dtype, dims, 72, "normal"))
    act, two, one = (iomx.DeviceTensor(dtype, dims, fill=0x5A) for _ in range(3))
    assert iomx.silu(g.view(), act.view()) == 0
    assert iomx.binary(OP_MUL, act.view(), u.view(), two.view()) == 0
    assert iomx.silu_mul(g.view(), u.view(), one.view()) == 0
    assert np.array_equal(one.raw(), two.raw())
    for t in (g, u, act, two, one):
        t.free()


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32, DT_I32])
@pytest.mark.parametrize("sd,ss,dd,ds,family", [
    ((2, 17, 33), [], (2, 17, 33), [], "copy_padded"),
    ((6, 20, 35), [("slice", (0, 1, 3, 2))], (3, 20, 35), [], "copy_padded"),
    ((4, 3, 16, 32), [("permute", ([1, 0],))], (3, 4, 16, 32), [], "copy_planes"),
    ((3, 16, 16), [], (5, 3, 16, 16), [("select", (0, 1))], "copy_planes"),
    ((8, 64, 512), [], (8, 64, 512), [], "copy_planes"),
])
def test_copy_bit_exact(dtype, sd, ss, dd, ds, family):
    ds_, hs = pair(dtype, sd, salt=51)
    dd_, hd = pair(dtype, dd, salt=52)
    assert iomx.copy(apply(ds_.view(), ss), apply(dd_.view(), ds)) == 0
    assert kernel_name() == family
    assert iomo.copy(apply(hs.view(), ss), apply(hd.view(), ds)) == 0
    assert np.array_equal(dd_.raw(), hd.storage)
    # an identical window is a no-op
    assert iomx.copy(dd_.view(), dd_.view()) == 0 and kernel_name() == "copy_noop"
    ds_.free()
    dd_.free()


# ---------------------------------------------------------------- softmax ----

def gpu_softmax(scores, a, L, scale=1.0, rows=None, pcols=None):
    scores = np.ascontiguousarray(scores, np.float32)
    planes, heads, prow, scol = scores.shape
    pcols = scol if pcols is None else pcols
    sb = iomx.Buffer(scores.nbytes)
    pb = iomx.Buffer(planes * heads * prow * pcols * 2)
    sb.upload(scores)
    pb.fill(0xAA)
    d = iomx.softmax_desc(sb.ptr.value, pb.ptr.value, planes, heads, prow, scol, a, L, scale, rows)
    d.probability_layout = iomx.dense_layout(heads, prow, pcols)
    rc = iomx.softmax(d)
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    iomx.synchronize()
    out = pb.download(np.uint16).reshape(planes, heads, prow, pcols)
    sb.free()
    pb.free()
    return out


def test_softmax_special_rows_exact():
    inf = np.inf
    rows = np.zeros((1, 1, 8, 4), np.float32)
    rows[0, 0, 0] = [np.nan, 0, 0, 0]
    rows[0, 0, 1] = [inf, inf, -3, 99]
    rows[0, 0, 2] = [-inf, -inf, -inf, 77]
    rows[0, 0, 3] = [0, -inf, 5, 5]
    rows[0, 0, 4] = [0, -90.0, 5, 5]
    got = gpu_softmax(rows, a=4, L=3)
    want = iomo.softmax(rows, a=4, L=3)
    assert np.array_equal(got, want)
    two = np.zeros((1, 1, 2, 4), np.float32)
    two[0, 0, 0] = [0, -inf, 1, 1]
    two[0, 0, 1] = [0, -90.0, 1, 1]
    got = gpu_softmax(two, a=4, L=2)
    assert list(got[0, 0, 0]) == [0x3F80, 0, 0, 0]
    assert got[0, 0, 1, 0] == 0x3F80 and 0 < got[0, 0, 1, 1] < 0x0080 and got[0, 0, 1, 2] == 0


@pytest.mark.parametrize("shape,a,L,family", [
    ((1, 1, 33, 200), 0, 150, "softmax_rows"),
    ((2, 3, 64, 256), 0, 256, "softmax_rows"),
    ((1, 2, 128, 2048), 0, 2048, "softmax_rows"),
    ((1, 2, 16, 2048), 2047, 2048, "softmax_rows"),
    ((1, 1, 8, 4096), 4000, 4096, "softmax_rows"),
    ((1, 1, 8, 1000), 10, 999, "softmax_rows"),
    ((1, 1, 5, 777), 3, 700, "softmax_generic"),
    ((1, 1, 4, 5000), 4990, 5000, "softmax_generic"),
])
def test_softmax_against_oracle(shape, a, L, family):
    n = int(np.prod(shape))
    s = datagen.normal_f32(n, 0, 3, 61).reshape(shape)
    # causal mask carried as data as well: strict upper triangle = -inf
    r = np.arange(shape[2])[:, None]
    t = np.arange(shape[3])[None, :]
    s[..., t > a + r] = -np.inf
    got = gpu_softmax(s, a=a, L=L, scale=0.125)
    assert kernel_name() == family
    want = iomo.softmax(s, a=a, L=L, scale=0.125)
    masked = np.broadcast_to((t > a + r) | (t >= L), shape)
    assert np.all(got[masked] == 0)                        # exactly +0
    assert_float_close(got[~masked], want[~masked], DT_BF16, "softmax", bf16_ulp=1)


def test_softmax_physical_rows_and_columns_beyond_the_logical_extent_are_zero():
    s = datagen.normal_f32(1 * 2 * 32 * 64, 0, 3, 62).reshape(1, 2, 32, 64)
    got = gpu_softmax(s, a=0, L=40, rows=20, pcols=96)
    want = iomo.softmax(s, a=0, L=40, rows=20)
    assert np.all(got[:, :, 20:, :] == 0)
    assert np.all(got[:, :, :, 64:] == 0)
    assert_float_close(got[:, :, :20, :64], want[:, :, :20, :], DT_BF16, "softmax phys", bf16_ulp=1)


# ------------------------------------------------------- reference vectors ----

@pytest.mark.parametrize("case", gc.manifest(), ids=gc.case_id)
def test_reference_cpu_vectors(case):
    z = gc.arrays()
    key, dtype, kind = case["key"], case["dtype"], case["kind"]
    if kind == "binary_directed":
        dims = tuple(case["dims"])
        a, b, o = (iomx.DeviceTensor(dtype, dims) for _ in range(3))
        a.view().from_host(z[key + "_a"])
        b.view().from_host(z[key + "_b"])
        assert iomx.binary(case["op"], a.view(), b.view(), o.view()) == 0
        assert np.array_equal(o.view().to_host(), z[key + "_y"])
        tensors = [a, b, o]
    elif kind == "binary_view":
        tensors, views = [], []
        for name in ("lhs", "rhs", "out"):
            dims, steps, values = gc.operand(case[name], dtype)
            t = iomx.DeviceTensor(dtype, dims)
            t.view().from_host(values)
            tensors.append(t)
            views.append(gc.apply(t.view(), steps))
        assert iomx.binary(case["op"], *views) == 0
        assert np.array_equal(tensors[2].view().to_host(), z[key + "_y"])
    elif kind == "rmsnorm":
        R, F = case["dims"]
        x, w, o = (iomx.DeviceTensor(dtype, d) for d in ((R, F), (1, F), (R, F)))
        x.view().from_host(z[key + "_x"])
        w.view().from_host(z[key + "_w"].reshape(1, F))
        assert iomx.rmsnorm(x.view(), w.view(), o.view(), case["eps"]) == 0
        assert_float_close(o.view().to_host(), z[key + "_y"], dtype, key)
        tensors = [x, w, o]
    else:
        dims = tuple(case["dims"])
        x, o = iomx.DeviceTensor(dtype, dims), iomx.DeviceTensor(dtype, dims)
        x.view().from_host(z[key + "_x"])
        assert iomx.silu(x.view(), o.view()) == 0
        assert_float_close(o.view().to_host(), z[key + "_y"], dtype, key, bf16_ulp=1, f32_ulp=8)
        tensors = [x, o]
    for t in tensors:
        t.free()
