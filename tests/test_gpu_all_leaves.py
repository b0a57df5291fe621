"""GPU parity of the every-leaf path, through the C ABI, against the CPU oracle
(itself checked against the compiled reference for all 23 leaves): packed
storage and host transfer, copy, the binary operations over the 21 numeric
leaves, SiLU and RMSNorm over the 9 floating leaves.

Bars: transfers, copies and binary results are bit-exact including untouched tile
padding (for F64 against the binary64-carrier rule; the x87 carrier of the CPU
codec differs from it by one unit in rare double-rounding cases, counted in the
CPU tests); SiLU and RMSNorm at most one encoding step of the leaf, special
classes exact.
"""
import numpy as np
import pytest

import datagen
import iomo
from iom_amd import iomx
from iomo import (ALL_LEAVES, DT_BOOL, DT_F16, DT_F64, DT_F8_E8M0, DT_I16, DT_I64, DT_U16, DT_U4,
                  DT_U64, FLOAT_LEAVES, LEAF_BITS, LEAF_NAME, NUMERIC_LEAVES, OP_ADD, OP_DIV, OP_MUL, OP_SUB)

pytestmark = pytest.mark.gpu

STREAMING = (iomo.DT_I32, iomo.DT_U32, iomo.DT_F32, iomo.DT_BF16)          # covered by test_gpu_parity
# leaves that also run on the chunk-mapped kernels; the rest run on the tile-row kernels
CHUNKED = STREAMING + (iomo.DT_I8, iomo.DT_U8, DT_I16, DT_U16, DT_I64, DT_U64, DT_F16, DT_F64)
ROWS_NUMERIC = [d for d in NUMERIC_LEAVES if d not in STREAMING]
ROWS_FLOAT = [d for d in FLOAT_LEAVES if d not in STREAMING]


def on_rows(dtype):
    return dtype not in CHUNKED
NARROW = [d for d in ROWS_NUMERIC if LEAF_BITS[d] <= 8]
names = lambda ds: [LEAF_NAME[d] for d in ds]


@pytest.fixture(scope="module", autouse=True)
def _device():
    assert iomx.device_count() >= 1
    iomx.check(iomx.lib().iomx_set_device(0))
    yield


def apply(view, steps):
    for name, args in steps:
        view = getattr(view, name)(*args)
    return view


def pattern(dtype, count, salt):
    v = datagen.pattern_bits(LEAF_BITS[dtype], count, salt)
    return v & 1 if dtype == DT_BOOL else v


def pair(dtype, dims, salt=None, values=None, fill=0x5A):
    dt = iomx.DeviceTensor(dtype, dims, fill=fill)
    ht = iomo.HostTensor(dtype, dims, fill=fill)
    if salt is not None:
        values = pattern(dtype, int(np.prod(dims)), salt).reshape(dims)
    if values is not None:
        dt.view().from_host(values)
        ht.view().from_logical(values)
    return dt, ht


def same_storage(dt, ht):
    return np.array_equal(dt.raw().view(np.uint8), ht.storage.view(np.uint8))


def kernel_name():
    return iomx.last_launch().kernel.decode()


# -- transfer / copy ----------------------------------------------------------------

@pytest.mark.parametrize("dtype", ALL_LEAVES, ids=names(ALL_LEAVES))
@pytest.mark.parametrize("dims,steps", [
    ((17, 33), []), ((3, 5, 7), []), ((2, 16, 32), []), ((1, 1), []), ((2, 3, 1, 50), []),
    ((6, 20, 35), [("slice", (0, 1, 3, 2))]),
    ((4, 3, 16, 32), [("permute", ([1, 0],))]),
    ((2, 64, 272), []),
])
def test_transfer_bit_exact(dtype, dims, steps):
    dt, ht = pair(dtype, dims, salt=0xA0)
    dv, hv = apply(dt.view(), steps), apply(ht.view(), steps)
    vals = pattern(dtype, hv.logical_count, 0xA1).reshape(hv.dims)
    dv.from_host(vals)
    hv.from_logical(vals)
    assert same_storage(dt, ht)                         # poisoned padding included
    assert np.array_equal(dv.to_host(), vals)
    # the packed stream, with the unused bits of a last partial byte zeroed
    assert np.array_equal(dv.to_host_stream(), iomo.pack_bits(vals, LEAF_BITS[dtype]))
    dt.free()


@pytest.mark.parametrize("dtype", ALL_LEAVES, ids=names(ALL_LEAVES))
@pytest.mark.parametrize("dims,family", [((17, 19), "rows"), ((16, 32), "copy_planes")])
def test_copy_between_views(dtype, dims, family):
    ds, hs = pair(dtype, (4, 3) + dims, salt=31)
    dd, hd = pair(dtype, (3, 6) + dims, salt=32)
    src = lambda t: t.view().slice(0, 0, 2, 2).permute([1, 0])
    dst = lambda t: t.view().slice(1, 1, 2, 3)
    assert iomx.copy(src(ds), dst(dd)) == 0
    if family == "copy_planes":
        assert kernel_name() == "copy_planes"
    else:
        assert kernel_name() == ("copy_padded" if LEAF_BITS[dtype] in (8, 16, 32, 64) else "rows_copy")
    assert iomo.copy(src(hs), dst(hd)) == 0
    assert same_storage(dd, hd)
    ds.free()
    dd.free()


# -- binary ---------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", NARROW, ids=names(NARROW))
@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
def test_binary_every_pair_of_a_narrow_leaf(dtype, op):
    if op == OP_DIV and dtype not in FLOAT_LEAVES:
        pytest.skip("division is defined on the floating leaves only")
    n = 1 << LEAF_BITS[dtype]
    every = np.arange(n).astype(np.uint8)
    dl, hl = pair(dtype, (n, 1), values=every.reshape(n, 1))
    dr, hr = pair(dtype, (1, n), values=every.reshape(1, n))
    do, ho = pair(dtype, (n, n))
    assert iomx.binary(op, dl.view(), dr.view(), do.view()) == 0
    assert kernel_name() == ("rows_binary" if on_rows(dtype) else "binary_general")
    assert iomo.binary(op, hl.view(), hr.view(), ho.view()) == 0          # the codec itself
    assert same_storage(do, ho)
    for t in (dl, dr, do):
        t.free()


F8_CONVERTED = [iomo.DT_F8_E4M3FN, iomo.DT_F8_E5M2]


def f8_table(dtype):
    """Value of each of the 256 encodings (src/shared/scalar_binary_codec.hpp:45-66): the top
    exponent of F8_E4M3FN is NaN throughout, that of F8_E5M2 holds the infinities and NaN."""
    ebits, fbits, bias = {iomo.DT_F8_E4M3FN: (4, 3, 7), iomo.DT_F8_E5M2: (5, 2, 15)}[dtype]
    raw = np.arange(256)
    frac, exp = raw & ((1 << fbits) - 1), (raw >> fbits) & ((1 << ebits) - 1)
    value = np.where(exp == 0, frac * 2.0 ** (1 - bias - fbits), (1 + frac / (1 << fbits)) * 2.0 ** (exp - bias))
    top = exp == (1 << ebits) - 1
    special = np.where((frac == 0) & (dtype == iomo.DT_F8_E5M2), np.inf, np.nan)
    return np.where(raw >> 7, -1.0, 1.0) * np.where(top, special, value)


def regrouped(in_range):
    """Indices of a row of 288: those in range first, padded to whole tile rows, then the others."""
    good, bad = np.flatnonzero(in_range), np.flatnonzero(~in_range)
    if good.size:
        good = np.concatenate([good, np.full(-good.size % 16, good[0])])
    row = np.concatenate([good, bad]).astype(np.int64)
    return np.concatenate([row, np.full(288 - row.size, row[-1])])


@pytest.mark.parametrize("dtype", F8_CONVERTED, ids=names(F8_CONVERTED))
@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
def test_f8_pairs_regrouped_by_the_range_of_their_result(dtype, op):
    """The tile-row kernel rounds a tile row with the conversion instructions when all sixteen
    results are numbers within the leaf's finite range, and element by element otherwise; in the
    all-pairs table above a pair in range often shares its tile row with one that is not.  Here a
    row holds one left operand against all 256 right operands regrouped, those with a result in
    range first and padded to whole tile rows, so every such pair goes through the instructions."""
    table = f8_table(dtype)
    limit = {iomo.DT_F8_E4M3FN: 240.0, iomo.DT_F8_E5M2: 57344.0}[dtype]
    rhs = np.zeros((256, 288), np.uint8)
    with np.errstate(all="ignore"):
        for x in range(256):
            r = {OP_ADD: table[x] + table, OP_SUB: table[x] - table, OP_MUL: table[x] * table,
                 OP_DIV: table[x] / table}[op]
            rhs[x] = regrouped(np.abs(r) <= limit)
    lhs = np.repeat(np.arange(256, dtype=np.uint8).reshape(256, 1), 288, axis=1)
    dl, hl = pair(dtype, (256, 288), values=lhs)
    dr, hr = pair(dtype, (256, 288), values=rhs)
    do, ho = pair(dtype, (256, 288))
    assert iomx.binary(op, dl.view(), dr.view(), do.view()) == 0
    assert kernel_name() == "rows_binary"
    assert iomo.binary(op, hl.view(), hr.view(), ho.view()) == 0
    assert same_storage(do, ho)
    for t in (dl, dr, do):
        t.free()


@pytest.mark.parametrize("dtype", F8_CONVERTED, ids=names(F8_CONVERTED))
def test_f8_silu_regrouped_by_the_range_of_its_result(dtype):
    """Every finite encoding in tile rows of finite encodings only (see the test above)."""
    table = f8_table(dtype)
    vals = regrouped(np.isfinite(table)).astype(np.uint8).reshape(1, 288)
    dx, hx = pair(dtype, (1, 288), values=vals)
    do, ho = pair(dtype, (1, 288))
    assert iomx.silu(dx.view(), do.view()) == 0
    assert kernel_name() == "rows_silu"
    assert iomo.silu(hx.view(), ho.view()) == 0
    got, want = do.view().to_host().reshape(-1), ho.view().to_logical().reshape(-1)
    nan = is_nan(want, dtype)
    assert np.array_equal(got[nan], want[nan])
    assert steps_apart(got[~nan], want[~nan], dtype).max() <= 1
    dx.free()
    do.free()


@pytest.mark.parametrize("dtype", [iomo.DT_U2, iomo.DT_I4, iomo.DT_F4_E2M1, iomo.DT_F6_E2M3, iomo.DT_F8_E5M2],
                         ids=["U2", "I4", "F4_E2M1", "F6_E2M3", "F8_E5M2"])
def test_row_kernel_with_several_planes_per_lane(dtype):
    """A launch large enough that a lane of the tile-row kernel walks two or more planes (the grid
    covers fewer planes than the view has): seven planes, every other one of a larger owner, so the
    last lane group has a plane less; a row vector on the right.  Against the oracle, padding and
    skipped planes untouched."""
    dims, owner = (7, 1024, 4096), (14, 1024, 4096)
    dl, hl = pair(dtype, owner, salt=0x771)
    dr, hr = pair(dtype, (1, 4096), salt=0x772)
    do, ho = pair(dtype, owner, salt=0x773)
    if dtype == iomo.DT_F8_E5M2:                      # finite magnitudes below 2: the converted route
        for t, h, d in ((dl, hl, owner), (dr, hr, (1, 4096))):
            v = (pattern(dtype, int(np.prod(d)), 0x774 + len(d)) & 0xBF).reshape(d)
            t.view().from_host(v)
            h.view().from_logical(v)
    sl = lambda t: t.view().slice(0, 1, 7, 2)
    assert iomx.binary(OP_MUL, sl(dl), dr.view(), sl(do)) == 0
    assert kernel_name() == "rows_binary"
    launch = iomx.last_launch()
    assert launch.work_items == 7 * 1024 * 256                  # every tile row of every plane ...
    assert iomo.binary(OP_MUL, sl(hl), hr.view(), sl(ho), ieee=True) == 0
    assert same_storage(do, ho)
    for t in (dl, dr, do):
        t.free()


@pytest.mark.parametrize("dtype", [iomo.DT_I8, iomo.DT_U8], ids=["I8", "U8"])
@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB])
def test_binary_every_8bit_pair_on_whole_planes(dtype, op):
    """Both operands materialised as [256,256], so the packed-lane arithmetic of the
    streaming kernel sees every operand pair."""
    every = np.arange(256, dtype=np.uint8)
    a = np.repeat(every.reshape(256, 1), 256, axis=1)
    b = np.repeat(every.reshape(1, 256), 256, axis=0)
    dl, hl = pair(dtype, (256, 256), values=a)
    dr, hr = pair(dtype, (256, 256), values=b)
    do, ho = pair(dtype, (256, 256))
    assert iomx.binary(op, dl.view(), dr.view(), do.view()) == 0
    assert kernel_name() == "binary_planes"
    assert iomo.binary(op, hl.view(), hr.view(), ho.view()) == 0
    assert same_storage(do, ho)
    for t in (dl, dr, do):
        t.free()


@pytest.mark.parametrize("dtype", [DT_I16, DT_U16, DT_F16], ids=["I16", "U16", "F16"])
@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
def test_binary_16bit_pairs_on_whole_planes(dtype, op):
    if op == OP_DIV and dtype != DT_F16:
        pytest.skip("division is defined on the floating leaves only")
    """4 million operand pairs (specials against everything) as whole planes: the packed
    two-lane integer arithmetic and the hardware F16 conversions, against the codec."""
    n = 2048
    spec = half_specials()
    vals = np.concatenate([spec, datagen.pattern_bits(16, n - spec.size, 141)])
    other = np.concatenate([datagen.pattern_bits(16, n - spec.size, 142), spec])
    a = np.repeat(vals.reshape(n, 1), n, axis=1)
    b = np.repeat(other.reshape(1, n), n, axis=0)
    dl, hl = pair(dtype, (n, n), values=a)
    dr, hr = pair(dtype, (n, n), values=b)
    do, ho = pair(dtype, (n, n))
    assert iomx.binary(op, dl.view(), dr.view(), do.view()) == 0
    assert kernel_name() == "binary_planes"
    assert iomo.binary(op, hl.view(), hr.view(), ho.view(), ieee=True) == 0
    assert same_storage(do, ho)
    for t in (dl, dr, do):
        t.free()


def test_f16_streaming_arithmetic_equals_the_codec_rule_for_every_pair():
    import ctypes as C
    bad = C.c_uint64(123)
    iomx.check(iomx.probe_lib().iomx_selftest_f16_binary(C.byref(bad), None))
    assert bad.value == 0


ROWS_CASES = [
    ((2, 17, 33), [], (2, 17, 33), [], (2, 17, 33), []),
    ((2, 1, 33), [], (1, 17, 1), [], (2, 17, 33), []),
    ((3, 32, 48), [], (1, 48), [], (3, 32, 48), []),
    ((1, 48), [], (3, 32, 48), [], (3, 32, 48), []),
    ((3, 32, 48), [], (32, 1), [], (3, 32, 48), []),
    ((1, 1), [], (2, 2, 16, 16), [], (2, 2, 16, 16), []),
    ((6, 20, 35), [("slice", (0, 1, 3, 2))], (3, 20, 35), [], (3, 20, 35), []),
    ((4, 3, 16, 32), [("permute", ([1, 0],))], (3, 4, 16, 32), [], (3, 4, 16, 32), []),
    ((4, 3, 16, 32), [("select", (0, 2))], (1, 16, 32), [], (5, 3, 16, 32), [("select", (0, 4))]),
    ((2, 1, 16, 16), [], (1, 5, 16, 16), [], (2, 5, 16, 16), []),
    ((5, 64, 272), [], (5, 64, 272), [], (5, 64, 272), []),
    ((3, 40, 4112), [], (1, 4112), [], (3, 40, 4112), []),
    ((16, 64), [], (1, 64), [], (16, 64), []),
    ((4, 6, 16, 32), [("slice", (0, 0, 2, 2)), ("slice", (1, 1, 2, 2))], (2, 2, 1, 32), [], (2, 2, 16, 32), []),
]


@pytest.mark.parametrize("dtype", ROWS_NUMERIC, ids=names(ROWS_NUMERIC))
@pytest.mark.parametrize("case", range(len(ROWS_CASES)))
def test_binary_views_and_broadcasts(dtype, case):
    ld, ls, rd, rs, od, os_ = ROWS_CASES[case]
    op = (OP_ADD, OP_MUL, OP_SUB)[case % 3]
    dl, hl = pair(dtype, ld, salt=0x100 + case)
    dr, hr = pair(dtype, rd, salt=0x200 + case)
    do, ho = pair(dtype, od, salt=0x300 + case)
    rc = iomx.binary(op, apply(dl.view(), ls), apply(dr.view(), rs), apply(do.view(), os_))
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    assert kernel_name().startswith("rows_") == on_rows(dtype)
    assert iomo.binary(op, apply(hl.view(), ls), apply(hr.view(), rs), apply(ho.view(), os_),
                       ieee=True) == 0
    assert same_storage(do, ho)
    for t in (dl, dr, do):
        t.free()


@pytest.mark.parametrize("dtype", [d for d in ROWS_NUMERIC if d in FLOAT_LEAVES],
                         ids=names([d for d in ROWS_NUMERIC if d in FLOAT_LEAVES]))
@pytest.mark.parametrize("case", range(len(ROWS_CASES)))
def test_division_views_and_broadcasts(dtype, case):
    ld, ls, rd, rs, od, os_ = ROWS_CASES[case]
    dl, hl = pair(dtype, ld, salt=0x400 + case)
    dr, hr = pair(dtype, rd, salt=0x500 + case)
    do, ho = pair(dtype, od, salt=0x600 + case)
    rc = iomx.binary(OP_DIV, apply(dl.view(), ls), apply(dr.view(), rs), apply(do.view(), os_))
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    assert kernel_name().startswith("rows_") == on_rows(dtype)
    assert iomo.binary(OP_DIV, apply(hl.view(), ls), apply(hr.view(), rs), apply(ho.view(), os_),
                       ieee=True) == 0
    assert same_storage(do, ho)
    for t in (dl, dr, do):
        t.free()


def half_specials():
    return np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x83FF, 0x8400, 0x3C00, 0xBC00,
                     0x3C01, 0x3BFF, 0x7BFF, 0xFBFF, 0x7C00, 0xFC00, 0x7C01, 0x7E00, 0xFE00, 0xFFFF,
                     0x0002, 0x1400, 0x13FF, 0x6800, 0x7800, 0x3555, 0x4248], np.uint16)


@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
def test_binary_f16_four_million_pairs_against_the_codec(op):
    n = 2048
    vals = np.concatenate([half_specials(), datagen.pattern_bits(16, n - half_specials().size, 41)])
    other = np.concatenate([datagen.pattern_bits(16, n - half_specials().size, 42), half_specials()])
    dl, hl = pair(DT_F16, (n, 1), values=vals.reshape(n, 1))
    dr, hr = pair(DT_F16, (1, n), values=other.reshape(1, n))
    do, ho = pair(DT_F16, (n, n))
    assert iomx.binary(op, dl.view(), dr.view(), do.view()) == 0
    assert iomo.binary(op, hl.view(), hr.view(), ho.view(), ieee=True) == 0
    assert same_storage(do, ho)
    # a band of it against the long-double codec
    got = do.view().to_host()[:64]
    L = iomo.lib()
    for i in range(64):
        for j in range(0, n, 3):
            assert L.iomo_scalar_binary(op, DT_F16, int(vals[i]), int(other[j])) == int(got[i, j])
    for t in (dl, dr, do):
        t.free()


def double_specials():
    return np.array([0, 1 << 63, 1, (1 << 63) | 1, 0x000FFFFFFFFFFFFF, 0x0010000000000000,
                     0x3FF0000000000000, 0xBFF0000000000000, 0x3FF0000000000001, 0x7FEFFFFFFFFFFFFF,
                     0xFFEFFFFFFFFFFFFF, 0x7FF0000000000000, 0xFFF0000000000000, 0x7FF0000000000001,
                     0x7FF8000000000000, 0xFFFFFFFFFFFFFFFF, 0x3CA0000000000000, 0x3CA0000000000001,
                     0x4340000000000000, 0x3FD5555555555555], np.uint64)


@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
def test_binary_f64_specials_and_random_pairs(op):
    n = 1024
    k = n - double_specials().size
    vals = np.concatenate([double_specials(), datagen.pattern_bits(64, k, 71)])
    other = np.concatenate([datagen.pattern_bits(64, k, 74), double_specials()])
    dl, hl = pair(DT_F64, (n, 1), values=vals.reshape(n, 1))
    dr, hr = pair(DT_F64, (1, n), values=other.reshape(1, n))
    do, ho = pair(DT_F64, (n, n))
    assert iomx.binary(op, dl.view(), dr.view(), do.view()) == 0
    assert iomo.binary(op, hl.view(), hr.view(), ho.view(), ieee=True) == 0
    assert same_storage(do, ho)
    for t in (dl, dr, do):
        t.free()


def test_non_numeric_leaves_and_exact_alias():
    for dtype in (DT_BOOL, DT_F8_E8M0):
        d, _ = pair(dtype, (16, 16), salt=1)
        o, _ = pair(dtype, (16, 16))
        assert iomx.binary(OP_ADD, d.view(), d.view(), o.view()) == -2
        d.free()
        o.free()
    # in-place on an exact alias, packed leaf with padding
    da, ha = pair(DT_U4, (2, 17, 33), salt=5)
    db, hb = pair(DT_U4, (2, 17, 33), salt=6)
    assert iomx.binary(OP_MUL, da.view(), db.view(), da.view()) == 0
    assert iomo.binary(OP_MUL, ha.view(), hb.view(), ha.view()) == 0
    assert same_storage(da, ha)
    # a shifted window of the same owner is refused
    dc, _ = pair(DT_U4, (3, 17, 33), salt=7)
    assert iomx.binary(OP_ADD, dc.view().slice(0, 0, 2), db.view(), dc.view().slice(0, 1, 2)) == -1
    for t in (da, db, dc):
        t.free()


# -- SiLU / RMSNorm ----------------------------------------------------------------------

def ordered(raw, bits):
    raw = raw.astype(np.int64)
    sign = 1 << (bits - 1)
    return np.where(raw & sign, sign - 1 - (raw & (sign - 1)), raw | sign) if bits < 64 else None


def steps_apart(a, b, dtype):
    """Distance in encoding steps along the real line (sign-magnitude order)."""
    bits = LEAF_BITS[dtype]
    if bits == 64:
        a, b = a.astype(np.uint64), b.astype(np.uint64)
        key = lambda v: np.where(v >> np.uint64(63), ~v, v | np.uint64(1 << 63))
        ka, kb = key(a), key(b)
        return np.where(ka > kb, ka - kb, kb - ka)
    return np.abs(ordered(a, bits) - ordered(b, bits))


def is_nan(raw, dtype):
    ebits, fbits = {13: (2, 1), 14: (2, 3), 15: (3, 2), 16: (4, 3), 17: (5, 2), 19: (5, 10), 22: (11, 52)}[dtype]
    if dtype in (13, 14, 15):
        return np.zeros(raw.shape, bool)
    raw = raw.astype(np.uint64)
    top = np.uint64((1 << ebits) - 1)
    exp = (raw >> np.uint64(fbits)) & top
    frac = raw & np.uint64((1 << fbits) - 1)
    return (exp == top) if dtype == 16 else ((exp == top) & (frac != 0))


@pytest.mark.parametrize("dtype", ROWS_FLOAT, ids=names(ROWS_FLOAT))
def test_silu_every_encoding(dtype):
    bits = LEAF_BITS[dtype]
    if bits <= 16:
        n = 1 << bits
        vals = np.arange(n, dtype=np.uint32).astype(iomo.NP_OF[dtype])
        dims = (max(n // 64, 1), min(n, 64))
    else:
        dims = (300, 333)
        k = 300 * 333
        vals = np.concatenate([double_specials(), datagen.pattern_bits(64, k - 20 - 3000, 91),
                               # moderate magnitudes, where the sigmoid is neither 0 nor 1
                               (datagen.uniform01(3000, 92) * 40 - 20).view(np.uint64)])
    dx, hx = pair(dtype, dims, values=vals.reshape(dims))
    do, ho = pair(dtype, dims)
    assert iomx.silu(dx.view(), do.view()) == 0
    assert kernel_name().startswith("rows_") == on_rows(dtype)
    assert iomo.silu(hx.view(), ho.view()) == 0
    got, want = do.view().to_host().reshape(-1), ho.view().to_logical().reshape(-1)
    nan = is_nan(want, dtype)
    assert np.array_equal(got[nan], want[nan])                     # canonical NaN, exactly
    d = steps_apart(got[~nan], want[~nan], dtype)
    assert d.max() <= (1 if bits <= 16 else 4)
    print(LEAF_NAME[dtype], "silu: %d of %d encodings one step from the CPU arithmetic" % (int((d > 0).sum()), d.size), flush=True)
    if int((d > 0).sum()) == 0:
        assert same_storage(do, ho)                                # poisoned padding untouched
    dx.free()
    do.free()


def finite_values(dtype, count, salt):
    bits = LEAF_BITS[dtype]
    v = datagen.pattern_bits(bits, count, salt)
    ebits, fbits = {13: (2, 1), 14: (2, 3), 15: (3, 2), 16: (4, 3), 17: (5, 2), 19: (5, 10), 22: (11, 52)}[dtype]
    if dtype in (13, 14, 15):
        return v
    top = (1 << ebits) - 1
    exp = (v.astype(np.uint64) >> np.uint64(fbits)) & np.uint64(top)
    if dtype == 22:
        exp = exp % np.uint64(17) + np.uint64(1023 - 8)
    else:
        exp = np.where(exp == top, np.uint64(top - 1), exp)
    cleared = v.astype(np.uint64) & ~np.uint64(top << fbits)
    return (cleared | (exp << np.uint64(fbits))).astype(v.dtype)


@pytest.mark.parametrize("dtype", ROWS_FLOAT, ids=names(ROWS_FLOAT))
@pytest.mark.parametrize("dims,steps", [((2, 5, 40), []), ((3, 17, 33), []), ((4, 16, 4112), [("slice", (0, 0, 2, 2))]),
                                        ((1, 1), []), ((40, 2048), []), ((2, 33, 256), [])])
def test_rmsnorm_float_leaves(dtype, dims, steps):
    F = dims[-1]
    dx, hx = pair(dtype, dims, values=finite_values(dtype, int(np.prod(dims)), 81).reshape(dims))
    dw, hw = pair(dtype, (1, F), values=finite_values(dtype, F, 82).reshape(1, F))
    do, ho = pair(dtype, dims, salt=83)
    rc = iomx.rmsnorm(apply(dx.view(), steps), dw.view(), apply(do.view(), steps), 1e-5)
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    # F16 always, and the two 8-bit leaves where a band is whole tiles, take the resident kernel
    resident = dtype == DT_F16 or (dtype in F8_CONVERTED and F % 16 == 0)
    assert (kernel_name() == "rows_rmsnorm") == (not resident)
    assert iomo.rmsnorm(apply(hx.view(), steps), hw.view(), apply(ho.view(), steps), 1e-5) == 0
    got, want = do.view().to_host().reshape(-1), ho.view().to_logical().reshape(-1)
    nan = is_nan(want, dtype)
    assert np.array_equal(got[nan], want[nan])
    d = steps_apart(got[~nan], want[~nan], dtype)
    if dtype == DT_F64:
        a, b = got[~nan].view(np.float64), want[~nan].view(np.float64)
        assert (np.abs(a - b) <= 1e-12 * np.abs(b)).all()
    else:
        assert d.max() <= 1
    dx.free(); dw.free(); do.free()


@pytest.mark.parametrize("dtype", [d for d in ROWS_FLOAT if LEAF_BITS[d] <= 16],
                         ids=names([d for d in ROWS_FLOAT if LEAF_BITS[d] <= 16]))
def test_rmsnorm_rows_with_specials(dtype):
    n = min(1 << LEAF_BITS[dtype], 4096)
    vals = (np.arange(n) * (1 if n < 4096 else 16)).astype(iomo.NP_OF[dtype])
    F = 16
    dims = (n // F, F)
    dx, hx = pair(dtype, dims, values=vals.reshape(dims))
    dw, hw = pair(dtype, (1, F), values=finite_values(dtype, F, 84).reshape(1, F))
    do, ho = pair(dtype, dims)
    assert iomx.rmsnorm(dx.view(), dw.view(), do.view(), 0.0) == 0
    assert iomo.rmsnorm(hx.view(), hw.view(), ho.view(), 0.0) == 0
    got, want = do.view().to_host().reshape(-1), ho.view().to_logical().reshape(-1)
    nan = is_nan(want, dtype)
    assert np.array_equal(got[nan], want[nan])
    assert steps_apart(got[~nan], want[~nan], dtype).max() <= 1
    dx.free(); dw.free(); do.free()
