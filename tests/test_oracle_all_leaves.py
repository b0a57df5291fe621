"""Every leaf the standard tiled backends advertise (23; src/shared/
standard_tiled_copy.hpp:17-31), against the reference CPU backend compiled into
oracle/_ref: storage and host transfer of packed 2/4/6-bit leaves, copy, the
binary operations over the 21 numeric leaves (exhaustively for every leaf of at
most 8 bits), RMSNorm and SiLU over the 9 floating leaves.
"""
import numpy as np
import pytest

import datagen
import iomo
from iomo import (ALL_LEAVES, DT_F16, DT_F64, DT_I16, DT_I64, DT_U16, DT_U64, FLOAT_LEAVES,
                  LEAF_BITS, LEAF_NAME, NUMERIC_LEAVES, OP_ADD, OP_DIV, OP_MUL, OP_SUB)

NARROW = [d for d in NUMERIC_LEAVES if LEAF_BITS[d] <= 8]
names = lambda ds: [LEAF_NAME[d] for d in ds]


def pattern(dtype, count, salt):
    v = datagen.pattern_bits(LEAF_BITS[dtype], count, salt)
    # BOOL host bytes must be zero or one (src/tensor_view.cpp:265-270)
    return v & 1 if dtype == iomo.DT_BOOL else v


def both(ref, dtype, dims, salt=None, values=None):
    rt = ref.tensor(dtype, dims)
    ht = iomo.HostTensor(dtype, dims)
    if salt is not None:
        values = pattern(dtype, int(np.prod(dims)), salt).reshape(dims)
    if values is not None:
        rt.view().from_host(values)
        ht.view().from_logical(values)
    return rt, ht


def same_storage(rt, ht):
    return np.array_equal(rt.view().raw_storage(), ht.storage.view(np.uint8))


# -- packing helpers of the test harness itself --------------------------------

@pytest.mark.parametrize("bits", [2, 4, 6])
def test_pack_bits_is_the_little_endian_bit_stream(bits):
    v = datagen.pattern_bits(bits, 37, 5)
    stream = iomo.pack_bits(v, bits)
    assert stream.size == (37 * bits + 7) // 8
    for i, e in enumerate(v):                       # bit by bit, as transfer_helpers.hpp:14-25
        got = 0
        for k in range(bits):
            bit = i * bits + k
            got |= ((int(stream[bit // 8]) >> (bit % 8)) & 1) << k
        assert got == int(e)
    assert np.array_equal(iomo.unpack_bits(stream, bits, 37), v)


# -- storage / transfer / copy ---------------------------------------------------

@pytest.mark.parametrize("dtype", ALL_LEAVES, ids=names(ALL_LEAVES))
@pytest.mark.parametrize("dims", [(17, 33), (3, 5, 7), (2, 16, 32), (1, 1), (2, 3, 1, 50)])
def test_transfer_and_storage_bytes(ref, dtype, dims):
    rt, ht = both(ref, dtype, dims, salt=11)
    assert same_storage(rt, ht)
    want = pattern(dtype, int(np.prod(dims)), 11).reshape(dims)
    assert np.array_equal(rt.view().to_host(), want)
    assert np.array_equal(ht.view().to_logical(), want)
    # the packed stream itself, including the zeroed tail bits of a last partial byte
    stream = rt.view().to_host_stream()
    assert np.array_equal(stream, iomo.pack_bits(want, LEAF_BITS[dtype]))


@pytest.mark.parametrize("dtype", ALL_LEAVES, ids=names(ALL_LEAVES))
def test_transfer_into_views_leaves_the_rest(ref, dtype):
    rt, ht = both(ref, dtype, (4, 3, 17, 19), salt=21)
    part = pattern(dtype, 2 * 3 * 17 * 19, 22).reshape(2, 3, 17, 19)
    rt.view().slice(0, 1, 2, 2).from_host(part)
    ht.view().slice(0, 1, 2, 2).from_logical(part)
    assert same_storage(rt, ht)
    assert np.array_equal(rt.view().permute([1, 0]).to_host(), ht.view().permute([1, 0]).to_logical())
    assert np.array_equal(rt.view().select(1, 2).to_host(), ht.view().select(1, 2).to_logical())


@pytest.mark.parametrize("dtype", ALL_LEAVES, ids=names(ALL_LEAVES))
def test_copy_between_views(ref, dtype):
    rs, hs = both(ref, dtype, (4, 3, 17, 19), salt=31)
    rd, hd = both(ref, dtype, (3, 6, 17, 19), salt=32)
    tok = ref.copy(rs.view().slice(0, 0, 2, 2).permute([1, 0]), rd.view().slice(1, 1, 2, 3))
    assert tok > 0, ref.error()
    assert iomo.copy(hs.view().slice(0, 0, 2, 2).permute([1, 0]), hd.view().slice(1, 1, 2, 3)) == 0
    assert same_storage(rd, hd)


# -- binary operations -----------------------------------------------------------

@pytest.mark.parametrize("dtype", NARROW, ids=names(NARROW))
@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
def test_binary_every_pair_of_a_narrow_leaf(ref, dtype, op):
    """[n,1] x [1,n] -> [n,n] holds every operand pair of the leaf."""
    if op == OP_DIV and dtype not in iomo.FLOAT_LEAVES:
        pytest.skip("division is defined on the floating leaves only")
    n = 1 << LEAF_BITS[dtype]
    every = np.arange(n, dtype=np.uint8 if n <= 256 else np.uint16)
    rl, hl = both(ref, dtype, (n, 1), values=every.reshape(n, 1))
    rr, hr = both(ref, dtype, (1, n), values=every.reshape(1, n))
    ro, ho = both(ref, dtype, (n, n))
    assert ref.binary(op, rl.view(), rr.view(), ro.view()) > 0, ref.error()
    want = ro.view().to_host()
    for ieee in (False, True):
        assert iomo.binary(op, hl.view(), hr.view(), ho.view(), ieee) == 0
        assert np.array_equal(ho.view().to_logical(), want), "ieee" if ieee else "codec"
        assert same_storage(ro, ho)


def half_specials():
    return np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x83FF, 0x8400, 0x3C00, 0xBC00,
                     0x3C01, 0x3BFF, 0x7BFF, 0xFBFF, 0x7C00, 0xFC00, 0x7C01, 0x7E00, 0xFE00, 0xFFFF,
                     0x0002, 0x1400, 0x13FF, 0x6800, 0x7800, 0x3555, 0x4248], np.uint16)


@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
def test_binary_f16_specials_and_random_pairs(ref, op):
    n = 1200
    vals = np.concatenate([half_specials(), datagen.pattern_bits(16, n - half_specials().size, 41)])
    other = np.concatenate([datagen.pattern_bits(16, n - half_specials().size, 42), half_specials()])
    rl, hl = both(ref, DT_F16, (n, 1), values=vals.reshape(n, 1))
    rr, hr = both(ref, DT_F16, (1, n), values=other.reshape(1, n))
    ro, ho = both(ref, DT_F16, (n, n))
    assert ref.binary(op, rl.view(), rr.view(), ro.view()) > 0
    want = ro.view().to_host()
    for ieee in (False, True):
        assert iomo.binary(op, hl.view(), hr.view(), ho.view(), ieee) == 0
        assert np.array_equal(ho.view().to_logical(), want)


def test_f16_closed_form_against_numpy_half():
    """numpy's float16 arithmetic is IEEE binary16 (computed in binary32 and rounded
    once more, innocuous for one operation): an implementation outside this repository."""
    L = iomo.lib()
    a = np.concatenate([half_specials(), datagen.pattern_bits(16, 4000, 51)])
    b = np.concatenate([half_specials()[::-1], datagen.pattern_bits(16, 4000, 52)])
    with np.errstate(all="ignore"):
        for op, fn in ((OP_ADD, np.add), (OP_MUL, np.multiply), (OP_SUB, np.subtract),
                       (OP_DIV, np.divide)):
            r = fn(a.view(np.float16), b.view(np.float16)).view(np.uint16)
            for x, y, z in zip(a.tolist(), b.tolist(), r.tolist()):
                got = L.iomo_scalar_binary_ieee(op, DT_F16, x, y)
                if (z & 0x7FFF) > 0x7C00:
                    assert got == 0x7E00
                elif op == OP_ADD and (z & 0x7FFF) == 0 and not ((x & y) >> 15):
                    assert got == 0          # exact zero sums are +0 unless both operands are -0
                else:
                    assert got == z, (op, hex(x), hex(y))


@pytest.mark.parametrize("dtype", [DT_I16, DT_U16, DT_I64, DT_U64], ids=names([DT_I16, DT_U16, DT_I64, DT_U64]))
@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB])
def test_binary_wide_integers(ref, dtype, op):
    dims = (3, 17, 21)
    rl, hl = both(ref, dtype, dims, salt=61)
    rr, hr = both(ref, dtype, (1, 21), salt=62)
    ro, ho = both(ref, dtype, dims)
    assert ref.binary(op, rl.view(), rr.view(), ro.view()) > 0
    want = ro.view().to_host()
    for ieee in (False, True):
        assert iomo.binary(op, hl.view(), hr.view(), ho.view(), ieee) == 0
        assert np.array_equal(ho.view().to_logical(), want)
    # two's-complement wrap, stated with numpy
    a, b = hl.view().to_logical(), hr.view().to_logical()
    with np.errstate(over="ignore"):
        closed = {OP_ADD: a + b, OP_MUL: a * b, OP_SUB: a - b}[op]
    assert np.array_equal(closed, want)


def double_specials():
    return np.array([0, 1 << 63, 1, (1 << 63) | 1, 0x000FFFFFFFFFFFFF, 0x0010000000000000,
                     0x3FF0000000000000, 0xBFF0000000000000, 0x3FF0000000000001, 0x7FEFFFFFFFFFFFFF,
                     0xFFEFFFFFFFFFFFFF, 0x7FF0000000000000, 0xFFF0000000000000, 0x7FF0000000000001,
                     0x7FF8000000000000, 0xFFFFFFFFFFFFFFFF, 0x3CA0000000000000, 0x3CA0000000000001,
                     0x4340000000000000, 0x3FD5555555555555], np.uint64)


def finite_doubles(n, salt):
    """Random binary64 values with exponents within 2^-40 .. 2^40, so sums and
    products are ordinary rounded results."""
    frac = datagen.pattern_bits(64, n, salt) & np.uint64((1 << 52) - 1)
    exp = (datagen.pattern_bits(32, n, salt + 1) % 81 + (1023 - 40)).astype(np.uint64)
    sign = (datagen.pattern_bits(8, n, salt + 2) & 1).astype(np.uint64)
    return (sign << np.uint64(63)) | (exp << np.uint64(52)) | frac


@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
def test_binary_f64_codec_and_binary64_carrier(ref, op):
    n = 600
    vals = np.concatenate([double_specials(), finite_doubles(n - double_specials().size, 71)])
    other = np.concatenate([finite_doubles(n - double_specials().size, 74), double_specials()])
    rl, hl = both(ref, DT_F64, (n, 1), values=vals.reshape(n, 1))
    rr, hr = both(ref, DT_F64, (1, n), values=other.reshape(1, n))
    ro, ho = both(ref, DT_F64, (n, n))
    assert ref.binary(op, rl.view(), rr.view(), ro.view()) > 0
    want = ro.view().to_host()
    assert iomo.binary(op, hl.view(), hr.view(), ho.view(), False) == 0
    assert np.array_equal(ho.view().to_logical(), want)            # the codec, bit for bit
    # binary64 carrier (what a device without an extended type computes): equal except
    # where the 64-bit-significand carrier of the host codec rounds twice: one unit apart
    assert iomo.binary(op, hl.view(), hr.view(), ho.view(), True) == 0
    carrier = ho.view().to_logical()
    differs = carrier != want
    gap = np.abs(carrier[differs].astype(np.int64) - want[differs].astype(np.int64))
    assert differs.mean() < 2e-3 and (gap.size == 0 or gap.max() == 1)
    # and binary64 itself, stated with numpy
    with np.errstate(all="ignore"):
        a, b = vals.view(np.float64).reshape(n, 1), other.view(np.float64).reshape(1, n)
        closed = {OP_ADD: a + b, OP_MUL: a * b, OP_SUB: a - b, OP_DIV: a / b}[op]
    bits = closed.view(np.uint64).copy()
    bits[np.isnan(closed)] = 0x7FF8000000000000
    if op == OP_ADD:     # exact-zero sums are +0 unless both operands are -0
        both_negative_zero = (vals.reshape(n, 1) == 1 << 63) & (other.reshape(1, n) == 1 << 63)
        bits[(closed == 0) & ~both_negative_zero] = 0
    assert np.array_equal(bits, carrier)


# -- RMSNorm / SiLU over the floating leaves ---------------------------------------

def finite_values(dtype, count, salt):
    """Raw encodings without NaN / infinity patterns (top exponent cleared where it is special)."""
    bits = LEAF_BITS[dtype]
    v = datagen.pattern_bits(bits, count, salt)
    ebits, fbits = {13: (2, 1), 14: (2, 3), 15: (3, 2), 16: (4, 3), 17: (5, 2), 19: (5, 10),
                    20: (8, 7), 21: (8, 23), 22: (11, 52)}[dtype]
    if dtype in (13, 14, 15):
        return v
    top = (1 << ebits) - 1
    exp = (v.astype(np.uint64) >> np.uint64(fbits)) & np.uint64(top)
    if dtype in (20, 21, 22):
        # keep magnitudes moderate so squares stay finite: exponent within bias +- 8
        bias = (1 << (ebits - 1)) - 1
        exp = exp % np.uint64(17) + np.uint64(bias - 8)
    else:
        exp = np.where(exp == top, np.uint64(top - 1), exp)
    cleared = v.astype(np.uint64) & ~np.uint64(top << fbits)
    return (cleared | (exp << np.uint64(fbits))).astype(v.dtype)


@pytest.mark.parametrize("dtype", FLOAT_LEAVES, ids=names(FLOAT_LEAVES))
def test_rmsnorm_every_float_leaf_bit_exact(ref, dtype):
    dims, F = (2, 5, 40), 40
    rx, hx = both(ref, dtype, dims, values=finite_values(dtype, 400, 81).reshape(dims))
    rw, hw = both(ref, dtype, (1, F), values=finite_values(dtype, F, 82).reshape(1, F))
    ro, ho = both(ref, dtype, dims, salt=83)
    assert ref.rmsnorm(rx.view(), rw.view(), ro.view(), 1e-5) > 0, ref.error()
    assert iomo.rmsnorm(hx.view(), hw.view(), ho.view(), 1e-5) == 0
    assert same_storage(ro, ho)


@pytest.mark.parametrize("dtype", [d for d in FLOAT_LEAVES if LEAF_BITS[d] <= 16],
                         ids=names([d for d in FLOAT_LEAVES if LEAF_BITS[d] <= 16]))
def test_rmsnorm_rows_with_specials(ref, dtype):
    """Every encoding of the leaf appears in some row, NaN and infinities included."""
    n = min(1 << LEAF_BITS[dtype], 4096)
    vals = (np.arange(n) * (1 if n < 4096 else 16)).astype(iomo.NP_OF[dtype])
    F = 16
    dims = (n // F, F)
    rx, hx = both(ref, dtype, dims, values=vals.reshape(dims))
    rw, hw = both(ref, dtype, (1, F), values=finite_values(dtype, F, 84).reshape(1, F))
    ro, ho = both(ref, dtype, dims)
    assert ref.rmsnorm(rx.view(), rw.view(), ro.view(), 0.0) > 0
    assert iomo.rmsnorm(hx.view(), hw.view(), ho.view(), 0.0) == 0
    assert same_storage(ro, ho)


@pytest.mark.parametrize("dtype", FLOAT_LEAVES, ids=names(FLOAT_LEAVES))
def test_silu_every_float_leaf_bit_exact(ref, dtype):
    bits = LEAF_BITS[dtype]
    if bits <= 16:
        n = 1 << bits                                    # every encoding
        vals = np.arange(n, dtype=np.uint32).astype(iomo.NP_OF[dtype])
        dims = (max(n // 64, 1), min(n, 64))
    else:
        dims = (50, 41)
        vals = datagen.pattern_bits(bits, 50 * 41, 91)
    rx, hx = both(ref, dtype, dims, values=vals.reshape(dims))
    ro, ho = both(ref, dtype, dims)
    assert ref.silu(rx.view(), ro.view()) > 0, ref.error()
    assert iomo.silu(hx.view(), ho.view()) == 0
    assert same_storage(ro, ho)


def test_non_numeric_leaves_are_refused(ref):
    for dtype in (iomo.DT_BOOL, iomo.DT_F8_E8M0):
        rl, hl = both(ref, dtype, (16, 16), salt=1)
        ro, ho = both(ref, dtype, (16, 16))
        assert ref.binary(OP_ADD, rl.view(), rl.view(), ro.view()) == -2
        assert iomo.binary(OP_ADD, hl.view(), hl.view(), ho.view()) == -2
