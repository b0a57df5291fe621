"""Pins the CPU oracle against the reference's own known answers and against
what the mathematics fixes.  No GPU, no reference binary needed.

Sources of the vectors (paths in the rlewczuk/iom tree):
  layout      test/test_iom.cpp:614-658
  binary      test/backend/test_scalar_add.cpp:40-94
  SiLU        test/backend/test_scalar_silu.cpp:138-167,313-327,
              docs/BACKEND_CONTRACT/silu-activation.md:156-158
  softmax     test/rocm/test_rocm_sdpa_nonmatrix.cpp:607-648
  RMSNorm     test/backend/backend_conformance_rmsnorm_reference.hpp:1347-1367
"""
import math

import numpy as np
import pytest

import datagen
import iomo
from iomo import DT_BF16, DT_F32, DT_I32, DT_U32, OP_ADD, OP_DIV, OP_MUL, OP_SUB

L = iomo.lib()


def plane_of(lead_dims, coord):
    p = 0
    for d, c in zip(lead_dims, coord):
        p = p * d + c
    return p


# ---------------------------------------------------------------- layout ----

@pytest.mark.parametrize("dims,coord,slot", [
    ((32, 32), (0, 0), 0), ((32, 32), (0, 16), 256), ((32, 32), (16, 0), 512),
    ((32, 32), (16, 16), 768), ((32, 32), (0, 15), 15),
    ((32, 32), (15, 31), 256 + 15 * 16 + 15), ((32, 32), (31, 31), 3 * 256 + 15 * 16 + 15),
    ((2, 3, 16, 16), (0, 0, 15, 15), 255), ((2, 3, 16, 16), (0, 1, 0, 0), 256),
    ((2, 3, 16, 16), (1, 0, 0, 0), 3 * 256), ((2, 3, 16, 16), (1, 2, 15, 15), 5 * 256 + 255),
    ((2, 2, 2, 16, 16), (1, 1, 1, 0, 0), 7 * 256), ((2, 2, 2, 16, 16), (0, 0, 1, 15, 15), 256 + 255),
    ((2, 3, 4, 17, 33), (1, 2, 3, 16, 32), 143 * 256),
    ((20, 35), (0, 34), 2 * 256 + 2), ((20, 35), (15, 34), 2 * 256 + 15 * 16 + 2),
    ((20, 35), (16, 0), 3 * 256),
    ((2, 8, 31, 33), (0, 1, 0, 0), 6 * 256), ((2, 8, 31, 33), (1, 0, 30, 32), 53 * 256 + 14 * 16),
])
def test_plane_slot_known_answers(dims, coord, slot):
    plane = plane_of(dims[:-2], coord[:-2])
    assert L.iomo_plane_slot(dims[-2], dims[-1], plane, coord[-2], coord[-1]) == slot


@pytest.mark.parametrize("dims", [(20, 35), (2, 3, 17, 33), (3, 16, 48), (1, 1)])
@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32])
def test_scatter_matches_closed_form_tiling_and_every_slot_is_unique(dims, dtype):
    n = int(np.prod(dims))
    bits = 16 if dtype == DT_BF16 else 32
    logical = datagen.pattern_bits(bits, n, 0xABC).reshape(dims)
    t = iomo.HostTensor(dtype, dims, fill=0x5A)
    t.view().from_logical(logical)
    fill = np.frombuffer(bytes([0x5A] * (bits // 8)), dtype=iomo.NP_OF[dtype])[0]
    assert np.array_equal(t.storage, iomo.tile_plane(logical, fill=fill))
    assert np.array_equal(t.view().to_logical(), logical)
    assert np.array_equal(iomo.untile_plane(t.storage, dims), logical)
    planes = n // (dims[-1] * dims[-2])
    seen = set()
    for p in range(planes):
        for r in range(dims[-2]):
            for c in range(dims[-1]):
                seen.add(L.iomo_plane_slot(dims[-2], dims[-1], p, r, c))
    assert len(seen) == n and max(seen) < t.storage.size


# ---------------------------------------------------------------- binary ----

KATS = [
    (OP_MUL, DT_I32, 0x80000000, 3, 0x80000000),
    (OP_SUB, DT_U32, 0, 1, 0xFFFFFFFF),
    (OP_ADD, DT_I32, 0xFFFFFFFF, 1, 0),
    (OP_MUL, DT_F32, 0x7F800000, 0, 0x7FC00000),
    (OP_SUB, DT_F32, 0x7F800000, 0x7F800000, 0x7FC00000),
    (OP_ADD, DT_F32, 0x3F800000, 0x3F800000, 0x40000000),
    (OP_ADD, DT_F32, 0x80000000, 0, 0),
    (OP_ADD, DT_F32, 0x80000000, 0x80000000, 0x80000000),
    (OP_ADD, DT_F32, 0x7F800000, 0xFF800000, 0x7FC00000),
    (OP_ADD, DT_BF16, 0x7F80, 0xFF80, 0x7FC0),
    # overflow cases of test_scalar_add.cpp:63-94
    (OP_ADD, DT_BF16, 0x7F7F, 0x7F7F, 0x7F80), (OP_MUL, DT_BF16, 0x7F7F, 0x4000, 0x7F80),
    (OP_SUB, DT_BF16, 0x7F7F, 0xFF7F, 0x7F80), (OP_ADD, DT_BF16, 0xFF7F, 0xFF7F, 0xFF80),
    (OP_MUL, DT_BF16, 0xFF7F, 0x4000, 0xFF80), (OP_SUB, DT_BF16, 0xFF7F, 0x7F7F, 0xFF80),
    (OP_ADD, DT_F32, 0x7F7FFFFF, 0x7F7FFFFF, 0x7F800000),
    (OP_MUL, DT_F32, 0x7F7FFFFF, 0x40000000, 0x7F800000),
    (OP_SUB, DT_F32, 0x7F7FFFFF, 0xFF7FFFFF, 0x7F800000),
    (OP_ADD, DT_F32, 0xFF7FFFFF, 0xFF7FFFFF, 0xFF800000),
    (OP_MUL, DT_F32, 0xFF7FFFFF, 0x40000000, 0xFF800000),
    (OP_SUB, DT_F32, 0xFF7FFFFF, 0x7F7FFFFF, 0xFF800000),
    # division: test_scalar_add.cpp:50-53 and the overflow cases of :94,:101
    (OP_DIV, DT_F32, 0, 0, 0x7FC00000), (OP_DIV, DT_F32, 0x80000000, 1, 0x80000000),
    (OP_DIV, DT_F32, 0x80000000, 0x80000000, 0x7FC00000),
    (OP_DIV, DT_F32, 0x3F800000, 0x7F800000, 0),
    (OP_DIV, DT_BF16, 0x7F7F, 0x3F00, 0x7F80), (OP_DIV, DT_BF16, 0xFF7F, 0x3F00, 0xFF80),
    (OP_DIV, DT_F32, 0x7F7FFFFF, 0x3F000000, 0x7F800000),
    (OP_DIV, DT_F32, 0xFF7FFFFF, 0x3F000000, 0xFF800000),
    # what IEEE 754 fixes: x/0 is a signed infinity, inf/inf is NaN, 1/3 rounds to nearest
    (OP_DIV, DT_F32, 0x3F800000, 0x80000000, 0xFF800000),
    (OP_DIV, DT_F32, 0x7F800000, 0xFF800000, 0x7FC00000),
    (OP_DIV, DT_F32, 0x3F800000, 0x40400000, 0x3EAAAAAB),
    (OP_DIV, DT_BF16, 0x3F80, 0x4040, 0x3EAB), (OP_DIV, DT_BF16, 0x4000, 0x4040, 0x3F2B),
    # NaN payloads and signs collapse to the positive canonical quiet NaN
    (OP_ADD, DT_F32, 0xFFC12345, 0x3F800000, 0x7FC00000),
    (OP_MUL, DT_BF16, 0xFFFF, 0x3F80, 0x7FC0),
]


@pytest.mark.parametrize("op,dtype,a,b,expect", KATS)
def test_scalar_binary_known_answers(op, dtype, a, b, expect):
    assert L.iomo_scalar_binary(op, dtype, a, b) == expect
    assert L.iomo_scalar_binary_ieee(op, dtype, a, b) == expect


def test_bf16_mul_through_f32_is_single_rounded_even_for_subnormal_products():
    # A BF16 product has at most 16 significant bits.  When it is an F32 subnormal its
    # lowest bit sits at 2^(e-15) with e >= -135 whenever the value can reach half of the
    # smallest BF16 subnormal (2^-134), i.e. on the 2^-149 grid or above: the F32 product
    # is then exact and BF16-RNE of it is the one rounding the codec performs.  Below that
    # both round to zero.  Checked here over the whole band, through numpy's binary32.
    sigs = np.arange(0, 128, dtype=np.uint16)
    for ea in range(40, 128, 7):
        for eb in range(1, 128):
            e = (ea - 127) + (eb - 127)
            if not -152 <= e <= -120:
                continue
            a = ((ea << 7) | sigs)[:, None].repeat(128, 1).reshape(-1)
            b = ((eb << 7) | sigs)[None, :].repeat(128, 0).reshape(-1)
            with np.errstate(all="ignore"):
                prod = datagen.bf16_to_f32(a) * datagen.bf16_to_f32(b)
            via_f32 = datagen.bf16_rne(prod)
            idx = np.arange(0, a.size, 13)
            want = np.array([L.iomo_scalar_binary(OP_MUL, DT_BF16, int(a[i]), int(b[i]))
                             for i in idx], np.uint16)
            assert np.array_equal(via_f32[idx], want), (ea, eb)


def _check_codec_equals_closed_form(op, dtype, a, b):
    for x, y in zip(a.tolist(), b.tolist()):
        assert L.iomo_scalar_binary(op, dtype, x, y) == \
            L.iomo_scalar_binary_ieee(op, dtype, x, y), (op, dtype, hex(x), hex(y))


@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
@pytest.mark.parametrize("dtype", [DT_I32, DT_F32, DT_BF16])
def test_codec_equals_ieee_closed_form_on_hash_patterns(op, dtype):
    if op == OP_DIV and dtype == DT_I32:
        pytest.skip("division is defined on the floating leaves only")
    bits = 16 if dtype == DT_BF16 else 32
    n = 20000
    a = datagen.pattern_bits(bits, n, 0x1234 + op)
    b = datagen.pattern_bits(bits, n, 0x9876 + dtype)
    _check_codec_equals_closed_form(op, dtype, a, b)
    # near-cancelling and same-exponent operands (hash patterns rarely produce them)
    b2 = a ^ (datagen.pattern_bits(bits, n, 77) & 0x7) ^ (1 << (bits - 1))
    _check_codec_equals_closed_form(op, dtype, a, b2.astype(a.dtype))


def test_bf16_mul_closed_form_over_the_subnormal_product_band():
    # every pair of exponents whose product lands in [2^-140, 2^-120) with a spread of
    # significands: the band where one rounding and two roundings differ
    sigs = [0, 1, 2, 3, 0x3F, 0x40, 0x41, 0x55, 0x7E, 0x7F]
    a, b = [], []
    for ea in range(1, 140, 3):
        for eb in range(1, 140):
            if -142 <= (ea - 127) + (eb - 127) <= -118:
                for sa in sigs:
                    for sb in sigs:
                        a.append((ea << 7) | sa)
                        b.append((eb << 7) | sb)
    a = np.array(a, np.uint16)
    b = np.array(b, np.uint16)
    _check_codec_equals_closed_form(OP_MUL, DT_BF16, a, b ^ 0x8000)


def test_bf16_quotient_is_rounded_once_over_the_subnormal_band():
    """Quotients that land in [2^-140, 2^-120): below 2^-126 the BF16 grid is fixed at 2^-133
    and a binary32 quotient is already rounded to the 2^-149 grid.  Three statements of the
    rule must agree there: the codec (64-bit carrier), the integer quotient with a sticky bit,
    and binary32 division followed by round-to-nearest-even narrowing (what a device computes)."""
    sigs = [0, 1, 2, 3, 0x2A, 0x3F, 0x40, 0x41, 0x55, 0x7E, 0x7F]
    a, b = [], []
    for ea in range(1, 120, 3):
        for eb in range(100, 255):
            if -142 <= ea - eb <= -118:
                for sa in sigs:
                    for sb in sigs:
                        a.append((ea << 7) | sa)
                        b.append((eb << 7) | sb)
    a = np.array(a, np.uint16)
    b = np.array(b, np.uint16) ^ 0x8000
    _check_codec_equals_closed_form(OP_DIV, DT_BF16, a[::3], b[::3])
    with np.errstate(all="ignore"):
        via_f32 = datagen.bf16_rne(datagen.bf16_to_f32(a) / datagen.bf16_to_f32(b))
    idx = np.arange(0, a.size, 7)
    want = np.array([L.iomo_scalar_binary(OP_DIV, DT_BF16, int(a[i]), int(b[i])) for i in idx],
                    np.uint16)
    assert np.array_equal(via_f32[idx], want)
    assert (want & 0x7FFF).min() == 0 and ((want & 0x7FFF) > 0).any()


def test_bf16_quotient_through_binary32_equals_the_codec_on_hash_patterns():
    n = 60000
    a = datagen.pattern_bits(16, n, 0x51)
    b = datagen.pattern_bits(16, n, 0x52)
    b[::5] = a[::5] ^ (datagen.pattern_bits(16, n, 0x53)[::5] & 0x7)   # quotients next to one
    with np.errstate(all="ignore"):
        q = datagen.bf16_to_f32(a) / datagen.bf16_to_f32(b)
    got = datagen.bf16_rne(q)
    got[np.isnan(q)] = 0x7FC0
    want = np.array([L.iomo_scalar_binary(OP_DIV, DT_BF16, int(x), int(y))
                     for x, y in zip(a.tolist(), b.tolist())], np.uint16)
    assert np.array_equal(got, want)


def test_f32_closed_form_equals_numpy_ieee():
    n = 200000
    a = datagen.pattern_bits(32, n, 5)
    b = datagen.pattern_bits(32, n, 6)
    with np.errstate(all="ignore"):
        for op, fn in ((OP_ADD, np.add), (OP_SUB, np.subtract), (OP_MUL, np.multiply),
                       (OP_DIV, np.divide)):
            r = fn(a.view(np.float32), b.view(np.float32)).view(np.uint32).copy()
            r[np.isnan(r.view(np.float32))] = 0x7FC00000
            idx = np.arange(0, n, 97)
            got = np.array([L.iomo_scalar_binary(op, DT_F32, int(a[i]), int(b[i])) for i in idx],
                           dtype=np.uint32)
            assert np.array_equal(got, r[idx])


def test_broadcast_mapping_invariant_brute_force():
    # out[p,r,c] reads in[p*(stride or 0), r or 0, c or 0]
    # shapes of test/backend/backend_conformance_add_gpu.hpp:242-394
    lhs_dims, rhs_dims, out_dims = (2, 1, 33), (1, 17, 1), (2, 17, 33)
    A = datagen.pattern_bits(32, 2 * 33, 1).reshape(lhs_dims) & 0x000FFFFF
    B = datagen.pattern_bits(32, 17, 2).reshape(rhs_dims) & 0x000FFFFF
    ta, tb, to = (iomo.HostTensor(DT_I32, d, fill=0xA5) for d in (lhs_dims, rhs_dims, out_dims))
    ta.view().from_logical(A)
    tb.view().from_logical(B)
    assert iomo.binary(OP_ADD, ta.view(), tb.view(), to.view()) == 0
    assert np.array_equal(to.view().to_logical(), (A + B).astype(np.uint32))
    # padding of the output owner is untouched
    mask = iomo.tile_plane(np.ones(out_dims, np.uint32)) == 0
    assert np.all(to.storage[mask] == 0xA5A5A5A5)


def test_binary_rejects_bad_shapes():
    a = iomo.HostTensor(DT_F32, (2, 16, 16)).view()
    b = iomo.HostTensor(DT_F32, (3, 16, 16)).view()
    o = iomo.HostTensor(DT_F32, (2, 16, 16)).view()
    assert iomo.binary(OP_ADD, a, b, o) == -1
    b1 = iomo.HostTensor(DT_F32, (1, 16, 16)).view()
    o3 = iomo.HostTensor(DT_F32, (3, 16, 16)).view()
    assert iomo.binary(OP_ADD, a, b1, o3) == -1
    assert iomo.binary(OP_ADD, a, b1, o) == 0


# ------------------------------------------------------------------ SiLU ----

def silu_ref64(x):
    if math.isnan(x):
        return math.nan
    if math.isinf(x):
        return -0.0 if x < 0 else math.inf
    if x == 0:
        return x
    if x < -700.0:
        # exp(-x) overflows binary64; x*exp(x) is the same value and underflows to -0
        return x * math.exp(x)
    return x / (1.0 + math.exp(-x))


def ordered(bits, width):
    sign = 1 << (width - 1)
    return (~bits) & ((1 << width) - 1) if bits & sign else bits | sign


@pytest.mark.parametrize("dtype,width,ulps", [(DT_BF16, 16, 1), (DT_F32, 32, 4)])
def test_silu_within_reference_ulp_ceiling(dtype, width, ulps):
    raws = datagen.pattern_bits(width, 4000, 0x51).tolist()
    raws += [0, 1 << (width - 1)]
    for raw in raws:
        if width == 16:
            x = float(datagen.bf16_to_f32(np.array([raw], np.uint16))[0])
        else:
            x = float(np.array([raw], np.uint32).view(np.float32)[0])
        got = L.iomo_scalar_silu(dtype, raw)
        want = silu_ref64(x)
        if math.isnan(want):
            assert got == (0x7FC0 if width == 16 else 0x7FC00000)
            continue
        with np.errstate(all="ignore"):
            w32 = np.array([want], np.float64).astype(np.float32)
        wbits = int(datagen.bf16_rne(w32)[0]) if width == 16 else int(w32.view(np.uint32)[0])
        assert abs(ordered(got, width) - ordered(wbits, width)) <= ulps, (hex(raw), hex(got), hex(wbits))


def test_silu_specials_and_negative_tail():
    f = lambda v: int(np.array([v], np.float32).view(np.uint32)[0])
    assert L.iomo_scalar_silu(DT_F32, f(np.inf)) == 0x7F800000
    assert L.iomo_scalar_silu(DT_F32, f(-np.inf)) == 0x80000000
    assert L.iomo_scalar_silu(DT_F32, 0x80000000) == 0x80000000
    assert L.iomo_scalar_silu(DT_F32, 0) == 0
    assert L.iomo_scalar_silu(DT_F32, 0xFFC00001) == 0x7FC00000
    assert L.iomo_scalar_silu(DT_BF16, 0xFF80) == 0x8000
    tail = L.iomo_scalar_silu(DT_F32, f(-104.0))
    assert tail & 0x80000000 and (tail & 0x7FFFFFFF) != 0  # negative, not flushed to zero
    assert L.iomo_scalar_silu(DT_I32, 0x12345678) == 0


# --------------------------------------------------------------- RMSNorm ----

@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32])
@pytest.mark.parametrize("rows,feats", [(1, 1), (15, 16), (16, 17), (17, 33), (3, 2048)])
def test_rmsnorm_all_ones_closed_form(dtype, rows, feats):
    eps = 1e-5
    one = 0x3F80 if dtype == DT_BF16 else 0x3F800000
    x = iomo.HostTensor(dtype, (rows, feats), fill=0x5A)
    w = iomo.HostTensor(dtype, (1, feats), fill=0x5A)
    o = iomo.HostTensor(dtype, (rows, feats), fill=0xA5)
    x.view().from_logical(np.full((rows, feats), one))
    if dtype == DT_BF16:
        wl = datagen.bf16_rne(datagen.uniform_f32(feats, 0.5, 1.5, 3))
        wf = datagen.bf16_to_f32(wl)
    else:
        wf = datagen.uniform_f32(feats, 0.5, 1.5, 3)
        wl = wf.view(np.uint32)
    w.view().from_logical(wl.reshape(1, feats))
    assert iomo.rmsnorm(x.view(), w.view(), o.view(), eps) == 0
    inv = np.float32(1.0) / np.sqrt(np.float32(1.0) + np.float32(eps))
    want = (np.float32(1.0) * inv) * wf
    want = datagen.bf16_rne(want) if dtype == DT_BF16 else want.view(np.uint32)
    got = o.view().to_logical()
    assert np.array_equal(got, np.broadcast_to(want, (rows, feats)))
    pad = iomo.tile_plane(np.ones((rows, feats), iomo.NP_OF[dtype])) == 0
    assert np.all(o.storage.view(np.uint8).reshape(-1, iomo.leaf_bytes(dtype))[pad] == 0xA5)


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32])
def test_rmsnorm_against_float64(dtype):
    rows, feats, eps = 9, 2048, 1e-5
    xf = datagen.normal_f32(rows * feats, 0, 1, 11).reshape(rows, feats)
    xf[3] *= 50
    wf = datagen.uniform_f32(feats, 0.5, 1.5, 12)
    if dtype == DT_BF16:
        xl, wl = datagen.bf16_rne(xf), datagen.bf16_rne(wf)
        xf, wf = datagen.bf16_to_f32(xl), datagen.bf16_to_f32(wl)
    else:
        xl, wl = xf.view(np.uint32), wf.view(np.uint32)
    x = iomo.HostTensor(dtype, (rows, feats))
    w = iomo.HostTensor(dtype, (1, feats))
    o = iomo.HostTensor(dtype, (rows, feats))
    x.view().from_logical(xl)
    w.view().from_logical(wl.reshape(1, feats))
    assert iomo.rmsnorm(x.view(), w.view(), o.view(), eps) == 0
    x64 = xf.astype(np.float64)
    want = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + eps) * wf.astype(np.float64)
    got = o.view().to_logical()
    if dtype == DT_BF16:
        g = datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(rows, feats)
        assert np.max(np.abs(g - want) / np.maximum(np.abs(want), 1e-30)) < 2 ** -7
    else:
        g = got.view(np.float32).astype(np.float64)
        assert np.max(np.abs(g - want) / np.maximum(np.abs(want), 1e-30)) < 1e-5


def test_rmsnorm_special_rows():
    feats = 32
    rows = np.zeros((4, feats), np.float32)
    rows[0, :] = 1.0
    rows[0, 5] = np.nan          # NaN row -> every output NaN, positive canonical
    rows[1, :] = -2.0
    rows[1, 7] = np.inf          # inf row -> finite*0 = signed zero, inf*0 = NaN
    rows[2, :] = 0.0             # zero row, eps>0 -> zeros keep sign
    rows[2, 3] = -0.0
    rows[3, :] = 3.0
    x = iomo.HostTensor(DT_F32, (4, feats))
    w = iomo.HostTensor(DT_F32, (1, feats))
    o = iomo.HostTensor(DT_F32, (4, feats))
    x.view().from_logical(rows.view(np.uint32))
    w.view().from_logical(np.ones((1, feats), np.float32).view(np.uint32))
    assert iomo.rmsnorm(x.view(), w.view(), o.view(), 1e-5) == 0
    got = o.view().to_logical()
    assert np.all(got[0] == 0x7FC00000)
    assert got[1, 7] == 0x7FC00000 and np.all(np.delete(got[1], 7) == 0x80000000)
    assert got[2, 3] == 0x80000000 and got[2, 0] == 0
    assert np.allclose(got[3].view(np.float32), 1.0, rtol=1e-5)


def test_rmsnorm_rejects_bad_requests():
    x = iomo.HostTensor(DT_F32, (4, 32)).view()
    o = iomo.HostTensor(DT_F32, (4, 32)).view()
    w = iomo.HostTensor(DT_F32, (1, 32)).view()
    w_bad = iomo.HostTensor(DT_F32, (2, 32)).view()
    assert iomo.rmsnorm(x, w_bad, o, 1e-5) == -1
    assert iomo.rmsnorm(x, w, x, 1e-5) == -1
    assert iomo.rmsnorm(x, w, o, -1.0) == -1
    assert iomo.rmsnorm(x, w, o, float("nan")) == -1
    xi = iomo.HostTensor(DT_I32, (4, 32)).view()
    oi = iomo.HostTensor(DT_I32, (4, 32)).view()
    wi = iomo.HostTensor(DT_I32, (1, 32)).view()
    assert iomo.rmsnorm(xi, wi, oi, 1e-5) == -2


# --------------------------------------------------------------- softmax ----

def run_row(values, L_, scale=1.0, a=None):
    s = np.zeros((1, 1, 1, len(values)), np.float32)
    s[0, 0, 0] = values
    return iomo.softmax(s, a=len(values) if a is None else a, L=L_, scale=scale)[0, 0, 0]


def test_softmax_special_rows():
    inf = np.inf
    r = run_row([np.nan, 0, 0, 0], 3)
    assert r[0] == 0x7FC0 and r[1] == 0x7FC0 and r[2] == 0x7FC0 and r[3] == 0
    r = run_row([inf, inf, -3, 99], 3)
    assert list(r) == [0x3F00, 0x3F00, 0, 0]
    r = run_row([-inf, -inf, -inf, 77], 3)
    assert list(r) == [0x7FC0, 0x7FC0, 0x7FC0, 0]
    r = run_row([0, -inf], 2)
    assert list(r) == [0x3F80, 0]
    r = run_row([0, -90.0], 2)
    assert r[0] == 0x3F80 and r[1] != 0 and r[1] < 0x0080   # nonzero BF16 subnormal
    # causal limit: row 0 at a=0 sees only token 0
    r = run_row([1.0, 5.0, 5.0], 3, a=0)
    assert list(r) == [0x3F80, 0, 0]


def test_softmax_rows_sum_to_one_and_mask_is_positive_zero():
    rows, cols = 33, 200
    s = datagen.normal_f32(rows * cols, 0, 3, 21).reshape(1, 1, rows, cols)
    p = iomo.softmax(s, a=0, L=150)
    pf = datagen.bf16_to_f32(p.reshape(-1)).reshape(rows, cols).astype(np.float64)
    for r in range(rows):
        vis = min(150, r + 1)
        assert np.all(p[0, 0, r, vis:] == 0)
        assert abs(pf[r, :vis].sum() - 1.0) < 2 ** -7
    want = np.exp(s[0, 0, 10, :11].astype(np.float64) - s[0, 0, 10, :11].max())
    want /= want.sum()
    got = pf[10, :11]
    assert np.max(np.abs(got - want) / want) < 2 ** -7
