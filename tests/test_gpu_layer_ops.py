"""GPU parity of cache_append, embedding and rope: through the C ABI against the CPU
oracle, and through the C++ backend next to the reference CPU backend.

Bars: cache_append and embedding move raw bits: bit-exact including untouched tile
padding and untouched destination rows.  RoPE: value class exact and
|actual - reference| <= one destination ulp + 2^-9 * pair norm (2^-44 for F64) against a
float64 evaluation, the reference's own acceptance rule
(test/backend/backend_conformance_rope.hpp:1180-1205); against the CPU oracle (binary32
arithmetic with the host libm) the same bound holds and most results are equal.
"""
import numpy as np
import pytest

import datagen
import iomo
from iom_amd import iomx
from iomo import (ALL_LEAVES, DT_BF16, DT_F32, DT_F64, DT_I16, DT_I32, DT_I64, DT_I8, DT_U8,
                  FLOAT_LEAVES, INTEGER_LEAVES, LEAF_BITS, LEAF_NAME)

pytestmark = pytest.mark.gpu
names = lambda ds: [LEAF_NAME[d] for d in ds]


@pytest.fixture(scope="module", autouse=True)
def _device():
    assert iomx.device_count() >= 1
    iomx.check(iomx.lib().iomx_set_device(0))
    yield


def pattern(dtype, count, salt):
    v = datagen.pattern_bits(LEAF_BITS[dtype], count, salt)
    return v & 1 if dtype == iomo.DT_BOOL else v


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


# -- cache append -------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ALL_LEAVES, ids=names(ALL_LEAVES))
@pytest.mark.parametrize("shape", [((2, 3, 5, 40), (2, 3, 37, 40), 0), ((2, 3, 5, 40), (2, 3, 37, 40), 32),
                                   ((4, 1, 64), (4, 20, 64), 19), ((1, 2, 17, 7), (1, 2, 17, 7), 0)])
def test_cache_append_bit_exact(dtype, shape):
    sd, dd, a = shape
    ds, hs = pair(dtype, sd, salt=3)
    dd_, hd = pair(dtype, dd, salt=4)
    assert iomx.cache_append(ds.view(), dd_.view(), a) == 0
    assert kernel_name() == "cache_append"
    assert iomo.cache_append(hs.view(), hd.view(), a) == 0
    assert same_storage(dd_, hd)
    ds.free(); dd_.free()


def test_cache_append_views_and_rejections():
    ds, hs = pair(DT_BF16, (4, 2, 3, 32), salt=5)
    dd, hd = pair(DT_BF16, (2, 4, 40, 32), salt=6)
    sv = lambda t: t.view().slice(0, 0, 2, 2).permute([1, 0])
    dv = lambda t: t.view().slice(1, 1, 2, 2).permute([1, 0])
    assert iomx.cache_append(sv(ds), dv(dd), 37) == 0
    assert iomo.cache_append(sv(hs), dv(hd), 37) == 0
    assert same_storage(dd, hd)
    for a in (38, 41, 1 << 40):
        assert iomx.cache_append(sv(ds), dv(dd), a) == -1
    d2, _ = pair(DT_BF16, (2, 2, 3, 48), salt=7)
    assert iomx.cache_append(d2.view(), dv(dd), 0) == -1
    assert iomx.cache_append(dv(dd), dv(dd), 0) == -1
    for t in (ds, dd, d2):
        t.free()


def test_cache_append_decode_steps_fill_a_cache():
    """Token-by-token appends (R = 1) then a prefill block: the cache equals the concatenation."""
    B, H, C, D = 2, 4, 40, 64
    cache, hc = pair(DT_BF16, (B, H, C, D), salt=1)
    rows = []
    pos = 0
    for step, R in enumerate([7, 1, 1, 1, 16, 1]):
        src, hsrc = pair(DT_BF16, (B, H, R, D), salt=100 + step)
        assert iomx.cache_append(src.view(), cache.view(), pos) == 0
        assert iomo.cache_append(hsrc.view(), hc.view(), pos) == 0
        rows.append(pattern(DT_BF16, B * H * R * D, 100 + step).reshape(B, H, R, D))
        pos += R
        src.free()
    assert same_storage(cache, hc)
    assert np.array_equal(cache.view().to_host()[:, :, :pos, :], np.concatenate(rows, axis=2))
    cache.free()


# -- embedding ----------------------------------------------------------------------

def run_embedding(dt, di, do):
    status = iomx.Buffer(32)
    status.fill(0xFF)
    iomx.synchronize()
    rc = iomx.embedding(dt, di, do, status)
    iomx.synchronize()
    word = int(status.download(np.uint32)[0])
    status.free()
    return rc, word


@pytest.mark.parametrize("dtype", ALL_LEAVES, ids=names(ALL_LEAVES))
def test_embedding_every_payload_leaf(dtype):
    V, F, R = 37, 40, 9
    dt, ht = pair(dtype, (V, F), salt=11)
    ids = (datagen.pattern_bits(32, 2 * 3 * R, 12) % V).reshape(2, 3, 1, R)
    di, hi = pair(DT_I32, (2, 3, 1, R), values=ids)
    do, ho = pair(dtype, (2, 3, R, F), salt=13)
    rc, word = run_embedding(dt.view(), di.view(), do.view())
    assert rc == 0 and word == 0
    assert kernel_name() == "embedding"
    assert iomo.embedding(ht.view(), hi.view(), ho.view()) == 0
    assert same_storage(do, ho)
    for t in (dt, di, do):
        t.free()


@pytest.mark.parametrize("index_dtype", INTEGER_LEAVES, ids=names(INTEGER_LEAVES))
def test_embedding_every_index_leaf_and_invalid_ids(index_dtype):
    bits = LEAF_BITS[index_dtype]
    signed = index_dtype in (iomo.DT_I2, iomo.DT_I4, DT_I8, DT_I16, DT_I32, DT_I64)
    top = (1 << (bits - 1 if signed else bits)) - 1
    V = min(top + 1, 50)
    R = 21
    dt, ht = pair(DT_BF16, (V, 16), salt=21)
    ids = (datagen.pattern_bits(32, 2 * R, 22) % V).astype(iomo.NP_OF[index_dtype]).reshape(2, 1, R)
    di, hi = pair(index_dtype, (2, 1, R), values=ids)
    do, ho = pair(DT_BF16, (2, R, 16))
    rc, word = run_embedding(dt.view(), di.view(), do.view())
    assert rc == 0 and word == 0
    assert iomo.embedding(ht.view(), hi.view(), ho.view()) == 0
    assert same_storage(do, ho)
    bad = ids.copy()
    bad[1, 0, R - 1] = (1 << bits) - 1 if bits < 64 else np.uint64(0xFFFFFFFFFFFFFFFF)
    if signed or (1 << bits) - 1 >= V:
        di2, _ = pair(index_dtype, (2, 1, R), values=bad)
        rc, word = run_embedding(dt.view(), di2.view(), do.view())
        assert rc == 0 and word == 1                   # raised status, no fault
        di2.free()
    for t in (dt, di, do):
        t.free()


def test_embedding_views_and_rejections():
    V, F, R = 20, 33, 5
    dt, ht = pair(DT_F32, (3, V, F), salt=31)
    ids = (datagen.pattern_bits(32, 4 * 2 * R, 32) % V).reshape(4, 2, 1, R).astype(np.uint8)
    di, hi = pair(DT_U8, (4, 2, 1, R), values=ids)
    do, ho = pair(DT_F32, (2, 6, R, F), salt=33)
    iv = lambda t: t.view().slice(0, 1, 2, 2).permute([1, 0])
    ov = lambda t: t.view().slice(1, 0, 2, 3).permute([1, 0])
    rc, word = run_embedding(dt.view().select(0, 2), iv(di), ov(do))
    assert rc == 0 and word == 0
    assert iomo.embedding(ht.view().select(0, 2), iv(hi), ov(ho)) == 0
    assert same_storage(do, ho)
    status = iomx.Buffer(32)
    assert iomx.embedding(dt.view(), iv(di), ov(do), status) == -1            # table must be rank two
    df, _ = pair(DT_F32, (2, 2, 1, R))
    assert iomx.embedding(dt.view().select(0, 0), df.view(), ov(do), status) == -2   # floating ids
    status.free()
    for t in (dt, di, do, df):
        t.free()


# -- rope ---------------------------------------------------------------------------

FMT = {13: (2, 1, 1), 14: (2, 3, 1), 15: (3, 2, 3), 16: (4, 3, 7), 17: (5, 2, 15), 19: (5, 10, 15),
       20: (8, 7, 127), 21: (8, 23, 127), 22: (11, 52, 1023)}


def decode(raw, dtype):
    """Raw encodings -> float64 (NaN / inf where the leaf has them)."""
    ebits, fbits, bias = FMT[dtype]
    raw = raw.astype(np.uint64)
    frac = (raw & np.uint64((1 << fbits) - 1)).astype(np.float64)
    exp = ((raw >> np.uint64(fbits)) & np.uint64((1 << ebits) - 1)).astype(np.int64)
    sign = np.where((raw >> np.uint64(ebits + fbits)) & np.uint64(1), -1.0, 1.0)
    mag = np.where(exp == 0, np.ldexp(frac, 1 - bias - fbits), np.ldexp(frac + (1 << fbits), exp - bias - fbits))
    top = (1 << ebits) - 1
    if dtype == 16:
        mag = np.where(exp == top, np.nan, mag)
    elif dtype not in (13, 14, 15):
        mag = np.where(exp == top, np.where(frac == 0, np.inf, np.nan), mag)
    return sign * mag


def ulp_at(ref, dtype):
    """Spacing of the leaf at |ref| (the subnormal spacing below the smallest normal)."""
    ebits, fbits, bias = FMT[dtype]
    e = np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** (1 - bias))))
    return np.ldexp(1.0, (e - fbits).astype(np.int64))


def finite_values(dtype, count, salt):
    bits = LEAF_BITS[dtype]
    v = datagen.pattern_bits(bits, count, salt)
    ebits, fbits, bias = FMT[dtype]
    if dtype in (13, 14, 15):
        return v
    top = (1 << ebits) - 1
    exp = (v.astype(np.uint64) >> np.uint64(fbits)) & np.uint64(top)
    if dtype in (20, 21, 22):
        exp = exp % np.uint64(17) + np.uint64(bias - 8)
    else:
        exp = np.where(exp == top, np.uint64(top - 1), exp)
    cleared = v.astype(np.uint64) & ~np.uint64(top << fbits)
    return (cleared | (exp << np.uint64(fbits))).astype(v.dtype)


def rope64(x, a, theta):
    *_, R, D = x.shape
    c = np.arange(D // 2)
    ang = (a + np.arange(R))[:, None] * theta ** (-2.0 * c / D)[None, :]
    x1, x2 = x[..., :D // 2], x[..., D // 2:]
    out = np.concatenate([x1 * np.cos(ang) - x2 * np.sin(ang), x2 * np.cos(ang) + x1 * np.sin(ang)], -1)
    norm = np.sqrt(x1 * x1 + x2 * x2)
    return out, np.concatenate([norm, norm], -1)


@pytest.mark.parametrize("dtype", FLOAT_LEAVES, ids=names(FLOAT_LEAVES))
@pytest.mark.parametrize("dims,a,family", [((2, 3, 5, 40), 1, "rope_general"), ((2, 3, 5, 40), 0, "rope_general"),
                                           ((2, 2, 33, 64), 0, "rope_pairs"), ((3, 4, 16, 128), 500, "rope_pairs"),
                                           ((1, 1, 2, 2), 7, "rope_general"),
                                           ((5, 7, 1, 64), 37, "rope_row"), ((3, 1, 32), 0, "rope_row"),
                                           ((2, 40, 1, 128), 1023, "rope_row")])
def test_rope_float_leaves(dtype, dims, a, family):
    theta = 10000.0
    vals = finite_values(dtype, int(np.prod(dims)), 41).reshape(dims)
    dx, hx = pair(dtype, dims, values=vals)
    do, ho = pair(dtype, dims, salt=42)
    assert iomx.rope(dx.view(), do.view(), a, theta) == 0
    assert kernel_name() == family
    assert iomo.rope(hx.view(), ho.view(), a, theta) == 0
    got_raw = do.view().to_host()
    got = decode(got_raw, dtype)
    x = decode(vals, dtype)
    ref, norm = rope64(x, a, theta)
    # the leaf's largest finite magnitude bounds what can be stored: clamp the float64 value
    ebits, fbits, bias = FMT[dtype]
    slack = np.ldexp(norm, -44 if dtype == DT_F64 else -9)
    finite = np.isfinite(got) & np.isfinite(ref)
    bound = ulp_at(ref, dtype) + slack
    saturated = ~np.isfinite(decode(ho.view().to_logical(), dtype)) | (np.abs(ref) >= np.abs(got) + bound)
    ok = (np.abs(got - ref) <= bound) | ~finite | saturated
    assert ok.all()
    # against the CPU arithmetic: same classes, at most the same bound apart, mostly equal
    want_raw = ho.view().to_logical()
    want = decode(want_raw, dtype)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    both = np.isfinite(got) & np.isfinite(want)
    assert (np.abs(got - want)[both] <= 2 * bound[both]).all()
    assert np.array_equal(np.isinf(got), np.isinf(want))
    if a == 0:      # row 0 is a raw copy
        assert np.array_equal(got_raw[..., 0, :], vals[..., 0, :])
    equal = float((got_raw == want_raw).mean())
    print(LEAF_NAME[dtype], dims, a, "equal to the CPU arithmetic: %.4f" % equal, flush=True)
    if LEAF_BITS[dtype] <= 16:     # binary32 / binary64 results differ in the last place with the libm
        assert equal > 0.9
    # tile padding of the output untouched: compare raw storage where every element agrees
    if equal == 1.0:
        assert same_storage(do, ho)
    dx.free(); do.free()


def test_rope_single_row_planes_through_views():
    """A decode step: one row per plane, the planes reached through a permuted and sliced view."""
    dims = (6, 9, 1, 64)
    vals = finite_values(DT_BF16, int(np.prod(dims)), 45).reshape(dims)
    dx, hx = pair(DT_BF16, dims, values=vals)
    do, ho = pair(DT_BF16, (9, 3, 1, 64), salt=46)
    xv = lambda t: t.view().permute([1, 0]).slice(1, 1, 3, 2)
    assert iomx.rope(xv(dx), do.view(), 123, 10000.0) == 0
    assert kernel_name() == "rope_row"
    assert iomo.rope(xv(hx), ho.view(), 123, 10000.0) == 0
    got, want = do.view().to_host(), ho.view().to_logical()
    assert (np.abs(got.astype(np.int64) - want.astype(np.int64)) <= 1).all()
    assert float((got == want).mean()) > 0.9
    mask = iomo.tile_plane(np.ones((9, 3, 1, 64), np.uint16)) == 0
    assert np.array_equal(do.raw()[mask], ho.storage[mask])      # the 15 padding rows of every tile untouched
    dx.free(); do.free()


def test_rope_views_specials_and_rejections():
    dims = (4, 2, 16, 128)
    vals = (np.arange(int(np.prod(dims)), dtype=np.uint32) * 4 + 3).astype(np.uint16).reshape(dims)
    dx, hx = pair(DT_BF16, dims, values=vals)              # every fourth BF16 encoding: NaN, inf, subnormals
    do, ho = pair(DT_BF16, (2, 4, 16, 128), salt=44)
    xv = lambda t: t.view().permute([1, 0])
    assert iomx.rope(xv(dx), do.view(), 7, 500000.0) == 0
    assert iomo.rope(xv(hx), ho.view(), 7, 500000.0) == 0
    got, want = do.view().to_host(), ho.view().to_logical()
    g, w = decode(got, DT_BF16), decode(want, DT_BF16)
    assert np.array_equal(np.isnan(g), np.isnan(w))
    assert np.all(got[np.isnan(g)] == 0x7FC0)                                     # canonical NaN
    fin = np.isfinite(g) & np.isfinite(w)
    assert np.array_equal(np.isinf(g), np.isinf(w)) and np.array_equal(g[np.isinf(g)], w[np.isinf(w)])
    d = np.abs(got[fin].astype(np.int64) - want[fin].astype(np.int64))
    assert (d <= 1).mean() > 0.999                    # one BF16 step wherever the operands are moderate
    o = do
    for args in ((0, 0.5), (0, float("inf")), (0, float("nan")), (1 << 24, 10000.0)):
        assert iomx.rope(xv(dx), o.view(), *args) == -1
    assert iomx.rope(dx.view(), dx.view(), 0, 10000.0) == -1
    d3, _ = pair(DT_F32, (2, 4, 15))
    d4, _ = pair(DT_F32, (2, 4, 15))
    assert iomx.rope(d3.view(), d4.view(), 0, 10000.0) == -1
    di, _ = pair(DT_I32, (2, 4, 16))
    dj, _ = pair(DT_I32, (2, 4, 16))
    assert iomx.rope(di.view(), dj.view(), 0, 10000.0) == -2
    for t in (dx, do, d3, d4, di, dj):
        t.free()


def test_rope_tinyllama_shape_against_float64():
    """[B=4, H=32, S=512, D=64] BF16, theta = 10000, positions 0..511."""
    dims = (4, 32, 512, 64)
    x32 = datagen.normal_f32(int(np.prod(dims)), 0, 1, 61)
    vals = datagen.bf16_rne(x32).reshape(dims)
    dx = iomx.DeviceTensor(DT_BF16, dims)
    do = iomx.DeviceTensor(DT_BF16, dims)
    dx.view().from_host(vals)
    assert iomx.rope(dx.view(), do.view(), 0, 10000.0) == 0
    got = decode(do.view().to_host(), DT_BF16)
    ref, norm = rope64(decode(vals, DT_BF16), 0, 10000.0)
    assert (np.abs(got - ref) <= ulp_at(ref, DT_BF16) + np.ldexp(norm, -9)).all()
    # the rotation preserves the norm of every pair up to the BF16 rounding of its two parts
    g1, g2 = got[..., :32], got[..., 32:]
    assert np.abs(np.sqrt(g1 * g1 + g2 * g2) - norm[..., :32]).max() <= 2.0 ** -6 * norm.max()
    # oracle on one plane
    hx, ho = iomo.HostTensor(DT_BF16, (1, 1, 512, 64)), iomo.HostTensor(DT_BF16, (1, 1, 512, 64))
    hx.view().from_logical(vals[3:4, 31:32])
    assert iomo.rope(hx.view(), ho.view(), 0, 10000.0) == 0
    mine, cpu = do.view().to_host()[3, 31], ho.view().to_logical()[0, 0]
    d = np.abs(mine.astype(np.int64) - cpu.astype(np.int64))
    print("rope BF16 [512,64] vs CPU arithmetic: %d of %d differ, %d by more than one step "
          "(cancelling pairs, tiny results)" % ((d > 0).sum(), d.size, (d > 1).sum()), flush=True)
    # a result far below its pair's norm carries the absolute error of the products, many of
    # its own steps: the bound is the reference's, one step plus 2^-9 of the pair norm
    w = decode(cpu, DT_BF16)
    assert (np.abs(decode(mine, DT_BF16) - w) <= ulp_at(w, DT_BF16) + np.ldexp(norm[3, 31], -9)).all()
    assert (d > 1).mean() < 1e-3
    dx.free(); do.free()


# -- through the C++ backend, next to the reference CPU backend -----------------------

@pytest.fixture(scope="module")
def devices():
    if not iomo.mi355x_available():
        pytest.skip("oracle/_ref/libiom_mi355x_shim.so not built (needs the reference headers)")
    gpu = iomo.mi355x_backend(arena_bytes=1 << 28, max_in_flight=4)
    cpu = iomo.cpu_backend_beside_mi355x()
    yield cpu, gpu
    gpu.close()
    cpu.close()


def on_both(devices, dtype, dims, values):
    out = []
    for dev in devices:
        t = dev.tensor(dtype, dims)
        t.view().from_host(values)
        out.append(t)
    return out


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32, iomo.DT_U4, DT_F64], ids=["BF16", "F32", "U4", "F64"])
def test_backend_cache_append_and_embedding(devices, dtype):
    cpu, gpu = devices
    src = pattern(dtype, 2 * 3 * 5 * 40, 1).reshape(2, 3, 5, 40)
    dst = pattern(dtype, 2 * 3 * 37 * 40, 2).reshape(2, 3, 37, 40)
    cs, gs = on_both(devices, dtype, src.shape, src)
    cd, gd = on_both(devices, dtype, dst.shape, dst)
    assert cpu.cache_append(cs.view(), cd.view(), 30) > 0
    assert gpu.cache_append(gs.view(), gd.view(), 30) > 0, gpu.error()
    assert np.array_equal(cd.view().to_host(), gd.view().to_host())
    assert gpu.cache_append(gs.view(), gd.view(), 33) == -1
    table = pattern(dtype, 37 * 40, 3).reshape(37, 40)
    ids = (datagen.pattern_bits(32, 2 * 9, 4) % 37).astype(np.uint16).reshape(2, 1, 9)
    ct, gt = on_both(devices, dtype, table.shape, table)
    ci, gi = on_both(devices, iomo.DT_U16, ids.shape, ids)
    co, go = on_both(devices, dtype, (2, 9, 40), np.zeros((2, 9, 40), iomo.NP_OF[dtype]))
    tc, wc = cpu.embedding(ct.view(), ci.view(), co.view())
    tg, wg = gpu.embedding(gt.view(), gi.view(), go.view())
    assert tc > 0 and tg > 0 and wc == 0 and wg == 0, gpu.error()
    assert np.array_equal(co.view().to_host(), go.view().to_host())
    ids[1, 0, 8] = 37                                                  # out of the vocabulary
    ci2, gi2 = on_both(devices, iomo.DT_U16, ids.shape, ids)
    tc, wc = cpu.embedding(ct.view(), ci2.view(), co.view())
    tg, wg = gpu.embedding(gt.view(), gi2.view(), go.view())
    assert tc > 0 and tg > 0 and wc == -1 and wg == -1                 # accepted, then InvalidArgument on wait
    # the queue keeps working after a retained data failure
    tg, wg = gpu.embedding(gt.view(), gi.view(), go.view())
    assert tg > 0 and wg == 0
    assert np.array_equal(co.view().to_host()[0], go.view().to_host()[0])
    for t in (cs, gs, cd, gd, ct, gt, ci, gi, co, go, ci2, gi2):
        t.close()


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32], ids=["BF16", "F32"])
def test_backend_rope(devices, dtype):
    cpu, gpu = devices
    dims = (2, 4, 33, 64)
    x32 = datagen.normal_f32(int(np.prod(dims)), 0, 1, 71)
    vals = (datagen.bf16_rne(x32) if dtype == DT_BF16 else x32.view(np.uint32)).reshape(dims)
    cx, gx = on_both(devices, dtype, dims, vals)
    co, go = on_both(devices, dtype, dims, np.zeros(dims, iomo.NP_OF[dtype]))
    assert cpu.rope(cx.view(), co.view(), 5, 10000.0) > 0
    assert gpu.rope(gx.view(), go.view(), 5, 10000.0) > 0, gpu.error()
    a, b = decode(co.view().to_host(), dtype), decode(go.view().to_host(), dtype)
    ref, norm = rope64(decode(vals, dtype), 5, 10000.0)
    assert (np.abs(b - ref) <= ulp_at(ref, dtype) + np.ldexp(norm, -9)).all()
    assert (np.abs(a - b) <= 2 * ulp_at(ref, dtype) + np.ldexp(norm, -12)).all()
    assert gpu.rope(gx.view(), gx.view(), 5, 10000.0) == -1
    for t in (cx, gx, co, go):
        t.close()
