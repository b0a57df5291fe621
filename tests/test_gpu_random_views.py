"""Differential test over seeded random views: the HIP library against the CPU oracle.

Every case draws a result shape of 2 to 5 axes, operands that broadcast along any subset of
them (including operands of lower rank), and for every operand an owner that is reached
through select / strided slice / permute; owners are pre-filled, so whatever a kernel writes
outside the selected window shows as a storage difference.  Binary operations and copy are
bit-exact (F64 against the binary64-carrier rule); RMSNorm is within one encoding step of the
leaf / 1e-5 relative.  The same cases run between the oracle and the compiled reference in
test_oracle_random_views.py.
"""
import ctypes

import numpy as np
import pytest

import datagen
import iomo
import view_cases
from iom_amd import iomx
from iomo import (DT_BF16, DT_F16, DT_F32, DT_F64, DT_F6_E2M3, DT_F8_E4M3FN, DT_I32, DT_I64, DT_I8, DT_U4,
                  FLOAT_LEAVES, LEAF_BITS, LEAF_NAME, OP_ADD, OP_DIV, OP_MUL, OP_SUB)

pytestmark = pytest.mark.gpu

LEAVES = tuple(iomo.NUMERIC_LEAVES)          # all 21: every kernel family sees every kind of view
CASES = 420


@pytest.fixture(scope="module", autouse=True)
def _device():
    assert iomx.device_count() >= 1
    iomx.check(iomx.lib().iomx_set_device(0))
    yield


def pair(dtype, dims, salt, small=False):
    dt = iomx.DeviceTensor(dtype, dims, fill=0x5A)
    ht = iomo.HostTensor(dtype, dims, fill=0x5A)
    values = datagen.pattern_bits(LEAF_BITS[dtype], int(np.prod(dims)), salt).reshape(dims)
    if dtype == iomo.DT_BOOL:
        values = values & 1                              # BOOL host bytes are zero or one
    if small and dtype in (iomo.DT_F8_E4M3FN, iomo.DT_F8_E5M2):
        values = values & 0xBF                           # magnitudes below 2: no NaN, no overflow
    dt.view().from_host(values)
    ht.view().from_logical(values)
    return dt, ht


def same_storage(dt, ht):
    return np.array_equal(dt.raw().view(np.uint8), ht.storage.view(np.uint8))


@pytest.mark.parametrize("case", range(CASES))
def test_binary_on_random_views(case):
    dtype = LEAVES[case % len(LEAVES)]
    op = (OP_ADD, OP_MUL, OP_SUB, OP_DIV)[(case // len(LEAVES)) % 4]
    if op == OP_DIV and dtype not in FLOAT_LEAVES:
        op = OP_SUB
    lead, rows, cols, operands = view_cases.binary_case(case)
    # every other block of four operations draws small magnitudes for the 8-bit floating leaves:
    # tile rows that the kernel rounds with the conversion instructions, not element by element
    small = (case // (4 * len(LEAVES))) % 2 == 1
    owners = [pair(dtype, dims, 0x900 + 3 * case + i, small) for i, (dims, _) in enumerate(operands)]
    dv = [view_cases.apply(d.view(), steps) for (d, _), (_, steps) in zip(owners, operands)]
    hv = [view_cases.apply(h.view(), steps) for (_, h), (_, steps) in zip(owners, operands)]
    rc = iomx.binary(op, dv[0], dv[1], dv[2])
    assert rc == 0, (iomx.lib().iomx_error_string(rc), LEAF_NAME[dtype], operands)
    assert iomo.binary(op, hv[0], hv[1], hv[2], ieee=True) == 0
    assert same_storage(*owners[2]), (LEAF_NAME[dtype], op, lead, rows, cols, operands)
    for d, h in owners[:2]:
        assert same_storage(d, h)                       # inputs untouched
    for d, _ in owners:
        d.free()


@pytest.mark.parametrize("case", range(120))
def test_binary_on_random_views_of_rank_up_to_eight(case):
    """Five or six leading axes of extent 1-2 (rank seven or eight, the largest a shape can have:
    include/iom/tensor.hpp:83-85), sliced, permuted and broadcast like the cases above."""
    dtype = (iomo.DT_BF16, iomo.DT_I32, iomo.DT_U8, iomo.DT_F32, iomo.DT_U4, iomo.DT_F8_E5M2)[case % 6]
    op = (OP_ADD, OP_MUL, OP_SUB)[(case // 6) % 3]
    draw = case
    lead, rows, cols, operands = view_cases.binary_case(draw, max_lead=6, max_extent=2, salt=0x808)
    while len(lead) < 5:
        draw += 1000
        lead, rows, cols, operands = view_cases.binary_case(draw, max_lead=6, max_extent=2, salt=0x808)
    owners = [pair(dtype, dims, 0x3F00 + 3 * case + i, True) for i, (dims, _) in enumerate(operands)]
    dv = [view_cases.apply(d.view(), steps) for (d, _), (_, steps) in zip(owners, operands)]
    hv = [view_cases.apply(h.view(), steps) for (_, h), (_, steps) in zip(owners, operands)]
    rc = iomx.binary(op, dv[0], dv[1], dv[2])
    assert rc == 0, (iomx.lib().iomx_error_string(rc), LEAF_NAME[dtype], operands)
    assert iomo.binary(op, hv[0], hv[1], hv[2], ieee=True) == 0
    assert same_storage(*owners[2]), (LEAF_NAME[dtype], op, lead, rows, cols, operands)
    for d, _ in owners:
        d.free()


@pytest.mark.parametrize("case", range(CASES // 2))
def test_copy_on_random_views(case):
    dtype = (LEAVES + (iomo.DT_BOOL, iomo.DT_F8_E8M0, iomo.DT_U2))[case % (len(LEAVES) + 3)]
    lead, rows, cols, operands = view_cases.unary_case(case)
    owners = [pair(dtype, dims, 0xA00 + 2 * case + i) for i, (dims, _) in enumerate(operands)]
    dv = [view_cases.apply(d.view(), steps) for (d, _), (_, steps) in zip(owners, operands)]
    hv = [view_cases.apply(h.view(), steps) for (_, h), (_, steps) in zip(owners, operands)]
    assert iomx.copy(dv[0], dv[1]) == 0
    assert iomo.copy(hv[0], hv[1]) == 0
    assert same_storage(*owners[1]), (LEAF_NAME[dtype], lead, rows, cols, operands)
    assert same_storage(*owners[0])
    for d, _ in owners:
        d.free()


@pytest.mark.parametrize("case", range(CASES // 3))
def test_silu_on_random_views(case):
    dtype = (DT_BF16, DT_F32, DT_F16, DT_F8_E4M3FN, DT_F64)[case % 5]
    lead, rows, cols, operands = view_cases.unary_case(case, salt=404)
    x32 = datagen.normal_f32(int(np.prod(operands[0][0])), 0, 3, 0xE00 + case)
    enc = {DT_BF16: datagen.bf16_rne, DT_F32: lambda v: v.view(np.uint32),
           DT_F16: lambda v: v.astype(np.float16).view(np.uint16),
           DT_F64: lambda v: v.astype(np.float64).view(np.uint64),
           DT_F8_E4M3FN: lambda v: (datagen.pattern_bits(8, v.size, 0xE50 + case) & 0x77).astype(np.uint8)}[dtype]
    values = enc(x32).reshape(operands[0][0])
    dx = iomx.DeviceTensor(dtype, operands[0][0], fill=0x5A)
    hx = iomo.HostTensor(dtype, operands[0][0], fill=0x5A)
    dx.view().from_host(values)
    hx.view().from_logical(values)
    do, ho = pair(dtype, operands[1][0], 0xF00 + case)
    dxv, hxv = view_cases.apply(dx.view(), operands[0][1]), view_cases.apply(hx.view(), operands[0][1])
    dov, hov = view_cases.apply(do.view(), operands[1][1]), view_cases.apply(ho.view(), operands[1][1])
    assert iomx.silu(dxv, dov) == 0
    assert iomo.silu(hxv, hov) == 0
    got, want = dov.to_host(), hov.to_logical()
    if dtype == DT_F32:
        # each side is within 4 binary32 units of the exact value (test_scalar_silu.cpp:163-167)
        def ordered(bits):
            b = bits.astype(np.int64)
            return np.where(b & 0x80000000, 0x80000000 - b, b)
        assert np.abs(ordered(got) - ordered(want)).max() <= 8, (lead, rows, cols, operands)
    elif dtype == DT_F64:
        g, w = got.view(np.float64), want.view(np.float64)
        assert np.all(np.abs(g - w) <= 1e-6 * np.abs(w) + 1e-300), (lead, rows, cols, operands)
    else:
        assert np.abs(got.astype(np.int64) - want.astype(np.int64)).max() <= 1, (lead, rows, cols, operands)
    # the rest of the output owner is what it was
    marker = iomo.HostTensor(dtype, operands[1][0], fill=0)
    mv = view_cases.apply(marker.view(), operands[1][1])
    mv.from_logical(np.full(mv.dims, 1, iomo.NP_OF[dtype]))
    untouched = marker.storage == 0
    assert np.array_equal(do.raw()[untouched], ho.storage[untouched])
    for t in (dx, do):
        t.free()


@pytest.mark.parametrize("case", range(CASES // 2))
def test_rmsnorm_on_random_views(case):
    dtype = (DT_BF16, DT_F32, DT_F16)[case % 3]
    lead, rows, cols, operands = view_cases.unary_case(case, salt=303)
    n = [int(np.prod(dims)) for dims, _ in operands]
    x32 = datagen.normal_f32(n[0], 0, 1, 0xB00 + case)
    w32 = datagen.uniform_f32(cols, 0.5, 1.5, 0xC00 + case)
    enc = {DT_BF16: datagen.bf16_rne, DT_F32: lambda v: v.view(np.uint32),
           DT_F16: lambda v: v.astype(np.float16).view(np.uint16)}[dtype]
    dx = iomx.DeviceTensor(dtype, operands[0][0], fill=0x5A)
    hx = iomo.HostTensor(dtype, operands[0][0], fill=0x5A)
    dx.view().from_host(enc(x32).reshape(operands[0][0]))
    hx.view().from_logical(enc(x32).reshape(operands[0][0]))
    dw = iomx.DeviceTensor(dtype, (1, cols), fill=0x5A)
    hw = iomo.HostTensor(dtype, (1, cols), fill=0x5A)
    dw.view().from_host(enc(w32).reshape(1, cols))
    hw.view().from_logical(enc(w32).reshape(1, cols))
    do, ho = pair(dtype, operands[1][0], 0xD00 + case)
    dxv, hxv = view_cases.apply(dx.view(), operands[0][1]), view_cases.apply(hx.view(), operands[0][1])
    dov, hov = view_cases.apply(do.view(), operands[1][1]), view_cases.apply(ho.view(), operands[1][1])
    assert iomx.rmsnorm(dxv, dw.view(), dov, 1e-5) == 0
    assert iomo.rmsnorm(hxv, hw.view(), hov, 1e-5) == 0
    got, want = do.raw(), ho.storage
    # which slots of the output owner the view selects: written through the same view steps
    marker = iomo.HostTensor(dtype, operands[1][0], fill=0)
    mv = view_cases.apply(marker.view(), operands[1][1])
    mv.from_logical(np.full(mv.dims, 1, iomo.NP_OF[dtype]))
    touched = marker.storage != 0
    assert touched.sum() == int(np.prod(mv.dims))
    if dtype == DT_F32:
        g, w = got.view(np.float32)[touched], want.view(np.float32)[touched]
        assert np.all(np.abs(g - w) <= 1e-5 * np.abs(w) + 1e-30), (lead, rows, cols, operands)
    else:
        step = np.abs(got[touched].astype(np.int64) - want[touched].astype(np.int64))
        assert step.max() <= 1, (lead, rows, cols, operands)
    # outside the selected window nothing changed: the pre-filled storage is still there
    assert np.array_equal(got[~touched], want[~touched])
    for t in (dx, dw, do):
        t.free()


# Row widths on both sides of every switch of the RMSNorm launch rule (chunks of one band:
# 64, 256, ... 131072; a BF16 tile column is 32 chunks of a band, an F32 one 64), whole tiles
# and ragged widths, with a partial last band and two planes.
BOUNDARY_TILE_COLUMNS = sorted({t + d for t in (1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048, 4096)
                                for d in (-1, 0, 1) if t + d >= 1})


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32], ids=["BF16", "F32"])
@pytest.mark.parametrize("tile_columns", BOUNDARY_TILE_COLUMNS)
def test_rmsnorm_on_both_sides_of_every_launch_boundary(dtype, tile_columns):
    for feats in (tile_columns * 16, tile_columns * 16 - 5):
        dims = (2, 19, feats)
        n = int(np.prod(dims))
        x32 = datagen.normal_f32(n, 0, 1, 0x1100 + tile_columns)
        w32 = datagen.uniform_f32(feats, 0.5, 1.5, 0x1200 + tile_columns)
        enc = datagen.bf16_rne if dtype == DT_BF16 else (lambda v: v.view(np.uint32))
        dx = iomx.DeviceTensor(dtype, dims, fill=0x5A)
        hx = iomo.HostTensor(dtype, dims, fill=0x5A)
        dx.view().from_host(enc(x32).reshape(dims))
        hx.view().from_logical(enc(x32).reshape(dims))
        dw = iomx.DeviceTensor(dtype, (1, feats), fill=0x5A)
        hw = iomo.HostTensor(dtype, (1, feats), fill=0x5A)
        dw.view().from_host(enc(w32).reshape(1, feats))
        hw.view().from_logical(enc(w32).reshape(1, feats))
        do, ho = pair(dtype, dims, 0x1300 + tile_columns)
        assert iomx.rmsnorm(dx.view(), dw.view(), do.view(), 1e-5) == 0
        assert iomo.rmsnorm(hx.view(), hw.view(), ho.view(), 1e-5) == 0
        got, want = do.view().to_host(), ho.view().to_logical()
        if dtype == DT_F32:
            g, w = got.view(np.float32), want.view(np.float32)
            assert np.all(np.abs(g - w) <= 1e-5 * np.abs(w) + 1e-30), (feats, iomx.last_launch().kernel)
        else:
            assert np.abs(got.astype(np.int64) - want.astype(np.int64)).max() <= 1, (feats, iomx.last_launch().kernel)
        pad = iomo.tile_plane(np.ones(dims, ho.storage.dtype)) == 0
        assert np.array_equal(do.raw()[pad], ho.storage[pad])
        for t in (dx, dw, do):
            t.free()


def gpu_softmax(scores, a, L, scale, pcols):
    scores = np.ascontiguousarray(scores, np.float32)
    planes, heads, prow, scol = scores.shape
    sb = iomx.Buffer(scores.nbytes)
    pb = iomx.Buffer(planes * heads * prow * pcols * 2)
    sb.upload(scores)
    pb.fill(0xAA)
    d = iomx.softmax_desc(sb.ptr.value, pb.ptr.value, planes, heads, prow, scol, a, L, scale, None)
    d.probability_layout = iomx.dense_layout(heads, prow, pcols)
    rc = iomx.softmax(d)
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    iomx.synchronize()
    out = pb.download(np.uint16).reshape(planes, heads, prow, pcols)
    sb.free()
    pb.free()
    return out


SOFTMAX_COLUMNS = sorted({c + d for c in (8, 256, 512, 1024, 2048, 4096) for d in (-4, -1, 0, 1, 4)} | {4, 5, 5000})


@pytest.mark.parametrize("cols", SOFTMAX_COLUMNS)
def test_softmax_on_both_sides_of_every_launch_boundary(cols):
    """Row lengths around every switch of the softmax launch rule (chunks of 256 columns per
    lane group: 256 ... 4096, then the generic kernel), lengths that are no multiple of four,
    the causal limit inside the first chunk, inside a middle chunk and at the row's end, and a
    probability row wider than the score row."""
    planes, heads, rows = 2, 2, 9
    shape = (planes, heads, rows, cols)
    s = datagen.normal_f32(int(np.prod(shape)), 0, 3, 0x1400 + cols).reshape(shape)
    r = np.arange(rows)[:, None]
    t = np.arange(cols)[None, :]
    for L, a in ((cols, cols - rows if cols > rows else 0), (max(cols - 3, 1), 0), (cols, max(cols // 2 - 4, 0))):
        for pcols in (cols, cols + 4):
            got = gpu_softmax(s, a, L, 0.125, pcols)
            want = iomo.softmax(s, a=a, L=L, scale=0.125)
            masked = np.broadcast_to((t > a + r) | (t >= L), shape)
            view = got[..., :cols]
            assert np.all(view[masked] == 0), (cols, L, a, pcols, iomx.last_launch().kernel)
            assert np.all(got[..., cols:] == 0)
            step = np.abs(view[~masked].astype(np.int64) - want[~masked].astype(np.int64))
            assert step.max() <= 1, (cols, L, a, pcols, iomx.last_launch().kernel)


def bf16_values(count, salt):
    """BF16 encodings with exponents within 2^-3 .. 2^1: sums of a few hundred products stay far
    from overflow and from total cancellation."""
    v = datagen.pattern_bits(16, count, salt).astype(np.uint64)
    exp = (v >> np.uint64(7)) & np.uint64(0xFF)
    exp = exp % np.uint64(5) + np.uint64(124)
    return ((v & np.uint64(0x807F)) | (exp << np.uint64(7))).astype(np.uint16)


@pytest.mark.parametrize("case", range(160))
def test_linear_bf16_on_random_shapes_and_views(case):
    """Rows, inner extent, heads and head size drawn at random, so the choice among the scalar,
    direct, split-inner and workgroup-tiled kernels and every ragged edge of their tiles is
    exercised; x is reached through strided leading axes, the output is ordinary or head-planar
    and pre-filled.  Bar: |actual - q| <= max(ulp(q), 2^-7, 2^-6 |q|) against float64 rounded once
    (docs/BACKEND_CONTRACT/linear-projections.md:334-341); nothing outside the window changes."""
    rng = view_cases.Stream(case, 505)
    nlead = rng.below(3)
    lead = tuple(1 + rng.below(3) for _ in range(nlead))
    big = rng.chance(1, 4)
    R = (1, 1, 3, 16, 17, 40, 130, 300)[rng.below(8 if big else 6)]
    s = rng.below(20)
    x_rows = s + R + rng.below(5)
    inner = (16, 32, 40, 64, 96, 200, 256, 512, 1000)[rng.below(9 if big else 7)]
    D = (16, 32, 48, 64, 80, 128)[rng.below(6)]
    H = 1 + rng.below(8 if big else 4)
    head_planar = rng.chance(1, 2)
    x_owner, x_steps = view_cases.viewed_operand(rng, lead, x_rows, inner)
    xv = bf16_values(int(np.prod(x_owner)), 0x1500 + case).reshape(x_owner)
    wv = bf16_values(H * D * inner, 0x1600 + case).reshape(H * D, inner)
    dx = iomx.DeviceTensor(DT_BF16, x_owner, fill=0x5A)
    hx = iomo.HostTensor(DT_BF16, x_owner, fill=0x5A)
    dx.view().from_host(xv)
    hx.view().from_logical(xv)
    dw = iomx.DeviceTensor(DT_BF16, (H * D, inner), fill=0x5A)
    dw.view().from_host(wv)
    out_dims = lead + ((H, R, D) if head_planar else (R, H * D))
    do, ho = pair(DT_BF16, out_dims, 0x1700 + case)
    dxv = view_cases.apply(dx.view(), x_steps)
    # the ordinary layout is one head as wide as the weight (src/device_ops_neural.cpp)
    rc = iomx.linear(dxv, dw.view(), do.view(), s, R, head_planar, H if head_planar else 1,
                     D if head_planar else H * D)
    assert rc == 0, (iomx.lib().iomx_error_string(rc), x_owner, x_steps, s, R, H, D, head_planar)
    kernel = iomx.last_launch().kernel.decode()
    got = do.view().to_host()
    x_logical = view_cases.apply(hx.view(), x_steps).to_logical()
    planes = int(np.prod(lead)) if lead else 1
    x3 = x_logical.reshape(planes, x_rows, inner)[:, s:s + R, :]
    g3 = (got.reshape(planes, H, R, D).transpose(0, 2, 1, 3).reshape(planes, R, H * D) if head_planar
          else got.reshape(planes, R, H * D))
    x64 = datagen.bf16_to_f32(x3.reshape(-1)).astype(np.float64).reshape(x3.shape)
    w64 = datagen.bf16_to_f32(wv.reshape(-1)).astype(np.float64).reshape(wv.shape)
    ref = x64 @ w64.T
    q = datagen.bf16_to_f32(datagen.bf16_rne(ref.astype(np.float32).reshape(-1))).astype(np.float64).reshape(ref.shape)
    g = datagen.bf16_to_f32(g3.reshape(-1)).astype(np.float64).reshape(ref.shape)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(q), 1e-30))) - 7)
    ok = np.abs(g - q) <= np.maximum(np.maximum(ulp, 2.0 ** -7), 2.0 ** -6 * np.abs(q))
    assert ok.all(), (kernel, x_owner, x_steps, s, R, inner, H, D, head_planar, int((~ok).sum()))
    pad = iomo.tile_plane(np.ones(out_dims, np.uint16)) == 0
    assert np.array_equal(do.raw()[pad], ho.storage[pad]), kernel
    for t in (dx, dw, do):
        t.free()


@pytest.mark.parametrize("case", range(120))
def test_rope_on_random_views(case):
    """Head sizes on both kernels' sides (D/2 a multiple of 16 or not), one row or many, any
    start position, x and out reached through different strided views.  Bar: one leaf spacing
    plus 2^-9 of the pair's norm against float64 (the CPU arithmetic differs from the device's
    in the last place of sine and cosine); at most twice that from the oracle; the rest of the
    output owner is what it was."""
    rng = view_cases.Stream(case, 606)
    dtype = DT_BF16 if case % 4 else DT_F32
    nlead = 1 + rng.below(3)                         # rope needs rank >= 3
    lead = tuple(1 + rng.below(4) for _ in range(nlead))
    rows = (1, 1, 5, 16, 17, 33, 40)[rng.below(7)]
    D = (2, 10, 32, 40, 64, 64, 96, 128, 160)[rng.below(9)]
    a = (0, 0, 1, 7, 500, 4000)[rng.below(6)]
    theta = (10000.0, 500000.0)[rng.below(2)]
    xo, xs = view_cases.viewed_operand(rng, lead, rows, D)
    oo, os_ = view_cases.viewed_operand(rng, lead, rows, D)
    x32 = datagen.normal_f32(int(np.prod(xo)), 0, 1, 0x1800 + case)
    enc = datagen.bf16_rne if dtype == DT_BF16 else (lambda v: v.view(np.uint32))
    dx = iomx.DeviceTensor(dtype, xo, fill=0x5A)
    hx = iomo.HostTensor(dtype, xo, fill=0x5A)
    dx.view().from_host(enc(x32).reshape(xo))
    hx.view().from_logical(enc(x32).reshape(xo))
    do, ho = pair(dtype, oo, 0x1900 + case)
    dxv, hxv = view_cases.apply(dx.view(), xs), view_cases.apply(hx.view(), xs)
    dov, hov = view_cases.apply(do.view(), os_), view_cases.apply(ho.view(), os_)
    rc = iomx.rope(dxv, dov, a, theta)
    assert rc == 0, (iomx.lib().iomx_error_string(rc), xo, xs, oo, os_, a)
    kernel = iomx.last_launch().kernel.decode()
    assert iomo.rope(hxv, hov, a, theta) == 0
    to64 = (lambda raw: datagen.bf16_to_f32(raw.reshape(-1)).astype(np.float64).reshape(raw.shape)) \
        if dtype == DT_BF16 else (lambda raw: raw.view(np.float32).astype(np.float64))
    x = to64(hxv.to_logical())
    got, want = to64(dov.to_host()), to64(hov.to_logical())
    half = D // 2
    c = np.arange(half)
    ang = (a + np.arange(rows))[:, None] * theta ** (-2.0 * c / D)[None, :]
    x1, x2 = x[..., :half], x[..., half:]
    ref = np.concatenate([x1 * np.cos(ang) - x2 * np.sin(ang), x2 * np.cos(ang) + x1 * np.sin(ang)], -1)
    norm = np.sqrt(x1 * x1 + x2 * x2)
    norm = np.concatenate([norm, norm], -1)
    fbits = 7 if dtype == DT_BF16 else 23
    spacing = np.ldexp(1.0, (np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** -126))) - fbits).astype(np.int64))
    # positions in the thousands lose bits of the angle in binary32: 2^-9 of the norm covers it
    bound = spacing + np.ldexp(norm, -9)
    assert (np.abs(got - ref) <= bound).all(), (kernel, xo, xs, oo, os_, a, D)
    assert (np.abs(got - want) <= 2 * bound).all(), (kernel, xo, xs, oo, os_, a, D)
    marker = iomo.HostTensor(dtype, oo, fill=0)
    mv = view_cases.apply(marker.view(), os_)
    mv.from_logical(np.full(mv.dims, 1, iomo.NP_OF[dtype]))
    untouched = marker.storage == 0
    assert np.array_equal(do.raw()[untouched], ho.storage[untouched]), kernel
    for t in (dx, do):
        t.free()


@pytest.mark.parametrize("case", range(120))
def test_attention_on_random_shapes(case):
    """Grouping, head size, new rows, prefix and cache capacity drawn at random: the decode
    kernel and its shares, the four work mappings of the tiled kernel and the row kernel
    (D > 128) each get ragged tiles, partial groups and rows that see one token or all.  Bar on
    every element: the float64 evaluation within the BF16-probability budget
    (test_gpu_sdpa.float64_attention); nothing outside the logical output is written."""
    import test_gpu_sdpa as ts
    rng = view_cases.Stream(case, 707)
    lead = ((), (2,), (1, 3), (3,))[rng.below(4)]
    grouping = (1, 2, 4, 8)[rng.below(4)]
    Hkv = 1 + rng.below(4 if grouping < 8 else 2)
    R = (1, 1, 2, 5, 16, 17, 33, 64, 70, 130)[rng.below(10)]
    D = (16, 32, 48, 64, 64, 80, 96, 128, 128, 160)[rng.below(10)]
    a = (0, 0, 3, 31, 32, 100, 500, 2100)[rng.below(8 if R <= 2 else 7)]
    L = a + R - (rng.below(R) if rng.chance(1, 4) else 0)          # some rows see a truncated prefix
    C = a + R + rng.below(40)                                       # the new rows fit the cache
    spec = ts.random_case(0x2000 + case, lead, Hkv * grouping, Hkv, R, D, C, a, L)
    got = ts.run(spec, 0, fill=0xFF)
    ref64, budget = ts.float64_attention(spec)
    g = datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    worst = np.abs(g - ref64) - budget
    assert np.all(worst <= 0), (iomx.last_launch().kernel, lead, Hkv, grouping, R, D, C, a, L, float(worst.max()))


@pytest.mark.parametrize("case", range(100))
def test_cache_append_on_random_views(case):
    """R new rows written at position a of a cache of capacity C, any leaf, source and cache
    reached through different strided views: the whole cache owner equals the oracle's bit for
    bit (the rows before a, after a + R, the tile padding and the planes outside the view keep
    their pre-filled bits)."""
    rng = view_cases.Stream(case, 808)
    dtype = (DT_BF16, DT_F32, DT_I8, DT_U4, DT_F16, DT_F6_E2M3, DT_I64, iomo.DT_BOOL)[case % 8]
    nlead = 1 + rng.below(3)
    lead = tuple(1 + rng.below(4) for _ in range(nlead))
    R = (1, 1, 3, 16, 17, 40)[rng.below(6)]
    D = (2, 16, 24, 64, 128)[rng.below(5)]
    a = (0, 1, 15, 16, 37)[rng.below(5)]
    capacity = a + R + rng.below(20)
    so, ss = view_cases.viewed_operand(rng, lead, R, D)
    co, cs = view_cases.viewed_operand(rng, lead, capacity, D)
    ds, hs = pair(dtype, so, 0x2100 + case)
    dc, hc = pair(dtype, co, 0x2200 + case)
    rc = iomx.cache_append(view_cases.apply(ds.view(), ss), view_cases.apply(dc.view(), cs), a)
    assert rc == 0, (iomx.lib().iomx_error_string(rc), so, ss, co, cs, a)
    assert iomo.cache_append(view_cases.apply(hs.view(), ss), view_cases.apply(hc.view(), cs), a) == 0
    assert same_storage(dc, hc), (LEAF_NAME[dtype], so, ss, co, cs, a, R, D)
    assert same_storage(ds, hs)
    ds.free()
    dc.free()


@pytest.mark.parametrize("case", range(100))
def test_embedding_on_random_views(case):
    """Rows of a [V,F] table gathered by ids of any integer leaf into [..., R, F]: ids and output
    reached through strided views, table possibly one plane of a larger owner; payloads of any
    leaf.  The whole output owner equals the oracle's and the status word stays clear."""
    rng = view_cases.Stream(case, 909)
    dtype = (DT_BF16, DT_F32, DT_I8, DT_U4, DT_F16, DT_F6_E2M3, DT_I64, iomo.DT_F8_E8M0)[case % 8]
    index_dtype = (DT_I32, iomo.DT_U8, iomo.DT_I16, iomo.DT_U64, iomo.DT_U32, iomo.DT_I64)[rng.below(6)]
    nlead = rng.below(3)
    lead = tuple(1 + rng.below(4) for _ in range(nlead))
    R = (1, 2, 9, 16, 21)[rng.below(5)]
    F = (1, 16, 33, 40, 128, 300)[rng.below(6)]
    V = (1, 7, 37, 100)[rng.below(4)]
    io, isteps = view_cases.viewed_operand(rng, lead, 1, R)
    oo, osteps = view_cases.viewed_operand(rng, lead, R, F)
    to, tsteps = view_cases.viewed_operand(rng, (), V, F)
    if rng.chance(1, 2):                              # the table as one plane of a rank-3 owner
        planes = 2 + rng.below(2)
        to, tsteps = (planes,) + to, [("select", (0, rng.below(planes)))] + tsteps
    dt, ht = pair(dtype, to, 0x2300 + case)
    ids = (datagen.pattern_bits(32, int(np.prod(io)), 0x2400 + case) % V).astype(iomo.NP_OF[index_dtype]).reshape(io)
    di = iomx.DeviceTensor(index_dtype, io, fill=0x5A)
    hi = iomo.HostTensor(index_dtype, io, fill=0x5A)
    di.view().from_host(ids)
    hi.view().from_logical(ids)
    do, ho = pair(dtype, oo, 0x2500 + case)
    status = iomx.Buffer(32)
    status.fill(0xFF)
    iomx.synchronize()
    rc = iomx.embedding(view_cases.apply(dt.view(), tsteps), view_cases.apply(di.view(), isteps),
                        view_cases.apply(do.view(), osteps), status)
    assert rc == 0, (iomx.lib().iomx_error_string(rc), to, tsteps, io, isteps, oo, osteps)
    iomx.synchronize()
    assert int(status.download(np.uint32)[0]) == 0
    assert iomo.embedding(view_cases.apply(ht.view(), tsteps), view_cases.apply(hi.view(), isteps),
                          view_cases.apply(ho.view(), osteps)) == 0
    assert same_storage(do, ho), (LEAF_NAME[dtype], LEAF_NAME[index_dtype], to, tsteps, io, isteps, oo, osteps)
    status.free()
    for t in (dt, di, do):
        t.free()


@pytest.fixture(scope="module")
def devices():
    if not iomo.mi355x_available():
        pytest.skip("oracle/_ref/libiom_mi355x_shim.so not built (needs the reference headers)")
    gpu = iomo.mi355x_backend(arena_bytes=1 << 28, max_in_flight=4)
    cpu = iomo.cpu_backend_beside_mi355x()
    yield cpu, gpu
    gpu.close()
    cpu.close()


@pytest.mark.parametrize("case", range(200))
def test_backend_binary_and_copy_on_random_views(devices, case):
    """The same random views through `DeviceOps` on make_rocm_device and on the reference CPU
    backend in one process: what the backend makes of a TensorView's snapshot (plane offset,
    physical and result-aligned strides, broadcast flags) must lead to the bits the reference
    computes.  Binary operations over every numeric leaf except F64 (whose CPU carrier rounds
    twice) and, every fourth case, a copy."""
    cpu, gpu = devices
    leaves = [d for d in iomo.NUMERIC_LEAVES if d != DT_F64]
    dtype = leaves[case % len(leaves)]
    op = (OP_ADD, OP_MUL, OP_SUB, OP_DIV)[(case // len(leaves)) % 4]
    if op == OP_DIV and dtype not in FLOAT_LEAVES:
        op = OP_MUL
    if case % 4 == 3:
        lead, rows, cols, operands = view_cases.unary_case(case)
    else:
        lead, rows, cols, operands = view_cases.binary_case(case)
    tensors = []
    for i, (dims, _) in enumerate(operands):
        values = datagen.pattern_bits(LEAF_BITS[dtype], int(np.prod(dims)), 0x2600 + 3 * case + i).reshape(dims)
        pairs = []
        for dev in (cpu, gpu):
            t = dev.tensor(dtype, dims)
            t.view().from_host(values)
            pairs.append(t)
        tensors.append(pairs)
    cv = [view_cases.apply(t[0].view(), steps) for t, (_, steps) in zip(tensors, operands)]
    gv = [view_cases.apply(t[1].view(), steps) for t, (_, steps) in zip(tensors, operands)]
    if case % 4 == 3:
        tc, tg = cpu.copy(cv[0], cv[1]), gpu.copy(gv[0], gv[1])
    else:
        tc, tg = cpu.binary(op, cv[0], cv[1], cv[2]), gpu.binary(op, gv[0], gv[1], gv[2])
    assert tc > 0 and tg > 0, (tc, tg, gpu.error(), LEAF_NAME[dtype], operands)
    out = tensors[-1]
    # the whole output owner, read back through each backend's own host transfer
    assert np.array_equal(out[0].view().to_host(), out[1].view().to_host()), \
        (LEAF_NAME[dtype], op, lead, rows, cols, operands)
    for pairs in tensors:
        for t in pairs:
            t.close()


GRID_LIMIT_CASES = [
    # (leaf, lhs owner, lhs steps, rhs owner, rhs steps, out owner, out steps): each has more planes,
    # bands or (plane, band) pairs than the 65535 a grid axis holds, so the kernels' own loops run
    ("BANDS", DT_BF16, (16 * 70000, 16), [], (1, 16), [], (16 * 70000, 16), []),
    ("AXIS1", DT_BF16, (140000, 16, 16), [("slice", (0, 1, 70000, 2))], (70000, 16, 16), [], (70000, 16, 16), []),
    ("AXIS2B", DT_BF16, (2, 1400, 1600, 16), [("slice", (1, 0, 700, 2))], (1, 16), [], (2, 700, 1600, 16), []),
    ("PLANES", DT_F32, (50, 80, 42, 16, 16), [("slice", (1, 0, 40, 2)), ("slice", (2, 1, 40, 1))], (40, 1, 16, 16), [],
     (50, 40, 40, 16, 16), []),
    ("padded", DT_I32, (70000, 17, 16), [], (17, 1), [], (70000, 17, 16), []),
    ("rows", DT_U4, (70000, 16, 16), [], (1, 16), [], (70000, 16, 16), []),
    ("general", DT_F16, (1, 16), [], (70000, 16, 1), [], (70000, 16, 16), []),
]


@pytest.mark.parametrize("case", range(len(GRID_LIMIT_CASES)), ids=[c[0] for c in GRID_LIMIT_CASES])
def test_more_planes_or_bands_than_a_grid_axis_holds(case):
    _, dtype, ld, ls, rd, rs, od, os_ = GRID_LIMIT_CASES[case]
    dl, hl = pair(dtype, ld, 0x2700 + case)
    dr, hr = pair(dtype, rd, 0x2800 + case)
    do, ho = pair(dtype, od, 0x2900 + case)
    rc = iomx.binary(OP_ADD, view_cases.apply(dl.view(), ls), view_cases.apply(dr.view(), rs),
                     view_cases.apply(do.view(), os_))
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    kernel = iomx.last_launch().kernel.decode()
    assert iomo.binary(OP_ADD, view_cases.apply(hl.view(), ls), view_cases.apply(hr.view(), rs),
                       view_cases.apply(ho.view(), os_), ieee=True) == 0
    assert same_storage(do, ho), kernel
    # and a copy of the same output window back over the left operand's window where shapes agree
    if tuple(view_cases.apply(hl.view(), ls).dims) == tuple(view_cases.apply(ho.view(), os_).dims):
        assert iomx.copy(view_cases.apply(do.view(), os_), view_cases.apply(dl.view(), ls)) == 0
        assert iomo.copy(view_cases.apply(ho.view(), os_), view_cases.apply(hl.view(), ls)) == 0
        assert same_storage(dl, hl), iomx.last_launch().kernel.decode()
    for t in (dl, dr, do):
        t.free()


def test_row_kernels_with_more_bands_or_planes_than_a_grid_axis_holds():
    """RMSNorm and SiLU over 70000 bands of one plane and over 70000 planes of one band, RoPE
    over 70000 planes: every grid these launches use has an axis that stops at 65535."""
    for dims in ((16 * 70000, 32), (70000, 16, 32)):
        n = int(np.prod(dims))
        x = datagen.bf16_rne(datagen.normal_f32(n, 0, 1, 0x2A00)).reshape(dims)
        w = datagen.bf16_rne(datagen.uniform_f32(32, 0.5, 1.5, 0x2A01)).reshape(1, 32)
        dx = iomx.DeviceTensor(DT_BF16, dims)
        hx = iomo.HostTensor(DT_BF16, dims)
        dx.view().from_host(x)
        hx.view().from_logical(x)
        dw = iomx.DeviceTensor(DT_BF16, (1, 32))
        hw = iomo.HostTensor(DT_BF16, (1, 32))
        dw.view().from_host(w)
        hw.view().from_logical(w)
        do, ho = pair(DT_BF16, dims, 0x2A02)
        assert iomx.rmsnorm(dx.view(), dw.view(), do.view(), 1e-5) == 0
        assert iomo.rmsnorm(hx.view(), hw.view(), ho.view(), 1e-5) == 0
        assert np.abs(do.raw().astype(np.int64) - ho.storage.astype(np.int64)).max() <= 1
        assert iomx.silu(dx.view(), do.view()) == 0
        assert iomo.silu(hx.view(), ho.view()) == 0
        assert np.abs(do.raw().astype(np.int64) - ho.storage.astype(np.int64)).max() <= 1
        if len(dims) == 3:
            assert iomx.rope(dx.view(), do.view(), 3, 10000.0) == 0
            assert iomo.rope(hx.view(), ho.view(), 3, 10000.0) == 0
            got = datagen.bf16_to_f32(do.raw()).astype(np.float64)
            want = datagen.bf16_to_f32(ho.storage).astype(np.float64)
            assert np.all(np.abs(got - want) <= 2.0 ** -6 * np.maximum(np.abs(want), 1.0))
            assert float((do.raw() == ho.storage).mean()) > 0.9
        for t in (dx, dw, do):
            t.free()


@pytest.mark.parametrize("case", range(120))
def test_host_transfer_on_random_views(case):
    """Logical row-major bytes written through a strided view land in the slots the oracle's
    layout rule names and nowhere else (every leaf, ragged tiles), and read back unchanged."""
    dtype = iomo.ALL_LEAVES[case % len(iomo.ALL_LEAVES)]
    lead, rows, cols, operands = view_cases.unary_case(case, salt=1010)
    dims, steps = operands[0]
    dt, ht = pair(dtype, dims, 0x2B00 + case)
    dv, hv = view_cases.apply(dt.view(), steps), view_cases.apply(ht.view(), steps)
    values = datagen.pattern_bits(LEAF_BITS[dtype], int(np.prod(hv.dims)), 0x2C00 + case).reshape(hv.dims)
    if dtype == iomo.DT_BOOL:
        values = values & 1
    dv.from_host(values)
    hv.from_logical(values)
    assert same_storage(dt, ht), (LEAF_NAME[dtype], dims, steps)
    assert np.array_equal(dv.to_host(), values)
    assert np.array_equal(dt.view().to_host(), ht.view().to_logical())
    dt.free()


@pytest.mark.parametrize("seed", range(6))
def test_backend_random_operation_sequences_keep_queue_order(devices, seed):
    """150 dependent operations on a pool of eight owners, submitted without waiting (four
    credits, so most are parked and started from the completion thread), every result feeding
    later ones through views: at the end all owners equal what the reference CPU backend holds
    after the same sequence.  Only bit-exact operations (ADD / MUL / SUB / DIV with exact-alias
    in-place forms, copy between disjoint windows)."""
    cpu, gpu = devices
    rng = view_cases.Stream(seed, 1111)
    dtype = (DT_F32, DT_BF16, DT_I32)[seed % 3]
    dims = (4, 17, 33)
    pool = []
    for i in range(8):
        values = datagen.pattern_bits(LEAF_BITS[dtype], int(np.prod(dims)), 0x2D00 + 8 * seed + i).reshape(dims)
        if dtype != DT_I32:
            # moderate magnitudes: long products stay finite for a while, then saturate alike
            enc = datagen.bf16_rne if dtype == DT_BF16 else (lambda v: v.view(np.uint32))
            values = enc(datagen.normal_f32(int(np.prod(dims)), 0, 1, 0x2E00 + 8 * seed + i)).reshape(dims)
        pair_ = []
        for dev in (cpu, gpu):
            t = dev.tensor(dtype, dims)
            t.view().from_host(values)
            pair_.append(t)
        pool.append(pair_)
    windows = [lambda v: v, lambda v: v.slice(0, 0, 2, 2), lambda v: v.slice(0, 1, 2, 2), lambda v: v.slice(0, 2, 2, 1)]
    tokens = []
    for step in range(150):
        kind = rng.below(5)
        out, a, b = rng.below(8), rng.below(8), rng.below(8)
        w = windows[rng.below(4)] if kind != 4 else windows[1 + rng.below(3)]
        for which, dev in enumerate((cpu, gpu)):
            ov = w(pool[out][which].view())
            if kind == 4:                                  # copy from another owner's window
                src = a if a != out else (out + 1) % 8
                tok = dev.l.iomc_copy(dev.queue, w(pool[src][which].view()).h, ov.h)
            else:
                op = (OP_ADD, OP_MUL, OP_SUB, OP_DIV if dtype != DT_I32 else OP_ADD)[kind]
                # an input that is the output owner must be the identical window (exact alias)
                tok = dev.l.iomc_binary(dev.queue, op, w(pool[a][which].view()).h, w(pool[b][which].view()).h, ov.h)
            assert tok > 0, (step, kind, tok, dev.error())
            if which == 1:
                tokens.append(tok)
            else:
                assert cpu.wait(tok) == 0
    for tok in tokens:
        assert gpu.wait(tok) == 0, gpu.error()
    assert gpu.snapshot()[1:] == (0, 0)
    for i, (c, g) in enumerate(pool):
        assert np.array_equal(c.view().to_host(), g.view().to_host()), (seed, i)
    for c, g in pool:
        c.close()
        g.close()


@pytest.mark.parametrize("case", range(100))
def test_softmax_stage_on_random_layouts(case):
    """The stage's two layouts drawn at random: row, head and plane strides with gaps, a plane
    offset, a column stride of 1 or 2, a probability region with more physical rows and columns
    than the logical extent, alignments that allow the row kernel or force the generic one.
    Both buffers are flat and pre-filled; the oracle runs on the same layouts, so the whole
    probability buffer is compared: written entries within one BF16 step (masked ones exactly
    +0), every other element untouched."""
    rng = view_cases.Stream(case, 1212)
    planes, heads = 1 + rng.below(3), 1 + rng.below(3)
    rows = (1, 4, 9, 17)[rng.below(4)]
    cols = (4, 5, 64, 250, 256, 300, 1024, 1100)[rng.below(8)]
    a = (0, 0, 3, 40)[rng.below(4)]
    L = min(cols, a + rows) if rng.chance(1, 2) else cols
    L = max(L, 1)

    def layout(phys_rows, phys_cols):
        l = iomx.StageLayout()
        l.column_stride = 2 if rng.chance(1, 6) else 1
        quantum = 4 if rng.chance(2, 3) else 1                       # multiples of 4 keep the row kernel
        l.row_stride = phys_cols * l.column_stride + quantum * rng.below(4)
        l.head_stride = phys_rows * l.row_stride + quantum * rng.below(5)
        l.plane_stride = heads * l.head_stride + quantum * rng.below(5)
        l.plane_offset = quantum * rng.below(6)
        l.rows, l.columns = phys_rows, phys_cols
        size = l.plane_offset + planes * l.plane_stride + 8
        return l, int(size)
    sl, s_size = layout(rows, cols)
    pl, p_size = layout(rows + rng.below(3), cols + (0, 0, 4, 7)[rng.below(4)])
    logical = datagen.normal_f32(planes * heads * rows * cols, 0, 3, 0x2F00 + case).reshape(planes, heads, rows, cols)
    flat = np.full(s_size, np.nan, np.float32)
    idx = (sl.plane_offset + np.arange(planes)[:, None, None, None] * sl.plane_stride
           + np.arange(heads)[None, :, None, None] * sl.head_stride
           + np.arange(rows)[None, None, :, None] * sl.row_stride
           + np.arange(cols)[None, None, None, :] * sl.column_stride)
    flat[idx] = logical
    want = np.full(p_size, 0xAAAA, np.uint16)
    d = iomo.SoftmaxDesc()
    d.planes, d.heads, d.rows, d.a, d.L, d.scale = planes, heads, rows, a, L, 0.125
    d.scores, d.p_bf16 = flat.ctypes.data, want.ctypes.data
    for name in ("plane_offset", "plane_stride", "head_stride", "row_stride", "column_stride", "rows", "columns"):
        setattr(d.scores_layout, name, getattr(sl, name))
        setattr(d.probability_layout, name, getattr(pl, name))
    assert iomo.lib().iomo_softmax(ctypes.byref(d)) == 0
    sb, pb = iomx.Buffer(flat.nbytes), iomx.Buffer(want.nbytes)
    sb.upload(flat)
    pb.upload(np.full(p_size, 0xAAAA, np.uint16))
    g = iomx.SoftmaxDesc()
    g.planes, g.heads, g.rows, g.a, g.L, g.scale = planes, heads, rows, a, L, 0.125
    g.scores, g.p_bf16 = sb.ptr.value, pb.ptr.value
    g.scores_layout, g.probability_layout = sl, pl
    rc = iomx.softmax(g)
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    iomx.synchronize()
    kernel = iomx.last_launch().kernel.decode()
    got = pb.download(np.uint16)
    untouched = want == 0xAAAA
    assert np.array_equal(got[untouched], want[untouched]), (kernel, planes, heads, rows, cols, a, L)
    assert np.array_equal(got == 0, want == 0), kernel
    step = np.abs(got[~untouched].astype(np.int64) - want[~untouched].astype(np.int64))
    assert step.max() <= 1, (kernel, planes, heads, rows, cols, a, L, int(step.max()))
    sb.free()
    pb.free()


@pytest.mark.parametrize("case", range(80))
def test_attention_through_random_views(case):
    """q, k, v and out each reached through their own select / strided slice / permute of the
    leading axes (the head axis included), pre-filled owners: the float64 budget on every
    element, and nothing of the output owner outside the window changes."""
    import test_gpu_sdpa as ts
    rng = view_cases.Stream(case, 1313)
    lead = ((), (2,), (2, 2), (3,))[rng.below(4)]
    grouping = (1, 2, 4)[rng.below(3)]
    Hkv = 1 + rng.below(3)
    Hq = Hkv * grouping
    R = (1, 3, 16, 20, 40)[rng.below(5)]
    D = (16, 32, 64, 128)[rng.below(4)]
    a = (0, 2, 31, 100)[rng.below(4)]
    L = a + R
    cap = L + rng.below(20)
    spec = ts.random_case(0x3000 + case, lead, Hq, Hkv, R, D, cap, a, L)
    qd, kd, od = ts.shapes(spec)
    owners, views = [], []
    for name, dims in (("q", qd), ("k", kd), ("v", kd), (None, od)):
        owner_dims, steps = view_cases.viewed_operand(rng, dims[:-2], dims[-2], dims[-1])
        t = iomx.DeviceTensor(DT_BF16, owner_dims, fill=0xFF)
        view = view_cases.apply(t.view(), steps)
        if name:
            view.from_host(np.array(spec[name], np.uint16).reshape(dims))
        owners.append((t, owner_dims, steps))
        views.append(view)
    out_owner, out_dims, out_steps = owners[3]
    before = out_owner.raw().copy()
    rc, nbytes, _ = iomx.sdpa_workspace(views[0], views[1], views[2], views[3], a, L)
    assert rc == 0
    ws = iomx.Buffer(nbytes) if nbytes else None
    rc = iomx.sdpa(views[0], views[1], views[2], views[3], a, L, ws)
    assert rc == 0, (iomx.lib().iomx_error_string(rc), [o[1:] for o in owners])
    iomx.synchronize()
    kernel = iomx.last_launch().kernel.decode()
    got = views[3].to_host()
    ref64, budget = ts.float64_attention(spec)
    g = datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(ref64.shape)
    assert np.all(np.abs(g - ref64) <= budget), (kernel, [o[1:] for o in owners])
    marker = iomo.HostTensor(DT_BF16, out_dims, fill=0)
    mv = view_cases.apply(marker.view(), out_steps)
    mv.from_logical(np.full(mv.dims, 1, np.uint16))
    untouched = marker.storage == 0
    assert np.array_equal(out_owner.raw()[untouched], before[untouched]), kernel
    for t, _, _ in owners:
        t.free()
    if ws:
        ws.free()


@pytest.mark.parametrize("case", range(105))
def test_linear_scalar_recurrence_on_random_shapes_and_views(case):
    """The contract's scalar recurrence (every numeric leaf; the path of everything that is not
    BF16) on random shapes, row windows and strided x and out views: bit for bit against the
    oracle over the whole output owner."""
    import test_gpu_linear as tl
    rng = view_cases.Stream(case, 1414)
    dtype = iomo.NUMERIC_LEAVES[case % len(iomo.NUMERIC_LEAVES)]
    nlead = rng.below(3)
    lead = tuple(1 + rng.below(3) for _ in range(nlead))
    R = (1, 3, 16, 17, 33)[rng.below(5)]
    s = rng.below(6)
    x_rows = s + R + rng.below(4)
    inner = (1, 3, 16, 40, 65)[rng.below(5)]
    D = (1, 5, 16, 17, 33)[rng.below(5)]
    H = 1 + rng.below(3)
    head_planar = rng.chance(1, 2)
    xo, xs = view_cases.viewed_operand(rng, lead, x_rows, inner)
    out_lead = lead + ((H,) if head_planar else ())
    oo, os_ = view_cases.viewed_operand(rng, out_lead, R, D if head_planar else H * D)
    dx, hx = tl.pair(dtype, xo, values=tl.small_values(dtype, int(np.prod(xo)), 0x3100 + case).reshape(xo))
    dw, hw = tl.pair(dtype, (H * D, inner), values=tl.small_values(dtype, H * D * inner, 0x3200 + case).reshape(H * D, inner))
    do, ho = tl.pair(dtype, oo, salt=0x3300 + case)
    args = (s, R, head_planar, H if head_planar else 1, D if head_planar else H * D)
    rc = iomx.linear(view_cases.apply(dx.view(), xs), dw.view(), view_cases.apply(do.view(), os_), *args,
                     path=0 if dtype == DT_BF16 and case % 2 else 1)
    assert rc == 0, (iomx.lib().iomx_error_string(rc), LEAF_NAME[dtype], xo, xs, oo, os_, args)
    kernel = iomx.last_launch().kernel.decode()
    assert iomo.linear(view_cases.apply(hx.view(), xs), hw.view(), view_cases.apply(ho.view(), os_), *args) == 0
    if kernel == "linear_rows":
        assert same_storage(do, ho), (LEAF_NAME[dtype], xo, xs, oo, os_, args)
    else:                                             # BF16 on the matrix cores: the owner outside the window
        marker = iomo.HostTensor(dtype, oo, fill=0)
        mv = view_cases.apply(marker.view(), os_)
        mv.from_logical(np.full(mv.dims, 1, np.uint16))
        untouched = marker.storage == 0
        assert np.array_equal(do.raw()[untouched], ho.storage[untouched]), kernel
        # (values on this path: test_linear_bf16_on_random_shapes_and_views, against float64)
    for t in (dx, dw, do):
        t.free()


@pytest.mark.parametrize("case", range(150))
def test_rejections_on_random_views(case):
    """A valid random binary request, then one thing wrong with it: the library refuses it with
    the class the reference's validation order gives (src/device_ops_binary.cpp:102-181: shape
    and broadcast and alias errors are invalid_argument = -1 and come before the leaf's
    Unsupported = -2), launches nothing and leaves every owner as it was."""
    rng = view_cases.Stream(case, 1717)
    dtype = (DT_F32, DT_BF16, DT_I32, DT_U4, DT_F16)[case % 5]
    lead, rows, cols, operands = view_cases.binary_case(case)
    owners = [pair(dtype, dims, 0x3400 + 3 * case + i) for i, (dims, _) in enumerate(operands)]
    dv = [view_cases.apply(d.view(), steps) for (d, _), (_, steps) in zip(owners, operands)]
    hv = [view_cases.apply(h.view(), steps) for (_, h), (_, steps) in zip(owners, operands)]
    kind = case % 6
    op, code, expect = OP_ADD, dtype, -1
    extra = []
    if kind == 0:                                     # output one row short or one plane long
        bad = list(operands[2][0])
        bad[-2 if rng.chance(1, 2) or len(bad) == 2 else 0] += 1
        t = pair(dtype, tuple(bad), 0x3500 + case)
        extra.append(t)
        dv[2], hv[2] = t[0].view(), t[1].view()
    elif kind == 1:                                   # an input that cannot broadcast
        bad = list(dv[0].dims)
        bad[-1] = cols + 2
        t = pair(dtype, tuple(bad), 0x3600 + case)
        extra.append(t)
        dv[0], hv[0] = t[0].view(), t[1].view()
    elif kind == 2:                                   # an input inside the output's owner, other window
        dims = (2,) + tuple(dv[2].dims)
        t = pair(dtype, dims, 0x3700 + case)
        extra.append(t)
        dv[2], hv[2] = t[0].view().select(0, 0), t[1].view().select(0, 0)
        if tuple(dv[0].dims) == tuple(dv[2].dims):
            dv[0], hv[0] = t[0].view().select(0, 1), t[1].view().select(0, 1)
        else:
            dv[1], hv[1] = dv[2], hv[2]               # a broadcasting input may not alias at all
            if tuple(dv[1].dims) == tuple(dv[2].dims) and tuple(dv[0].dims) == tuple(dv[2].dims):
                expect = 0
    elif kind == 3:                                   # a leaf without arithmetic
        code, expect = (iomo.DT_BOOL, iomo.DT_F8_E8M0)[rng.below(2)], -2
    elif kind == 4:                                   # integer division: refused after the shape checks
        op = OP_DIV
        expect = -2 if dtype in (DT_I32, DT_U4) else 0
    else:                                             # unknown operation
        op = 4 + rng.below(100)
    before = [d.raw().copy() for d, _ in owners + extra]
    if kind == 3:
        a, b, o = (v.cview() for v in dv)
        rc = iomx.lib().iomx_launch_binary(op, code, ctypes.byref(a), ctypes.byref(b), ctypes.byref(o), None)
    else:
        rc = iomx.binary(op, dv[0], dv[1], dv[2])
    if kind == 2 and expect == -1:
        # whether the request is an exact alias (allowed) depends on the drawn shapes: decide by rule
        same = [tuple(v.dims) == tuple(dv[2].dims) and v.owner is dv[2].owner and v.plane_offset == dv[2].plane_offset
                and tuple(v.plane_strides) == tuple(dv[2].plane_strides) for v in dv[:2]]
        shares = [v.owner is dv[2].owner for v in dv[:2]]
        expect = -1 if any(s and not e for s, e in zip(shares, same)) else 0
    assert rc == expect, (kind, rc, expect, LEAF_NAME[dtype], operands)
    if expect != 0:
        iomx.synchronize()
        for (d, _), image in zip(owners + extra, before):
            assert np.array_equal(d.raw(), image)
    for d, _ in owners + extra:
        d.free()


def on_both(devices, dtype, dims, values):
    out = []
    for dev in devices:
        t = dev.tensor(dtype, dims)
        t.view().from_host(values)
        out.append(t)
    return out


def prefilled(devices, dtype, dims, salt):
    values = datagen.pattern_bits(LEAF_BITS[dtype], int(np.prod(dims)), salt).reshape(dims)
    if dtype == iomo.DT_BOOL:
        values = values & 1
    return on_both(devices, dtype, dims, values)


def bf16_steps(a, b):
    return np.abs(a.astype(np.int64) - b.astype(np.int64))


@pytest.mark.parametrize("case", range(120))
def test_backend_layer_operations_on_random_views(devices, case):
    """RMSNorm, SiLU, RoPE, cache append, embedding and the linear projection through `DeviceOps`
    on make_rocm_device and on the reference CPU backend, operands reached through random views:
    every hook turns its own kind of request snapshot into kernel arguments, and each must lead
    to what the reference computes (data movement bit for bit; RMSNorm and SiLU within one BF16
    step; RoPE within two; linear within the contract's bound of either result)."""
    cpu, gpu = devices
    rng = view_cases.Stream(case, 1818)
    kind = case % 6
    nlead = 1 + rng.below(2)
    lead = tuple(1 + rng.below(3) for _ in range(nlead))
    R = (1, 3, 16, 17, 33)[rng.below(5)]
    D = (16, 32, 64, 128)[rng.below(4)]
    dt = DT_BF16
    x32 = lambda n, s: datagen.bf16_rne(datagen.normal_f32(n, 0, 1, s))
    closing = []

    def make(dims, values=None, salt=None):
        pair_ = on_both(devices, dt, dims, values) if values is not None else prefilled(devices, dt, dims, salt)
        closing.extend(pair_)
        return pair_
    if kind in (0, 1, 2):                                   # rmsnorm / silu / rope: x -> out, same shape
        xo, xs = view_cases.viewed_operand(rng, lead, R, D)
        oo, os_ = view_cases.viewed_operand(rng, lead, R, D)
        x = make(xo, x32(int(np.prod(xo)), 0x3800 + case).reshape(xo))
        o = make(oo, salt=0x3900 + case)
        xv = [view_cases.apply(t.view(), xs) for t in x]
        ov = [view_cases.apply(t.view(), os_) for t in o]
        if kind == 0:
            w = make((1, D), x32(D, 0x3A00 + case).reshape(1, D))
            tokens = [dev.rmsnorm(xv[i], w[i].view(), ov[i], 1e-5) for i, dev in enumerate(devices)]
            bar = 1
        elif kind == 1:
            tokens = [dev.silu(xv[i], ov[i]) for i, dev in enumerate(devices)]
            bar = 1
        else:
            a = (0, 5, 300)[rng.below(3)]
            tokens = [dev.rope(xv[i], ov[i], a, 10000.0) for i, dev in enumerate(devices)]
            bar = 2
        assert all(t > 0 for t in tokens), (tokens, gpu.error())
        c, g = o[0].view().to_host(), o[1].view().to_host()
        assert bf16_steps(c, g).max() <= bar, (kind, xo, xs, oo, os_)
    elif kind == 3:                                         # cache append
        a = (0, 1, 16, 37)[rng.below(4)]
        cap = a + R + rng.below(10)
        so, ss = view_cases.viewed_operand(rng, lead, R, D)
        co, cs = view_cases.viewed_operand(rng, lead, cap, D)
        s_, c_ = make(so, salt=0x3B00 + case), make(co, salt=0x3C00 + case)
        tokens = [dev.cache_append(view_cases.apply(s_[i].view(), ss), view_cases.apply(c_[i].view(), cs), a)
                  for i, dev in enumerate(devices)]
        assert all(t > 0 for t in tokens), (tokens, gpu.error())
        assert np.array_equal(c_[0].view().to_host(), c_[1].view().to_host()), (so, ss, co, cs, a)
    elif kind == 4:                                         # embedding
        V, F = (7, 37, 100)[rng.below(3)], (16, 33, 128)[rng.below(3)]
        io, isteps = view_cases.viewed_operand(rng, lead, 1, R)
        oo, os_ = view_cases.viewed_operand(rng, lead, R, F)
        table = make((V, F), salt=0x3D00 + case)
        ids = (datagen.pattern_bits(32, int(np.prod(io)), 0x3E00 + case) % V).astype(np.uint32).reshape(io)
        idx = on_both(devices, iomo.DT_U32, io, ids)
        closing.extend(idx)
        o = make(oo, salt=0x3F00 + case)
        for i, dev in enumerate(devices):
            token, status = dev.embedding(table[i].view(), view_cases.apply(idx[i].view(), isteps),
                                          view_cases.apply(o[i].view(), os_))
            assert token > 0 and status == 0, (token, status, dev.error())
        assert np.array_equal(o[0].view().to_host(), o[1].view().to_host()), (io, isteps, oo, os_)
    else:                                                   # linear, ordinary or head-planar
        s = rng.below(5)
        x_rows = s + R + rng.below(3)
        inner = (32, 64, 96)[rng.below(3)]
        H = 1 + rng.below(3)
        hp = rng.chance(1, 2)
        xo, xs = view_cases.viewed_operand(rng, lead, x_rows, inner)
        oo, os_ = view_cases.viewed_operand(rng, lead + ((H,) if hp else ()), R, D if hp else H * D)
        x = make(xo, bf16_values(int(np.prod(xo)), 0x4000 + case).reshape(xo))
        w = make((H * D, inner), bf16_values(H * D * inner, 0x4100 + case).reshape(H * D, inner))
        o = make(oo, salt=0x4200 + case)
        args = (s, R, hp, H if hp else 1, D if hp else H * D)
        tokens = [dev.linear(view_cases.apply(x[i].view(), xs), w[i].view(), view_cases.apply(o[i].view(), os_), *args)
                  for i, dev in enumerate(devices)]
        assert all(t > 0 for t in tokens), (tokens, gpu.error())
        cv, gv = (view_cases.apply(o[i].view(), os_).to_host() for i in range(2))
        c64 = datagen.bf16_to_f32(cv.reshape(-1)).astype(np.float64)
        g64 = datagen.bf16_to_f32(gv.reshape(-1)).astype(np.float64)
        ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(c64), 1e-30))) - 7)
        assert np.all(np.abs(g64 - c64) <= 2 * np.maximum(np.maximum(ulp, 2.0 ** -7), 2.0 ** -6 * np.abs(c64)))
        # outside the window both owners still hold the pre-filled pattern
        marker = iomo.HostTensor(dt, oo, fill=0)
        mv = view_cases.apply(marker.view(), os_)
        mv.from_logical(np.full(mv.dims, 1, np.uint16))
        outside = iomo.untile_plane(marker.storage, oo) == 0
        assert np.array_equal(o[0].view().to_host()[outside], o[1].view().to_host()[outside])
    for t in closing:
        t.close()


@pytest.mark.parametrize("case", range(48))
def test_backend_attention_on_random_views(devices, case):
    """Attention through `DeviceOps` on both backends with q, k, v and out behind random views:
    both results inside the float64 budget of the BF16 probability, hence within twice the
    budget of each other (the reference's own fixture rule is no bound under cancellation)."""
    import test_gpu_sdpa as ts
    cpu, gpu = devices
    rng = view_cases.Stream(case, 1919)
    lead = ((), (2,), (2, 2))[rng.below(3)]
    grouping = (1, 2, 4)[rng.below(3)]
    Hkv = 1 + rng.below(2)
    Hq = Hkv * grouping
    R = (1, 3, 17, 40)[rng.below(4)]
    D = (16, 64, 128)[rng.below(3)]
    a = (0, 2, 31, 90)[rng.below(4)]
    L = a + R
    cap = L + rng.below(12)
    spec = ts.random_case(0x4300 + case, lead, Hq, Hkv, R, D, cap, a, L)
    qd, kd, od = ts.shapes(spec)
    tensors, views = [], []
    for name, dims in (("q", qd), ("k", kd), ("v", kd), (None, od)):
        owner_dims, steps = view_cases.viewed_operand(rng, dims[:-2], dims[-2], dims[-1])
        pair_ = prefilled(devices, DT_BF16, owner_dims, 0x4400 + 4 * case + len(tensors))
        vs = [view_cases.apply(t.view(), steps) for t in pair_]
        if name:
            for v in vs:
                v.from_host(np.array(spec[name], np.uint16).reshape(dims))
        tensors.append(pair_)
        views.append(vs)
    for i, dev in enumerate(devices):
        tok = dev.sdpa(views[0][i], views[1][i], views[2][i], views[3][i], a, L)
        assert tok > 0, (tok, dev.error())
    ref64, budget = ts.float64_attention(spec)
    results = []
    for i in range(2):
        got = views[3][i].to_host()
        results.append(datagen.bf16_to_f32(got.reshape(-1)).astype(np.float64).reshape(ref64.shape))
        assert np.all(np.abs(results[i] - ref64) <= budget), ("cpu", "gpu")[i]
    assert np.all(np.abs(results[0] - results[1]) <= 2 * budget)
    for pair_ in tensors:
        for t in pair_:
            t.close()


def test_four_queues_driven_from_four_threads(devices):
    """Four host threads, each with a queue of its own on the one device, run 120 dependent
    operations on their own owners while creating and closing scratch tensors and reading results
    back (arena, registry and transfer path are shared by all of them).  Every thread's owners
    end up as the reference CPU backend leaves them after the same sequence."""
    import threading
    cpu, gpu = devices
    dims = (3, 17, 33)
    count = int(np.prod(dims))
    plans, pools, queues, errors = [], [], [], []
    for th in range(4):
        rng = view_cases.Stream(th, 2020)
        plans.append([(rng.below(4), rng.below(4), rng.below(4), rng.below(3), rng.below(7)) for _ in range(120)])
        values = [datagen.normal_f32(count, 0, 1, 0x4500 + 4 * th + i).view(np.uint32).reshape(dims) for i in range(4)]
        pools.append(([on_both((cpu,), DT_F32, dims, v)[0] for v in values],
                      [on_both((gpu,), DT_F32, dims, v)[0] for v in values]))
        queues.append(gpu if th == 0 else gpu.second_queue())

    def drive(th):
        try:
            q = queues[th]
            pool = pools[th][1]
            tokens = []
            for out, a, b, op, extra in plans[th]:
                tok = q.l.iomc_binary(q.queue, (OP_ADD, OP_MUL, OP_SUB)[op], pool[a].view().h, pool[b].view().h,
                                      pool[out].view().h)
                assert tok > 0, (th, tok, q.error())
                tokens.append(tok)
                if extra == 0:                          # a scratch owner comes and goes
                    t = gpu.tensor(DT_F32, (2, 16, 16))
                    t.view().from_host(np.zeros((2, 16, 16), np.uint32))
                    t.close()
                elif extra == 1:                        # observe an earlier result mid-stream
                    assert q.wait(tokens[len(tokens) // 2]) == 0
                    pool[a].view().to_host()
            for tok in tokens:
                assert q.wait(tok) == 0, q.error()
        except BaseException as exc:                    # reported by the main thread
            errors.append((th, repr(exc)))
    threads = [threading.Thread(target=drive, args=(th,)) for th in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert errors == []
    for th in range(4):
        pool = pools[th][0]
        for out, a, b, op, _ in plans[th]:
            assert cpu.binary((OP_ADD, OP_MUL, OP_SUB)[op], pool[a].view(), pool[b].view(), pool[out].view()) > 0
        for c, g in zip(*pools[th]):
            assert np.array_equal(c.view().to_host(), g.view().to_host()), th
    for th in range(1, 4):
        queues[th].close()
    for th in range(4):
        for t in pools[th][0] + pools[th][1]:
            t.close()
