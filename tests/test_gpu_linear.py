"""GPU parity of the linear projection, through the C ABI against the CPU oracle (the
contract's scalar recurrence) and through the C++ backend next to the reference CPU backend.

Bars (docs/BACKEND_CONTRACT/linear-projections.md:334-341): integer leaves exact bits; the
scalar-recurrence path exact bits for every floating leaf too (same fused multiply-add order);
BF16 on the matrix cores |actual - q| <= max(ulp_bf16(q), 2^-7, 2^-6 |q|) against the float64
evaluation rounded once to BF16.
"""
import numpy as np
import pytest

import datagen
import iomo
from iom_amd import iomx
from iomo import DT_BF16, DT_F32, DT_F64, INTEGER_LEAVES, LEAF_BITS, LEAF_NAME, NUMERIC_LEAVES

pytestmark = pytest.mark.gpu
names = lambda ds: [LEAF_NAME[d] for d in ds]
FMT = {13: (2, 1, 1), 14: (2, 3, 1), 15: (3, 2, 3), 16: (4, 3, 7), 17: (5, 2, 15), 19: (5, 10, 15),
       20: (8, 7, 127), 21: (8, 23, 127), 22: (11, 52, 1023)}


@pytest.fixture(scope="module", autouse=True)
def _device():
    assert iomx.device_count() >= 1
    iomx.check(iomx.lib().iomx_set_device(0))
    yield


def small_values(dtype, count, salt):
    bits = LEAF_BITS[dtype]
    v = datagen.pattern_bits(bits, count, salt)
    if dtype in INTEGER_LEAVES or dtype in (13, 14, 15):
        return v
    ebits, fbits, bias = FMT[dtype]
    exp = (v.astype(np.uint64) >> np.uint64(fbits)) & np.uint64((1 << ebits) - 1)
    exp = exp % np.uint64(5) + np.uint64(bias - 3)
    cleared = v.astype(np.uint64) & ~np.uint64(((1 << ebits) - 1) << fbits)
    return (cleared | (exp << np.uint64(fbits))).astype(v.dtype)


def pair(dtype, dims, values=None, salt=None, fill=0x5A):
    dt = iomx.DeviceTensor(dtype, dims, fill=fill)
    ht = iomo.HostTensor(dtype, dims, fill=fill)
    if salt is not None:
        values = datagen.pattern_bits(LEAF_BITS[dtype], int(np.prod(dims)), salt).reshape(dims)
    if values is not None:
        dt.view().from_host(values)
        ht.view().from_logical(values)
    return dt, ht


def same_storage(dt, ht):
    return np.array_equal(dt.raw().view(np.uint8), ht.storage.view(np.uint8))


FIXTURES = [
    ((19, 3), (10, 3), 2, 17, False, 1, 10), ((19, 3), (10, 3), 2, 16, False, 1, 10),
    ((19, 3), (10, 3), 2, 15, True, 2, 5), ((19, 3), (10, 3), 2, 1, True, 2, 5),
    ((2, 3, 20, 65), (33, 65), 3, 17, False, 1, 33), ((2, 3, 20, 65), (34, 65), 0, 20, True, 2, 17),
    ((7, 48), (100, 48), 6, 1, False, 1, 100),
    ((2, 40, 128), (96, 128), 4, 36, True, 3, 32),
]


@pytest.mark.parametrize("dtype", NUMERIC_LEAVES, ids=names(NUMERIC_LEAVES))
@pytest.mark.parametrize("case", range(len(FIXTURES)))
def test_scalar_recurrence_is_bit_exact(dtype, case):
    xd, wd, s, R, hp, H, D = FIXTURES[case]
    dx, hx = pair(dtype, xd, values=small_values(dtype, int(np.prod(xd)), 1 + case).reshape(xd))
    dw, hw = pair(dtype, wd, values=small_values(dtype, int(np.prod(wd)), 11 + case).reshape(wd))
    od = xd[:-2] + ((H, R, D) if hp else (R, D))
    do, ho = pair(dtype, od, salt=21 + case)
    rc = iomx.linear(dx.view(), dw.view(), do.view(), s, R, hp, H, D, path=1)
    assert rc == 0, iomx.lib().iomx_error_string(rc)
    assert iomx.last_launch().kernel.decode() == "linear_rows"
    assert iomo.linear(hx.view(), hw.view(), ho.view(), s, R, hp, H, D) == 0
    assert same_storage(do, ho)                    # poisoned padding and untouched rows included
    for t in (dx, dw, do):
        t.free()


def bf16_bound(g_raw, x_raw, w_raw):
    x64 = datagen.bf16_to_f32(x_raw.reshape(-1)).astype(np.float64).reshape(x_raw.shape)
    w64 = datagen.bf16_to_f32(w_raw.reshape(-1)).astype(np.float64).reshape(w_raw.shape)
    ref = x64 @ w64.T
    q = datagen.bf16_to_f32(datagen.bf16_rne(ref.astype(np.float32).reshape(-1))).astype(np.float64).reshape(ref.shape)
    g = datagen.bf16_to_f32(g_raw.reshape(-1)).astype(np.float64).reshape(ref.shape)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(q), 1e-30))) - 7)
    return np.abs(g - q) <= np.maximum(np.maximum(ulp, 2.0 ** -7), 2.0 ** -6 * np.abs(q))


@pytest.mark.parametrize("path,kernel", [(0, "linear_mfma_splitk"), (2, "linear_mfma")], ids=["split_inner", "direct"])
@pytest.mark.parametrize("case", range(len(FIXTURES)))
def test_bf16_matrix_cores_on_the_fixtures(case, path, kernel):
    xd, wd, s, R, hp, H, D = FIXTURES[case]
    xv = small_values(DT_BF16, int(np.prod(xd)), 1 + case).reshape(xd)
    wv = small_values(DT_BF16, int(np.prod(wd)), 11 + case).reshape(wd)
    dx, hx = pair(DT_BF16, xd, values=xv)
    dw, hw = pair(DT_BF16, wd, values=wv)
    od = xd[:-2] + ((H, R, D) if hp else (R, D))
    do, ho = pair(DT_BF16, od, salt=21 + case)
    assert iomx.linear(dx.view(), dw.view(), do.view(), s, R, hp, H, D, path=path) == 0
    assert iomx.last_launch().kernel.decode() == kernel
    assert iomo.linear(hx.view(), hw.view(), ho.view(), s, R, hp, H, D) == 0
    got = do.view().to_host()
    lead = int(np.prod(xd[:-2])) if len(xd) > 2 else 1
    x3 = xv.reshape(lead, xd[-2], xd[-1])[:, s:s + R, :]
    g3 = got.reshape(lead, H, R, D).transpose(0, 2, 1, 3).reshape(lead, R, H * D) if hp else got.reshape(lead, R, H * D)
    for b in range(lead):
        assert bf16_bound(g3[b], x3[b], wv).all()
    # everything the operation does not own is untouched: compare storage outside the logical window
    mask = iomo.tile_plane(np.ones(od, np.uint16)) == 0
    assert np.array_equal(do.raw()[mask], ho.storage[mask])
    want = ho.view().to_logical()
    d = np.abs(got.astype(np.int64) - want.astype(np.int64))
    print("case", case, "differs from the scalar recurrence in", int((d > 0).sum()), "of", d.size, flush=True)
    for t in (dx, dw, do):
        t.free()


def test_bf16_matrix_cores_layer_shapes_and_views():
    """[4,64,2048] x [2048+,2048]: prefill rows, decode row, GQA head-planar K projection, views."""
    I = 2048
    xv = datagen.bf16_rne(datagen.normal_f32(4 * 64 * I, 0, 1, 3)).reshape(4, 64, I)
    wv = datagen.bf16_rne(datagen.normal_f32(5632 * I, 0, 0.02, 4)).reshape(5632, I)
    dx = iomx.DeviceTensor(DT_BF16, (4, 64, I)); dx.view().from_host(xv)
    dw = iomx.DeviceTensor(DT_BF16, (5632, I)); dw.view().from_host(wv)
    # ordinary, all rows
    do = iomx.DeviceTensor(DT_BF16, (4, 64, 5632))
    assert iomx.linear(dx.view(), dw.view(), do.view(), 0, 64, False, 1, 5632) == 0
    got = do.view().to_host()
    for b in (0, 3):
        assert bf16_bound(got[b], xv[b], wv).all()
    # the last row only (logits-like), every second plane of x
    d1 = iomx.DeviceTensor(DT_BF16, (2, 1, 5632))
    assert iomx.linear(dx.view().slice(0, 1, 2, 2), dw.view(), d1.view(), 63, 1, False, 1, 5632) == 0
    g1 = d1.view().to_host()
    assert bf16_bound(g1[0], xv[1, 63:64], wv).all() and bf16_bound(g1[1], xv[3, 63:64], wv).all()
    # head planar: 4 KV heads of 64 from the first 256 weight rows (a [256, I] owner)
    dk = iomx.DeviceTensor(DT_BF16, (256, I)); dk.view().from_host(wv[:256])
    dh = iomx.DeviceTensor(DT_BF16, (4, 4, 17, 64))
    assert iomx.linear(dx.view(), dk.view(), dh.view(), 40, 17, True, 4, 64) == 0
    gh = dh.view().to_host()
    for b in (0, 2):
        flat = gh[b].transpose(1, 0, 2).reshape(17, 256)
        assert bf16_bound(flat, xv[b, 40:57], wv[:256]).all()
    # the scalar path on a slice of the same problem agrees within the same bound
    ds = iomx.DeviceTensor(DT_BF16, (4, 4, 17, 64))
    assert iomx.linear(dx.view(), dk.view(), ds.view(), 40, 17, True, 4, 64, path=1) == 0
    d = np.abs(ds.view().to_host().astype(np.int64) - gh.astype(np.int64))
    assert d.max() <= 2
    for t in (dx, dw, do, d1, dk, dh, ds):
        t.free()


def test_linear_rejections():
    dx, _ = pair(DT_F32, (19, 3), salt=1)
    dw, _ = pair(DT_F32, (10, 3), salt=2)
    do, _ = pair(DT_F32, (17, 10))
    dh, _ = pair(DT_F32, (2, 17, 5))
    for args in ((2, 18, False, 1, 10), (20, 1, False, 1, 10), (2, 0, False, 1, 10), (2, 17, False, 2, 5),
                 (2, 17, False, 1, 9)):
        assert iomx.linear(dx.view(), dw.view(), do.view(), *args) == -1, args
    assert iomx.linear(dx.view(), dw.view(), dh.view(), 2, 17, True, 2, 6) == -1
    assert iomx.linear(dx.view(), dw.view(), dh.view(), 2, 17, True, 5, 2) == -1
    assert iomx.linear(dx.view(), dw.view(), dx.view(), 2, 17, False, 1, 10) == -1
    db, _ = pair(iomo.DT_BOOL, (19, 3))
    dbw, _ = pair(iomo.DT_BOOL, (10, 3))
    dbo, _ = pair(iomo.DT_BOOL, (17, 10))
    assert iomx.linear(db.view(), dbw.view(), dbo.view(), 2, 17, False, 1, 10) == -2
    for t in (dx, dw, do, dh, db, dbw, dbo):
        t.free()


# -- through the C++ backend -----------------------------------------------------------

@pytest.fixture(scope="module")
def devices():
    if not iomo.mi355x_available():
        pytest.skip("oracle/_ref/libiom_mi355x_shim.so not built (needs the reference headers)")
    gpu = iomo.mi355x_backend(arena_bytes=1 << 28, max_in_flight=4)
    cpu = iomo.cpu_backend_beside_mi355x()
    yield cpu, gpu
    gpu.close()
    cpu.close()


@pytest.mark.parametrize("dtype", [iomo.DT_I8, iomo.DT_U4, DT_F32, iomo.DT_F16, DT_F64, DT_BF16],
                         ids=["I8", "U4", "F32", "F16", "F64", "BF16"])
def test_backend_linear_next_to_the_reference_cpu_backend(devices, dtype):
    cpu, gpu = devices
    xd, wd, s, R, H, D = (2, 3, 20, 65), (34, 65), 2, 18, 2, 17
    xv = small_values(dtype, int(np.prod(xd)), 5).reshape(xd)
    wv = small_values(dtype, int(np.prod(wd)), 6).reshape(wd)
    outs = []
    for dev in (cpu, gpu):
        x = dev.tensor(dtype, xd); x.view().from_host(xv)
        w = dev.tensor(dtype, wd); w.view().from_host(wv)
        o = dev.tensor(dtype, (2, 3, H, R, D))
        assert dev.linear(x.view(), w.view(), o.view(), s, R, True, H, D) > 0, dev.error()
        outs.append(o.view().to_host())
        assert dev.linear(x.view(), w.view(), o.view(), s, 19, True, H, D) == -1
        for t in (x, w, o):
            t.close()
    if dtype == DT_BF16:          # matrix cores against the CPU recurrence: a few BF16 steps on sums of 65 terms
        a, b = (datagen.bf16_to_f32(v.reshape(-1)).astype(np.float64) for v in outs)
        assert (np.abs(a - b) <= np.maximum(2.0 ** -7, 2.0 ** -6 * np.abs(a))).all()
    else:
        assert np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("hp", [False, True], ids=["ordinary", "head_planar"])
@pytest.mark.parametrize("window", [(0, 200), (5, 190)], ids=["all_rows", "window"])
def test_bf16_matrix_cores_staged_through_lds(hp, window):
    """Many rows: the workgroup-tiled kernel.  Rows of different planes share row tiles
    (R is not a multiple of 16), the last workgroup column is mostly past O."""
    s, R = window
    xd, wd, H, D = (3, 200, 128), (272, 128), 17, 16
    xv = datagen.bf16_rne(datagen.normal_f32(int(np.prod(xd)), 0, 1, 31)).reshape(xd)
    wv = datagen.bf16_rne(datagen.normal_f32(int(np.prod(wd)), 0, 0.1, 32)).reshape(wd)
    dx, hx = pair(DT_BF16, xd, values=xv)
    dw, hw = pair(DT_BF16, wd, values=wv)
    od = (3, H, R, D) if hp else (3, R, H * D)
    do, ho = pair(DT_BF16, od, salt=33)
    args = (s, R, hp, H if hp else 1, D if hp else H * D)
    assert iomx.linear(dx.view(), dw.view(), do.view(), *args) == 0
    assert iomx.last_launch().kernel.decode() == "linear_mfma_lds"
    got = do.view().to_host()
    g3 = got.transpose(0, 2, 1, 3).reshape(3, R, H * D) if hp else got
    for b in range(3):
        assert bf16_bound(g3[b], xv[b, s:s + R], wv).all()
    mask = iomo.tile_plane(np.ones(od, np.uint16)) == 0
    assert np.array_equal(do.raw()[mask], ho.storage[mask])
    # the direct-from-global kernel adds the same products in the same order
    d2, _ = pair(DT_BF16, od, salt=33)
    assert iomx.linear(dx.view(), dw.view(), d2.view(), *args, path=2) == 0
    assert iomx.last_launch().kernel.decode() == "linear_mfma"
    assert np.array_equal(d2.raw(), do.raw())
    for t in (dx, dw, do, d2):
        t.free()


@pytest.mark.parametrize("path", [5, 4, 3], ids=["tile64", "tile128", "tile256"])
@pytest.mark.parametrize("inner", [32, 64, 96, 160, 288])
def test_bf16_workgroup_tiled_kernels_on_short_and_odd_inner_extents(inner, path):
    """One to nine 32-element stages (fewer than the ring holds, odd counts), both workgroup
    tile sizes; 300 rows over 2 planes with a window, 80 outputs in 5 heads."""
    xd, wd, s, R, H, D = (2, 160, inner), (80, inner), 7, 150, 5, 16
    xv = datagen.bf16_rne(datagen.normal_f32(int(np.prod(xd)), 0, 1, 51 + inner)).reshape(xd)
    wv = datagen.bf16_rne(datagen.normal_f32(int(np.prod(wd)), 0, 0.2, 52 + inner)).reshape(wd)
    dx, _ = pair(DT_BF16, xd, values=xv)
    dw, _ = pair(DT_BF16, wd, values=wv)
    od = (2, H, R, D)
    do, ho = pair(DT_BF16, od, salt=53)
    assert iomx.linear(dx.view(), dw.view(), do.view(), s, R, True, H, D, path=path) == 0
    assert iomx.last_launch().kernel.decode() == "linear_mfma_lds"
    got = do.view().to_host().transpose(0, 2, 1, 3).reshape(2, R, H * D)
    for b in range(2):
        assert bf16_bound(got[b], xv[b, s:s + R], wv).all()
    mask = iomo.tile_plane(np.ones(od, np.uint16)) == 0
    assert np.array_equal(do.raw()[mask], ho.storage[mask])
    d2, _ = pair(DT_BF16, od, salt=53)
    assert iomx.linear(dx.view(), dw.view(), d2.view(), s, R, True, H, D, path=2) == 0
    assert np.array_equal(d2.raw(), do.raw())          # same products in the same order
    for t in (dx, dw, do, d2):
        t.free()


@pytest.mark.parametrize("inner", [544, 1056, 2048, 4128])
def test_bf16_small_tiles_with_the_inner_axis_shared_by_groups_of_waves(inner):
    """Few 64 x 64 blocks and a long inner axis: two or four groups of waves each take a part
    of the stages (17, 33, 64 or 129 of them: parts of unequal length, a last part that is
    shorter) and their partial sums meet in LDS.  300 rows over 2 planes with a window, 80
    outputs in 5 heads; the contract's BF16 bound against float64, one-hot rows exactly, and
    untouched padding."""
    xd, wd, s, R, H, D = (2, 160, inner), (80, inner), 7, 150, 5, 16
    xv = datagen.bf16_rne(datagen.normal_f32(int(np.prod(xd)), 0, 1, 61 + inner)).reshape(xd)
    wv = datagen.bf16_rne(datagen.normal_f32(int(np.prod(wd)), 0, 0.2, 62 + inner)).reshape(wd)
    xv[1, s + 3, :] = 0
    xv[1, s + 3, inner - 1] = 0x3F80              # a one-hot row in the last stage of the last group
    xv[0, s + 149, :] = 0
    xv[0, s + 149, 0] = 0x3F80                    # ... and in the first stage of the first
    dx, _ = pair(DT_BF16, xd, values=xv)
    dw, _ = pair(DT_BF16, wd, values=wv)
    od = (2, H, R, D)
    do, ho = pair(DT_BF16, od, salt=63)
    assert iomx.linear(dx.view(), dw.view(), do.view(), s, R, True, H, D, path=0) == 0
    assert iomx.last_launch().kernel.decode() == "linear_mfma_lds"
    got = do.view().to_host().transpose(0, 2, 1, 3).reshape(2, R, H * D)
    for b in range(2):
        assert bf16_bound(got[b], xv[b, s:s + R], wv).all()
    assert np.array_equal(got[1, 3], wv[:, inner - 1]) and np.array_equal(got[0, 149], wv[:, 0])
    mask = iomo.tile_plane(np.ones(od, np.uint16)) == 0
    assert np.array_equal(do.raw()[mask], ho.storage[mask])
    for t in (dx, dw, do):
        t.free()


@pytest.mark.parametrize("inner", [128, 192, 448, 2048])
def test_bf16_tiles_of_128_with_the_inner_axis_in_two_halves(inner):
    """128 x 128 blocks whose two groups of waves each take half of the stages (2, 3, 7 and 32
    stages a group: fewer than the ring holds, odd counts) and add their partial sums in LDS.
    300 rows over 2 planes with a window, 80 outputs in 5 heads; the contract's BF16 bound
    against float64, one-hot rows at both ends of both halves exactly, untouched padding."""
    xd, wd, s, R, H, D = (2, 160, inner), (80, inner), 7, 150, 5, 16
    xv = datagen.bf16_rne(datagen.normal_f32(int(np.prod(xd)), 0, 1, 71 + inner)).reshape(xd)
    wv = datagen.bf16_rne(datagen.normal_f32(int(np.prod(wd)), 0, 0.2, 72 + inner)).reshape(wd)
    hot = {(1, 3): inner - 1, (0, 149): 0, (1, 77): inner // 2, (0, 20): inner // 2 - 1}
    for (b, r), i in hot.items():
        xv[b, s + r, :] = 0
        xv[b, s + r, i] = 0x3F80
    dx, _ = pair(DT_BF16, xd, values=xv)
    dw, _ = pair(DT_BF16, wd, values=wv)
    od = (2, H, R, D)
    do, ho = pair(DT_BF16, od, salt=73)
    assert iomx.linear(dx.view(), dw.view(), do.view(), s, R, True, H, D, path=6) == 0
    assert iomx.last_launch().kernel.decode() == "linear_mfma_lds"
    assert iomx.last_launch().block == 512
    got = do.view().to_host().transpose(0, 2, 1, 3).reshape(2, R, H * D)
    for b in range(2):
        assert bf16_bound(got[b], xv[b, s:s + R], wv).all()
    for (b, r), i in hot.items():
        assert np.array_equal(got[b, r], wv[:, i]), (b, r, i)
    mask = iomo.tile_plane(np.ones(od, np.uint16)) == 0
    assert np.array_equal(do.raw()[mask], ho.storage[mask])
    for t in (dx, dw, do):
        t.free()


def test_bf16_one_round_of_128_blocks_takes_the_two_halves():
    """512 rows x [5632,2048] is 176 blocks of 128 x 128: one workgroup on each of 176 CUs, so the
    launch picks the two-group form; sampled rows against float64, and the rows of a second
    plane with the same values give the same bits."""
    S, I, O = 512, 2048, 5632
    xv = datagen.bf16_rne(datagen.normal_f32(S * I, 0, 1, 81)).reshape(1, S, I)
    wv = datagen.bf16_rne(datagen.normal_f32(O * I, 0, 0.02, 82)).reshape(O, I)
    dx, _ = pair(DT_BF16, (1, S, I), values=xv)
    dw, _ = pair(DT_BF16, (O, I), values=wv)
    do, _ = pair(DT_BF16, (1, S, O), salt=83)
    assert iomx.linear(dx.view(), dw.view(), do.view(), 0, S, False, 1, O) == 0
    launch = iomx.last_launch()
    assert launch.kernel.decode() == "linear_mfma_lds" and launch.block == 512 and launch.grid == 176
    got = do.view().to_host()
    for r in (0, 17, 255, 256, 511):
        assert bf16_bound(got[0, r:r + 1], xv[0, r:r + 1], wv).all()
    d2, _ = pair(DT_BF16, (1, S, O), salt=84)
    assert iomx.linear(dx.view(), dw.view(), d2.view(), 0, S, False, 1, O, path=6) == 0
    assert np.array_equal(d2.raw(), do.raw())
    for t in (dx, dw, do, d2):
        t.free()


# (x dims, s, R, head planar, H, D, inner, workgroups expected): decode steps of 17-64
# sequences, where one workgroup takes two or four row tiles against two or four output
# tiles; ragged last row tile, ragged last output tile, ragged inner axis, rows of one plane
DECODE_TILES = [
    ((64, 1), 0, 1, False, 1, 4096, 200, 2 * 128),              # 2 x 2
    ((50, 1), 0, 1, False, 1, 5640, 96, 2 * 96),                # 2 x 4: 353 output tiles -> 89 blocks, padded to 96
    ((33, 1), 0, 1, True, 88, 64, 160, 2 * 88),                 # 2 x 4: three row tiles, head planar
    ((1, 70), 5, 60, False, 1, 5632, 72, 2 * 88),               # 2 x 4: rows of one plane
    ((20, 1), 0, 1, False, 1, 16384, 64, 256),                  # 2 x 4: two row tiles
    ((64, 1), 0, 1, False, 1, 10248, 3912, 168),                # 4 x 4: 641 output tiles -> 161 blocks, padded to 168
    # long inner axes: at most 256 workgroups walk it with two register sets of slices in
    # turn (several whole sets, then single slices, then the ragged end), more with one set
    ((64, 1), 0, 1, False, 1, 4096, 2080, 256),                 # 2 x 2, two sets of 4 slices
    ((64, 1), 0, 1, False, 1, 2048, 5648, 256),                 # 1 x 2, two sets of 8 slices, ragged end
    ((3, 1), 0, 1, False, 1, 2048, 1504, 128),                  # 1 x 1, two sets: an odd number of whole sets
    ((1, 1), 0, 1, False, 1, 5632, 2048, 352),                  # 1 x 1, one set of 8 slices
    # many row blocks of one row tile each next to one another in the workgroup sequence
    ((100, 1), 0, 1, False, 1, 2048, 96, 7 * 64),               # 1 x 2, seven row blocks
    ((130, 1), 0, 1, False, 1, 272, 40, 9 * 24),                # 1 x 1, nine row blocks, 17 output blocks padded to 24
]


@pytest.mark.parametrize("case", range(len(DECODE_TILES)))
def test_bf16_decode_steps_with_larger_workgroup_tiles(case):
    lead, s, R, hp, H, D, inner, workgroups = DECODE_TILES[case]
    xd, wd = lead + (inner,), (H * D, inner)
    xv = datagen.bf16_rne(datagen.normal_f32(int(np.prod(xd)), 0, 1, 61 + case)).reshape(xd)
    wv = datagen.bf16_rne(datagen.normal_f32(int(np.prod(wd)), 0, 0.05, 71 + case)).reshape(wd)
    dx, _ = pair(DT_BF16, xd, values=xv)
    dw, _ = pair(DT_BF16, wd, values=wv)
    od = xd[:-2] + ((H, R, D) if hp else (R, H * D))
    do, ho = pair(DT_BF16, od, salt=81 + case)
    assert iomx.linear(dx.view(), dw.view(), do.view(), s, R, hp, H, D) == 0
    ll = iomx.last_launch()
    assert ll.kernel.decode() == "linear_mfma_splitk" and ll.grid == workgroups
    got = do.view().to_host()
    g3 = got.reshape(xd[0], H, R, D).transpose(0, 2, 1, 3).reshape(xd[0], R, H * D) if hp else got
    for b in range(xd[0]):
        assert bf16_bound(g3[b], xv[b, s:s + R], wv).all(), b
    mask = iomo.tile_plane(np.ones(od, np.uint16)) == 0
    assert np.array_equal(do.raw()[mask], ho.storage[mask])     # padding untouched
    for t in (dx, dw, do):
        t.free()
