"""The private fusion iomx_launch_add_rmsnorm (sum = x + y, out = rmsnorm(sum, scale)) against the
two public launches it replaces -- bit for bit in both outputs, tile padding of unselected planes
untouched -- and against the CPU oracle's ADD (bit-exact) and RMSNorm (the bar of the operation:
<= 1 BF16 / F16 ulp, 1e-5 relative for F32).  Called through the C ABI."""
import numpy as np
import pytest

import datagen
import iomo
from iom_amd import iomx
from iomo import DT_BF16, DT_F16, DT_F32, OP_ADD

pytestmark = pytest.mark.gpu

BITS = {DT_BF16: 16, DT_F16: 16, DT_F32: 32}


@pytest.fixture(scope="module", autouse=True)
def _device():
    assert iomx.device_count() >= 1, "no HIP device visible"
    iomx.check(iomx.lib().iomx_set_device(0))
    yield


def values_of(dtype, dims, salt, sigma=1.0):
    v = datagen.normal_f32(int(np.prod(dims)), 0.0, sigma, salt)
    if dtype == DT_BF16:
        return datagen.bf16_rne(v).reshape(dims)
    if dtype == DT_F16:
        return v.astype(np.float16).view(np.uint16).reshape(dims)
    return v.view(np.uint32).reshape(dims)


def apply(view, steps):
    for name, args in steps:
        view = getattr(view, name)(*args)
    return view


def owner_pair(dtype, dims, values=None, fill=0x5A):
    d = iomx.DeviceTensor(dtype, dims, fill=fill)
    h = iomo.HostTensor(dtype, dims, fill=fill)
    if values is not None:
        d.view().from_host(values)
        h.view().from_logical(values)
    return d, h


def ordered(bits, width):
    bits = bits.astype(np.int64)
    sign = 1 << (width - 1)
    return np.where(bits & sign, (~bits) & ((1 << width) - 1), bits | sign)


# (owner dims, view steps) of the four full operands; every view has the same logical shape
VIEW_CASES = [
    ("dense rank 2", (64, 256), [], (64, 256), [], (64, 256), [], (64, 256), []),
    ("dense rank 3", (5, 32, 512), [], (5, 32, 512), [], (5, 32, 512), [], (5, 32, 512), []),
    ("stepped x, offset y, stepped outputs",
     (7, 32, 128), [("slice", (0, 1, 3, 2))], (5, 32, 128), [("slice", (0, 2, 3, 1))],
     (6, 32, 128), [("slice", (0, 0, 3, 2))], (4, 32, 128), [("slice", (0, 1, 3, 1))]),
    ("permuted leading axes",
     (3, 4, 16, 64), [("permute", ([1, 0],))], (4, 3, 16, 64), [],
     (4, 3, 16, 64), [], (3, 4, 16, 64), [("permute", ([1, 0],))]),
    ("selected plane of a rank-4 owner",
     (2, 3, 48, 2048), [("select", (0, 1))], (3, 48, 2048), [],
     (3, 48, 2048), [], (2, 3, 48, 2048), [("select", (0, 0))]),
    ("wide rows, split bands", (2, 16, 8192), [], (2, 16, 8192), [], (2, 16, 8192), [], (2, 16, 8192), []),
]


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F16, DT_F32], ids=["BF16", "F16", "F32"])
@pytest.mark.parametrize("case", VIEW_CASES, ids=[c[0] for c in VIEW_CASES])
def test_fused_equals_the_two_launches_and_the_oracle(dtype, case):
    _, xd, xs, yd, ys, sd, ss, od, os_ = case
    dx, hx = owner_pair(dtype, xd, values_of(dtype, xd, 101))
    dy, hy = owner_pair(dtype, yd, values_of(dtype, yd, 102))
    F = xd[-1]
    w = values_of(dtype, (1, F), 103, 0.25)
    if dtype == DT_F32:
        w = (w.view(np.float32) + 1.0).view(np.uint32)
    dw, hw = owner_pair(dtype, (1, F), w)
    # fused outputs, two-launch outputs, oracle outputs: same poison everywhere
    dsum_f, _ = owner_pair(dtype, sd)
    dout_f, _ = owner_pair(dtype, od)
    dsum_s, hsum = owner_pair(dtype, sd)
    dout_s, hout = owner_pair(dtype, od)
    vx, vy = apply(dx.view(), xs), apply(dy.view(), ys)
    iomx.check(iomx.add_rmsnorm(vx, vy, apply(dsum_f.view(), ss), dw.view(), apply(dout_f.view(), os_), 1e-5),
               "add_rmsnorm")
    assert iomx.last_launch().kernel.decode().startswith("add_rmsnorm")
    iomx.check(iomx.binary(OP_ADD, vx, vy, apply(dsum_s.view(), ss)), "add")
    iomx.check(iomx.rmsnorm(apply(dsum_s.view(), ss), dw.view(), apply(dout_s.view(), os_), 1e-5), "rmsnorm")
    # 1. bit for bit the sequence, raw storage (padding and unselected planes included)
    assert np.array_equal(dsum_f.raw(), dsum_s.raw())
    assert np.array_equal(dout_f.raw(), dout_s.raw())
    # 2. the oracle: ADD bit-exact, RMSNorm within the operation's bar
    assert iomo.binary(OP_ADD, apply(hx.view(), xs), apply(hy.view(), ys), apply(hsum.view(), ss)) == 0
    assert iomo.rmsnorm(apply(hsum.view(), ss), hw.view(), apply(hout.view(), os_), 1e-5) == 0
    assert np.array_equal(dsum_f.raw(), hsum.storage)
    got = apply(dout_f.view(), os_).to_host()
    want = apply(hout.view(), os_).to_logical()
    if dtype == DT_F32:
        g, r = got.view(np.float32).astype(np.float64), want.view(np.float32).astype(np.float64)
        assert (np.abs(g - r) <= 1e-5 * np.abs(r) + 1e-30).all()
    else:
        assert np.abs(ordered(got, 16) - ordered(want, 16)).max() <= 1
    for t in (dx, dy, dw, dsum_f, dout_f, dsum_s, dout_s):
        t.free()


def test_sum_may_be_written_over_x():
    """The residual stream updated in place: sum is the identical window of x."""
    dims = (3, 32, 256)
    vals = values_of(DT_BF16, dims, 7)
    dx, _ = owner_pair(DT_BF16, dims, vals)
    dx2, _ = owner_pair(DT_BF16, dims, vals)
    dy, _ = owner_pair(DT_BF16, dims, values_of(DT_BF16, dims, 8))
    dw, _ = owner_pair(DT_BF16, (1, 256), values_of(DT_BF16, (1, 256), 9))
    df, ds = iomx.DeviceTensor(DT_BF16, dims, fill=0x11), iomx.DeviceTensor(DT_BF16, dims, fill=0x11)
    iomx.check(iomx.add_rmsnorm(dx.view(), dy.view(), dx.view(), dw.view(), df.view(), 1e-5), "fused in place")
    iomx.check(iomx.binary(OP_ADD, dx2.view(), dy.view(), dx2.view()), "add in place")
    iomx.check(iomx.rmsnorm(dx2.view(), dw.view(), ds.view(), 1e-5), "rmsnorm")
    assert np.array_equal(dx.raw(), dx2.raw()) and np.array_equal(df.raw(), ds.raw())
    for t in (dx, dx2, dy, dw, df, ds):
        t.free()


def test_special_values_follow_the_sequence():
    """Rows holding NaN, infinities of both signs (inf + -inf), signed zeros and subnormals."""
    F = 64
    rows = 32
    a = np.zeros((rows, F), np.float32)
    b = np.zeros((rows, F), np.float32)
    a[0, 3], b[0, 3] = np.inf, -np.inf        # invalid sum -> NaN row
    a[1, 5] = np.nan
    a[2, :], b[2, :] = -0.0, -0.0             # all -0
    a[3, :], b[3, :] = 0.0, -0.0              # +0
    a[4, 7], b[4, 7] = 3.0e38, 3.0e38         # overflow to +inf in the sum
    a[5, :], b[5, :] = 1e-40, -1e-40          # subnormals cancelling
    a[6:, :] = datagen.normal_f32((rows - 6) * F, 0, 1, 5).reshape(rows - 6, F)
    b[6:, :] = datagen.normal_f32((rows - 6) * F, 0, 1, 6).reshape(rows - 6, F)
    for dtype in (DT_BF16, DT_F32):
        conv = (lambda v: datagen.bf16_rne(v)) if dtype == DT_BF16 else (lambda v: v.view(np.uint32))
        dx, _ = owner_pair(dtype, (rows, F), conv(a.reshape(-1)).reshape(rows, F))
        dy, _ = owner_pair(dtype, (rows, F), conv(b.reshape(-1)).reshape(rows, F))
        w = conv(datagen.uniform_f32(F, 0.5, 1.5, 4)).reshape(1, F)
        dw, _ = owner_pair(dtype, (1, F), w)
        sf, of, ss, os_ = (iomx.DeviceTensor(dtype, (rows, F), fill=0x22) for _ in range(4))
        iomx.check(iomx.add_rmsnorm(dx.view(), dy.view(), sf.view(), dw.view(), of.view(), 1e-5), "fused")
        iomx.check(iomx.binary(OP_ADD, dx.view(), dy.view(), ss.view()), "add")
        iomx.check(iomx.rmsnorm(ss.view(), dw.view(), os_.view(), 1e-5), "rmsnorm")
        assert np.array_equal(sf.raw(), ss.raw()) and np.array_equal(of.raw(), os_.raw())
        for t in (dx, dy, dw, sf, of, ss, os_):
            t.free()


def test_rejections():
    dims = (32, 64)
    t = [iomx.DeviceTensor(DT_BF16, dims) for _ in range(4)]
    w = iomx.DeviceTensor(DT_BF16, (1, 64))
    x, y, s, o = (q.view() for q in t)
    assert iomx.add_rmsnorm(x, y, s, w.view(), o, 1e-5) == 0
    # out must not share storage with an input or with the sum
    assert iomx.add_rmsnorm(x, y, s, w.view(), x, 1e-5) == iomx.ERR_INVALID
    assert iomx.add_rmsnorm(x, y, o, w.view(), o, 1e-5) == iomx.ERR_INVALID
    # negative or non-finite eps
    assert iomx.add_rmsnorm(x, y, s, w.view(), o, -1.0) == iomx.ERR_INVALID
    assert iomx.add_rmsnorm(x, y, s, w.view(), o, float("nan")) == iomx.ERR_INVALID
    # shapes must agree, the scale is [1, F]
    other = iomx.DeviceTensor(DT_BF16, (32, 80))
    assert iomx.add_rmsnorm(x, other.view(), s, w.view(), o, 1e-5) == iomx.ERR_INVALID
    assert iomx.add_rmsnorm(x, y, s, x, o, 1e-5) == iomx.ERR_INVALID
    # padded shapes and other leaves go through the two public launches
    pad = [iomx.DeviceTensor(DT_BF16, (30, 64)) for _ in range(4)]
    assert iomx.add_rmsnorm(pad[0].view(), pad[1].view(), pad[2].view(), w.view(), pad[3].view(), 1e-5) \
        == iomx.ERR_UNSUPPORTED
    i32 = [iomx.DeviceTensor(iomo.DT_I32, dims) for _ in range(4)]
    wi = iomx.DeviceTensor(iomo.DT_I32, (1, 64))
    assert iomx.add_rmsnorm(i32[0].view(), i32[1].view(), i32[2].view(), wi.view(), i32[3].view(), 1e-5) \
        == iomx.ERR_UNSUPPORTED
    # a sum that overlaps x in a different window
    big = iomx.DeviceTensor(DT_BF16, (4, 32, 64))
    three = [iomx.DeviceTensor(DT_BF16, (2, 32, 64)) for _ in range(2)]
    w3 = iomx.DeviceTensor(DT_BF16, (1, 64))
    assert iomx.add_rmsnorm(big.view().slice(0, 0, 2, 1), three[0].view(), big.view().slice(0, 1, 2, 1),
                            w3.view(), three[1].view(), 1e-5) == iomx.ERR_INVALID
    for q in t + [w, other] + pad + i32 + [wi, big, w3] + three:
        q.free()


def test_layer_size_64x512x2048_bf16_bit_identical_to_the_sequence():
    dims = (64, 512, 2048)
    n = int(np.prod(dims))
    base = datagen.bf16_rne(datagen.normal_f32(1 << 22, 0, 1, 21))
    xs = np.concatenate([np.roll(base, 977 * i) for i in range(n >> 22)])
    ys = np.concatenate([np.roll(base, 1013 * i + 5) for i in range(n >> 22)])
    dx, dy = iomx.DeviceTensor(DT_BF16, dims, fill=None), iomx.DeviceTensor(DT_BF16, dims, fill=None)
    dx.upload_raw(xs)
    dy.upload_raw(ys)
    dw = iomx.DeviceTensor(DT_BF16, (1, 2048))
    dw.view().from_host(datagen.bf16_rne(datagen.uniform_f32(2048, 0.5, 1.5, 22)).reshape(1, 2048))
    sf, of, ss, os_ = (iomx.DeviceTensor(DT_BF16, dims, fill=None) for _ in range(4))
    iomx.check(iomx.add_rmsnorm(dx.view(), dy.view(), sf.view(), dw.view(), of.view(), 1e-5), "fused")
    print("kernel:", iomx.last_launch().kernel.decode(), flush=True)
    iomx.check(iomx.binary(OP_ADD, dx.view(), dy.view(), ss.view()), "add")
    iomx.check(iomx.rmsnorm(ss.view(), dw.view(), os_.view(), 1e-5), "rmsnorm")
    assert np.array_equal(sf.raw(), ss.raw())
    assert np.array_equal(of.raw(), os_.raw())
    # the sum is the closed form bf16_rne(float(x) + float(y)) with the codec's NaN rule
    f = datagen.bf16_to_f32(xs) + datagen.bf16_to_f32(ys)
    assert np.array_equal(sf.raw(), datagen.bf16_rne(f))
    for t in (dx, dy, dw, sf, of, ss, os_):
        t.free()
