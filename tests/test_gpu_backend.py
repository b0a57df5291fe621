"""The C++ backend (iom::make_rocm_device of iom_amd/host) driven through IOM's own
Device / TensorView / DeviceOps API next to the reference CPU backend in one
process, as the reference's conformance drivers do
(test/backend/backend_conformance_common.hpp:310: reference + candidate devices).

Skipped where the backend library was not built (it needs the reference headers)."""
import ctypes as C

import numpy as np
import pytest

import datagen
import iomo
from iomo import (ALL_LEAVES, DT_BF16, DT_BOOL, DT_F32, DT_F64, DT_I32, FLOAT_LEAVES, LEAF_BITS,
                  LEAF_NAME, NUMERIC_LEAVES, OP_ADD, OP_DIV, OP_MUL, OP_SUB)

pytestmark = pytest.mark.gpu

BITS = {d: LEAF_BITS[d] for d in ALL_LEAVES}


@pytest.fixture(scope="module")
def devices():
    if not iomo.mi355x_available():
        pytest.skip("oracle/_ref/libiom_mi355x_shim.so not built (needs the reference headers)")
    gpu = iomo.mi355x_backend(arena_bytes=1 << 30, max_in_flight=4)
    cpu = iomo.cpu_backend_beside_mi355x()
    yield cpu, gpu
    gpu.close()
    cpu.close()


def apply(view, steps):
    for name, args in steps:
        view = getattr(view, name)(*args)
    return view


def both(devices, dtype, dims, salt=None, values=None):
    cpu, gpu = devices
    if salt is not None:
        values = datagen.pattern_bits(BITS[dtype], int(np.prod(dims)), salt).reshape(dims)
        if dtype == DT_BOOL:
            values = values & 1          # BOOL host bytes are zero or one (src/tensor_view.cpp:265-270)
    out = []
    for dev in (cpu, gpu):
        t = dev.tensor(dtype, dims)
        if values is not None:
            t.view().from_host(values)
        out.append(t)
    return out


def close(*tensors):
    for t in tensors:
        t.close()


def test_device_identity(devices):
    cpu, gpu = devices
    assert gpu.l.iomc_device_backend_kind(gpu.dev) == 2      # BackendKind::ROCM
    assert cpu.l.iomc_device_backend_kind(cpu.dev) == 0


CASES = [
    ((2, 17, 33), [], (2, 17, 33), [], (2, 17, 33), []),
    ((2, 1, 33), [], (1, 17, 1), [], (2, 17, 33), []),
    ((3, 32, 48), [], (1, 48), [], (3, 32, 48), []),
    ((6, 20, 35), [("slice", (0, 1, 3, 2))], (3, 20, 35), [], (3, 20, 35), []),
    ((4, 3, 16, 32), [("permute", ([1, 0],))], (3, 4, 16, 32), [], (3, 4, 16, 32), []),
    ((4, 3, 16, 32), [("select", (0, 2))], (1, 16, 32), [], (5, 3, 16, 32), [("select", (0, 4))]),
    ((8, 64, 256), [], (8, 64, 256), [], (8, 64, 256), []),
]


@pytest.mark.parametrize("dtype", [DT_I32, DT_F32, DT_BF16])
@pytest.mark.parametrize("op", [OP_ADD, OP_MUL, OP_SUB, OP_DIV])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_binary_matches_reference_cpu_backend_bit_for_bit(devices, dtype, op, case):
    cpu, gpu = devices
    if op == OP_DIV and dtype == DT_I32:
        pytest.skip("refused by both backends: test_integer_division_is_refused_like_the_reference")
    ld, ls, rd, rs, od, os_ = CASES[case]
    cl, gl = both(devices, dtype, ld, salt=0x100 + case)
    cr, gr = both(devices, dtype, rd, salt=0x200 + case)
    co, go = both(devices, dtype, od, salt=0x300 + case)
    tc = cpu.binary(op, apply(cl.view(), ls), apply(cr.view(), rs), apply(co.view(), os_))
    tg = gpu.binary(op, apply(gl.view(), ls), apply(gr.view(), rs), apply(go.view(), os_))
    assert tc > 0 and tg > 0, (tc, tg, gpu.error())
    assert np.array_equal(co.view().to_host(), go.view().to_host())
    close(cl, gl, cr, gr, co, go)


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F32])
@pytest.mark.parametrize("dims,steps", [((17, 33), []), ((40, 2048), []),
                                        ((2, 3, 17, 64), [("permute", ([1, 0],))])])
def test_rmsnorm_and_silu_within_the_bar(devices, dtype, dims, steps):
    cpu, gpu = devices
    n = int(np.prod(dims))
    x = datagen.normal_f32(n, 0, 1, 5)
    w = datagen.uniform_f32(dims[-1], 0.5, 1.5, 6)
    xl = (datagen.bf16_rne(x) if dtype == DT_BF16 else x.view(np.uint32)).reshape(dims)
    wl = (datagen.bf16_rne(w) if dtype == DT_BF16 else w.view(np.uint32)).reshape(1, dims[-1])
    cx, gx = both(devices, dtype, dims, values=xl)
    cw, gw = both(devices, dtype, (1, dims[-1]), values=wl)
    vdims = apply(cx.view(), steps).describe()[0]
    co, go = both(devices, dtype, vdims)
    assert cpu.rmsnorm(apply(cx.view(), steps), cw.view(), co.view(), 1e-5) > 0
    assert gpu.rmsnorm(apply(gx.view(), steps), gw.view(), go.view(), 1e-5) > 0, gpu.error()
    a, b = co.view().to_host(), go.view().to_host()
    if dtype == DT_BF16:
        assert np.abs(a.astype(np.int64) - b.astype(np.int64)).max() <= 1      # 1 BF16 ulp
    else:
        fa, fb = a.view(np.float32).astype(np.float64), b.view(np.float32).astype(np.float64)
        assert np.max(np.abs(fa - fb) / np.maximum(np.abs(fa), 1e-30)) <= 1e-5
    cs, gs = both(devices, dtype, vdims)
    assert cpu.silu(apply(cx.view(), steps), cs.view()) > 0
    assert gpu.silu(apply(gx.view(), steps), gs.view()) > 0, gpu.error()
    a, b = cs.view().to_host().astype(np.int64), gs.view().to_host().astype(np.int64)
    assert np.abs(a - b).max() <= (1 if dtype == DT_BF16 else 8)
    close(cx, gx, cw, gw, co, go, cs, gs)


def test_every_standard_leaf_is_advertised_in_order(devices):
    """23 leaves in the published order (src/shared/standard_tiled_copy.hpp:17-31); the
    conformance drivers iterate exactly this list (test/rocm/test_rocm_conformance.cpp:225-240)."""
    cpu, gpu = devices
    assert gpu.supported_types() == list(ALL_LEAVES) == cpu.supported_types()
    for dtype in ALL_LEAVES:                     # creation is refused for an unadvertised leaf
        t = gpu.tensor(dtype, (3, 5))
        t.close()


@pytest.mark.parametrize("dtype", ALL_LEAVES, ids=[LEAF_NAME[d] for d in ALL_LEAVES])
def test_copy_and_host_transfer_round_trip(devices, dtype):
    cpu, gpu = devices
    dims = (6, 20, 35)
    cs, gs = both(devices, dtype, dims, salt=77)
    vals = cs.view().to_host()
    assert np.array_equal(gs.view().to_host(), vals)
    assert np.array_equal(gs.view().to_host_stream(), cs.view().to_host_stream())
    cd, gd = both(devices, dtype, (3, 20, 35), salt=78)
    assert cpu.copy(cs.view().slice(0, 1, 3, 2), cd.view()) > 0
    assert gpu.copy(gs.view().slice(0, 1, 3, 2), gd.view()) > 0, gpu.error()
    assert np.array_equal(cd.view().to_host(), gd.view().to_host())
    close(cs, gs, cd, gd)


OTHER_NUMERIC = [d for d in NUMERIC_LEAVES if d not in (DT_I32, iomo.DT_U32, DT_F32, DT_BF16)]


@pytest.mark.parametrize("dtype", OTHER_NUMERIC, ids=[LEAF_NAME[d] for d in OTHER_NUMERIC])
@pytest.mark.parametrize("case", [0, 1, 2, 3, 4])
def test_binary_every_other_numeric_leaf(devices, dtype, case):
    """Bit for bit against the reference CPU backend (F64 inputs are kept to values whose
    sums and products are exact or far from a rounding tie of the 64-bit carrier)."""
    cpu, gpu = devices
    op = (OP_ADD, OP_MUL, OP_SUB)[case % 3]
    ld, ls, rd, rs, od, os_ = CASES[case]
    if dtype == DT_F64:
        mk = lambda dims, salt: (datagen.uniform_i32(int(np.prod(dims)), -1000, 1000, salt)
                                 .view(np.int32).astype(np.float64).view(np.uint64).reshape(dims))
        cl, gl = both(devices, dtype, ld, values=mk(ld, 1 + case))
        cr, gr = both(devices, dtype, rd, values=mk(rd, 2 + case))
    else:
        cl, gl = both(devices, dtype, ld, salt=0x100 + case)
        cr, gr = both(devices, dtype, rd, salt=0x200 + case)
    co, go = both(devices, dtype, od, salt=0x300 + case)
    tc = cpu.binary(op, apply(cl.view(), ls), apply(cr.view(), rs), apply(co.view(), os_))
    tg = gpu.binary(op, apply(gl.view(), ls), apply(gr.view(), rs), apply(go.view(), os_))
    assert tc > 0 and tg > 0, (tc, tg, gpu.error())
    assert np.array_equal(co.view().to_host(), go.view().to_host())
    close(cl, gl, cr, gr, co, go)


OTHER_FLOAT = [d for d in FLOAT_LEAVES if d not in (DT_F32, DT_BF16)]


@pytest.mark.parametrize("dtype", OTHER_FLOAT, ids=[LEAF_NAME[d] for d in OTHER_FLOAT])
@pytest.mark.parametrize("case", [0, 1, 2, 3])
def test_division_every_other_float_leaf(devices, dtype, case):
    """Bit for bit against the reference CPU backend (F64 divides whole numbers by powers of
    two, which neither carrier rounds)."""
    cpu, gpu = devices
    ld, ls, rd, rs, od, os_ = CASES[case]
    if dtype == DT_F64:
        num = lambda dims, salt: (datagen.uniform_i32(int(np.prod(dims)), -1000, 1000, salt)
                                  .view(np.int32).astype(np.float64).view(np.uint64).reshape(dims))
        den = lambda dims, salt: np.ldexp(
            1.0, datagen.uniform_i32(int(np.prod(dims)), -8, 8, salt).view(np.int32)
        ).view(np.uint64).reshape(dims)
        cl, gl = both(devices, dtype, ld, values=num(ld, 1 + case))
        cr, gr = both(devices, dtype, rd, values=den(rd, 2 + case))
    else:
        cl, gl = both(devices, dtype, ld, salt=0x400 + case)
        cr, gr = both(devices, dtype, rd, salt=0x500 + case)
    co, go = both(devices, dtype, od, salt=0x600 + case)
    tc = cpu.binary(OP_DIV, apply(cl.view(), ls), apply(cr.view(), rs), apply(co.view(), os_))
    tg = gpu.binary(OP_DIV, apply(gl.view(), ls), apply(gr.view(), rs), apply(go.view(), os_))
    assert tc > 0 and tg > 0, (tc, tg, gpu.error())
    assert np.array_equal(co.view().to_host(), go.view().to_host())
    close(cl, gl, cr, gr, co, go)


def test_integer_division_is_refused_like_the_reference(devices):
    cpu, gpu = devices
    for dtype in (DT_I32, iomo.DT_U8, iomo.DT_I4, iomo.DT_U64):
        ca, ga = both(devices, dtype, (2, 16, 16), salt=1)
        co, go = both(devices, dtype, (2, 16, 16), salt=2)
        before = go.view().to_host().copy()
        tc = cpu.binary(OP_DIV, ca.view(), ca.view(), co.view())
        tg = gpu.binary(OP_DIV, ga.view(), ga.view(), go.view())
        assert tc < 0 and tg == tc, (tc, tg)
        assert np.array_equal(go.view().to_host(), before)
        close(ca, ga, co, go)


@pytest.mark.parametrize("dtype", OTHER_FLOAT, ids=[LEAF_NAME[d] for d in OTHER_FLOAT])
def test_rmsnorm_and_silu_every_other_float_leaf(devices, dtype):
    cpu, gpu = devices
    dims = (3, 17, 40)
    n = int(np.prod(dims))
    if dtype == DT_F64:
        xl = datagen.normal_f32(n, 0, 1, 5).astype(np.float64).view(np.uint64).reshape(dims)
        wl = datagen.uniform_f32(40, 0.5, 1.5, 6).astype(np.float64).view(np.uint64).reshape(1, 40)
    else:
        # every finite-looking pattern: clear the top exponent bit so no NaN / infinity appears
        ebits, fbits = {13: (2, 1), 14: (2, 3), 15: (3, 2), 16: (4, 3), 17: (5, 2), 19: (5, 10)}[dtype]
        keep = ~(1 << (fbits + ebits - 1)) & ((1 << LEAF_BITS[dtype]) - 1)
        xl = (datagen.pattern_bits(LEAF_BITS[dtype], n, 5) & keep).reshape(dims)
        wl = (datagen.pattern_bits(LEAF_BITS[dtype], 40, 6) & keep).reshape(1, 40)
    cx, gx = both(devices, dtype, dims, values=xl)
    cw, gw = both(devices, dtype, (1, 40), values=wl)
    co, go = both(devices, dtype, dims)
    assert cpu.rmsnorm(cx.view(), cw.view(), co.view(), 1e-5) > 0
    assert gpu.rmsnorm(gx.view(), gw.view(), go.view(), 1e-5) > 0, gpu.error()
    cs, gs = both(devices, dtype, dims)
    assert cpu.silu(cx.view(), cs.view()) > 0
    assert gpu.silu(gx.view(), gs.view()) > 0, gpu.error()
    for a, b in ((co, go), (cs, gs)):
        a, b = a.view().to_host(), b.view().to_host()
        if dtype == DT_F64:
            fa, fb = a.view(np.float64), b.view(np.float64)
            assert np.max(np.abs(fa - fb) / np.maximum(np.abs(fa), 1e-300)) <= 1e-12
        else:
            assert np.abs(a.astype(np.int64) - b.astype(np.int64)).max() <= 1   # one encoding step
    close(cx, gx, cw, gw, co, go, cs, gs)


def test_error_classes_match_the_reference(devices):
    cpu, gpu = devices
    for dev in (cpu, gpu):
        a = dev.tensor(DT_F32, (2, 16, 16))
        b = dev.tensor(DT_F32, (3, 16, 16))
        o = dev.tensor(DT_F32, (2, 16, 16))
        assert dev.binary(OP_ADD, a.view(), b.view(), o.view()) == -1        # InvalidArgument
        assert dev.binary(OP_ADD, a.view(), a.view(), b.view()) == -1
        w = dev.tensor(DT_F32, (1, 16))
        assert dev.rmsnorm(a.view(), w.view(), a.view(), 1e-5) == -1         # output aliases input
        assert dev.rmsnorm(a.view(), w.view(), o.view(), -1.0) == -1
        assert dev.wait(12345) != 0                                           # foreign / unsubmitted token
        close(a, b, o, w)
    # the two leaves that carry no arithmetic are Unsupported on both devices, and an
    # integer leaf takes no silu
    for dev in (cpu, gpu):
        for dtype in (DT_BOOL, iomo.DT_F8_E8M0):
            h = dev.tensor(dtype, (2, 16, 16))
            ho = dev.tensor(dtype, (2, 16, 16))
            assert dev.binary(OP_ADD, h.view(), h.view(), ho.view()) == -2
            assert dev.silu(h.view(), ho.view()) == -2
            close(h, ho)
        i = dev.tensor(iomo.DT_I16, (2, 16, 16))
        io = dev.tensor(iomo.DT_I16, (2, 16, 16))
        assert dev.silu(i.view(), io.view()) == -2
        close(i, io)
    # a view of the other device is rejected by the queue
    ca = cpu.tensor(DT_F32, (2, 16, 16))
    ga = gpu.tensor(DT_F32, (2, 16, 16))
    assert gpu.l.iomc_binary(gpu.queue, OP_ADD, ca.view().h, ga.view().h, ga.view().h) == -1
    close(ca, ga)


def test_in_order_queue_with_more_submissions_than_credits(devices):
    """C = 4 in flight; 64 dependent submissions without waiting, then one wait."""
    cpu, gpu = devices
    dims = (4, 64, 128)
    ones = np.full(dims, 1, np.uint32)
    acc_c, acc_g = both(devices, DT_I32, dims, values=np.zeros(dims, np.uint32))
    one_c, one_g = both(devices, DT_I32, dims, values=ones)
    last = 0
    for _ in range(64):
        last = gpu.l.iomc_binary(gpu.queue, OP_ADD, acc_g.view().h, one_g.view().h, acc_g.view().h)
        assert last > 0
    assert gpu.wait(last) == 0
    assert gpu.wait(last) == 0                      # repeat-waitable
    assert np.all(acc_g.view().to_host() == 64)
    close(acc_c, acc_g, one_c, one_g)


def test_two_queues_and_an_owner_released_while_its_work_is_in_flight(devices):
    """Queues of one device run independently and keep their own token spaces; an owner
    destroyed right after submission is kept alive by the queue until completion
    (docs/BACKEND_CONTRACT/queue-and-token-contract.md)."""
    cpu, gpu = devices
    q2 = gpu.second_queue()
    dims = (8, 64, 256)
    a = gpu.tensor(DT_F32, dims); b = gpu.tensor(DT_F32, dims)
    o1 = gpu.tensor(DT_F32, dims); o2 = gpu.tensor(DT_F32, dims)
    va = datagen.uniform_f32(int(np.prod(dims)), -1, 1, 1).view(np.uint32).reshape(dims)
    vb = datagen.uniform_f32(int(np.prod(dims)), -1, 1, 2).view(np.uint32).reshape(dims)
    a.view().from_host(va); b.view().from_host(vb)
    t1 = gpu.l.iomc_binary(gpu.queue, OP_ADD, a.view().h, b.view().h, o1.view().h)
    t2 = q2.l.iomc_binary(q2.queue, OP_MUL, a.view().h, b.view().h, o2.view().h)
    assert t1 > 0 and t2 > 0
    assert (t1 >> 55) != (t2 >> 55)                       # different queue ids in the tokens
    assert gpu.wait(t2) != 0                              # a token of the other queue is refused
    assert q2.wait(t2) == 0 and gpu.wait(t1) == 0
    fa, fb = va.view(np.float32), vb.view(np.float32)
    assert np.array_equal(o1.view().to_host().view(np.float32), fa + fb)
    assert np.array_equal(o2.view().to_host().view(np.float32), fa * fb)
    # release the inputs immediately after submitting
    tmp = gpu.tensor(DT_F32, dims)
    tmp.view().from_host(va)
    t3 = gpu.l.iomc_binary(gpu.queue, OP_SUB, tmp.view().h, b.view().h, o1.view().h)
    tmp.close()
    assert t3 > 0 and gpu.wait(t3) == 0
    assert np.array_equal(o1.view().to_host().view(np.float32), fa - fb)
    q2.close()
    close(a, b, o1, o2)


def test_arena_exhaustion_and_reuse(devices):
    cpu, gpu = devices
    small = iomo.mi355x_backend(arena_bytes=1 << 20, max_in_flight=2)
    try:
        t = small.tensor(DT_F32, (256, 256))            # 256 KiB
        with pytest.raises(RuntimeError, match="bad_alloc"):
            small.tensor(DT_F32, (512, 512))            # 1 MiB does not fit beside it
        t.close()
        t2 = small.tensor(DT_F32, (384, 512))           # fits again once the first is gone
        t2.close()
        queues = [small.l.iomc_queue_create(small.dev) for _ in range(3)]   # + the backend's own = 4
        assert all(queues)
        assert not small.l.iomc_queue_create(small.dev)                      # the fifth is refused
        for q in queues:
            small.l.iomc_queue_destroy(q)
    finally:
        small.close()


def test_bad_factory_configuration_is_rejected_before_any_native_effect():
    if not iomo.mi355x_available():
        pytest.skip("backend library not built")
    l = iomo.mi355x_lib()
    assert not l.iomc_mi355x_device_create(0, 0, 16)
    assert b"invalid_argument" in l.iomc_last_error()
    assert not l.iomc_mi355x_device_create(0, 1000, 16)           # not a multiple of 32
    assert not l.iomc_mi355x_device_create(99, 1 << 20, 16)       # no such ordinal


def test_submit_and_wait_cost_through_device_ops(devices, capsys):
    """What a caller pays on top of the kernel: one add submitted and waited for through
    DeviceOps (validation, snapshots, registry entries, admission, launch, event, completion
    thread), and a burst of 64 submissions with one wait.  Printed for the record; the bounds
    only catch a queue that has started to serialise on something slow."""
    import time
    del devices                      # (the shared fixture keeps four operations in flight; the default is 16)
    gpu = iomo.mi355x_backend(arena_bytes=1 << 29, max_in_flight=16)
    small = (1, 16, 2048)
    big = (16, 512, 2048)
    for dims, label in ((small, "64 KiB"), (big, "32 MiB")):
        a, b, o = (gpu.tensor(DT_BF16, dims) for _ in range(3))
        av, bv, ov = a.view(), b.view(), o.view()
        for _ in range(20):
            assert gpu.wait(gpu.l.iomc_binary(gpu.queue, OP_ADD, av.h, bv.h, ov.h)) == 0
        single = []
        for _ in range(200):
            t0 = time.perf_counter()
            tok = gpu.l.iomc_binary(gpu.queue, OP_ADD, av.h, bv.h, ov.h)
            assert gpu.wait(tok) == 0
            single.append(time.perf_counter() - t0)
        t0 = time.perf_counter()
        for _ in range(64):
            tok = gpu.l.iomc_binary(gpu.queue, OP_ADD, av.h, bv.h, ov.h)
            assert tok > 0
        assert gpu.wait(tok) == 0
        burst = (time.perf_counter() - t0) / 64
        single.sort()
        with capsys.disabled():
            print("\n  DeviceOps add BF16 %s: submit+wait median %.1f us (p90 %.1f), burst of 64 %.1f us per op"
                  % (label, single[100] * 1e6, single[180] * 1e6, burst * 1e6), flush=True)
        assert single[100] < 2e-3 and burst < 1e-3
        close(a, b, o)
    gpu.close()


def test_tensors_beyond_4_gib_in_a_large_arena():
    """An 18 GiB arena with two [40,64,2^20] BF16 tensors (5 GiB each) and room for the 5 GiB
    staging range of a whole-tensor transfer: arena offsets, window byte counts and the host
    transfers of the backend beyond 32 bits.  t = a + 0 over forty planes
    (a scalar per plane), u = t * r with a row vector; every plane against the closed form."""
    if not iomo.mi355x_available():
        pytest.skip("oracle/_ref/libiom_mi355x_shim.so not built (needs the reference headers)")
    gpu = iomo.mi355x_backend(arena_bytes=18 << 30, max_in_flight=4)
    planes, rows, cols = 40, 64, 1 << 20
    a_values = datagen.bf16_rne(datagen.normal_f32(rows * cols, 0, 1, 301)).reshape(1, rows, cols)
    r_values = datagen.bf16_rne(datagen.uniform_f32(cols, 0.5, 1.5, 302)).reshape(1, cols)
    a = gpu.tensor(DT_BF16, (1, rows, cols)); a.view().from_host(a_values)
    r = gpu.tensor(DT_BF16, (1, cols)); r.view().from_host(r_values)
    zero = gpu.tensor(DT_BF16, (planes, 1, 1)); zero.view().from_host(np.zeros((planes, 1, 1), np.uint16))
    t = gpu.tensor(DT_BF16, (planes, rows, cols))
    u = gpu.tensor(DT_BF16, (planes, rows, cols))
    assert gpu.binary(OP_ADD, a.view(), zero.view(), t.view()) > 0, gpu.error()
    assert gpu.binary(OP_MUL, t.view(), r.view(), u.view()) > 0, gpu.error()
    fa = datagen.bf16_to_f32(a_values.reshape(-1))
    e1 = datagen.bf16_rne(fa + np.float32(0)).reshape(rows, cols)
    e2 = datagen.bf16_rne(datagen.bf16_to_f32(e1.reshape(-1)).reshape(rows, cols)
                          * datagen.bf16_to_f32(r_values.reshape(-1))[None, :]).reshape(rows, cols)
    got = t.view().to_host()
    for p in range(planes):
        assert np.array_equal(got[p], e1), p
    got = u.view().to_host()
    for p in range(planes):
        assert np.array_equal(got[p], e2), p
    close(a, r, zero, t, u)
    gpu.close()


def test_rank_eight_operands_like_the_reference_conformance_cases(devices):
    """test/backend/backend_conformance_common.hpp:581-690: a rank-eight owner against a rank-two
    operand, and the rank-eight broadcast add (a row vector per plane against one column vector)
    with its closed form; both against the reference CPU backend as well."""
    cpu, gpu = devices
    DT_U8 = iomo.DT_U8
    # rank eight + rank two
    dims8 = (1, 1, 1, 1, 1, 1, 17, 33)
    a_vals = datagen.pattern_bits(8, 17 * 33, 0x8A).reshape(dims8)
    b_vals = datagen.pattern_bits(8, 17 * 33, 0x8B).reshape(17, 33)
    results = []
    for dev in (cpu, gpu):
        l = dev.tensor(DT_U8, dims8); l.view().from_host(a_vals)
        r = dev.tensor(DT_U8, (17, 33)); r.view().from_host(b_vals)
        o = dev.tensor(DT_U8, dims8); o.view().from_host(np.zeros(dims8, np.uint8))
        assert dev.binary(OP_ADD, l.view(), r.view(), o.view()) > 0, dev.error()
        results.append(o.view().to_host())
        close(l, r, o)
    assert np.array_equal(results[0], results[1])
    assert np.array_equal(results[1].reshape(17, 33), (a_vals.reshape(17, 33) + b_vals).astype(np.uint8))
    # the rank-eight broadcast: lhs [.., 17, 1] carries one plane, rhs [.., 2, 1, 33] a row per plane
    lhs_dims, rhs_dims, out_dims = (1, 1, 1, 1, 1, 1, 17, 1), (1, 1, 1, 1, 1, 2, 1, 33), (1, 1, 1, 1, 1, 2, 17, 33)
    lhs_vals = datagen.pattern_bits(8, 17, 0x8C).reshape(lhs_dims)
    rhs_vals = datagen.pattern_bits(8, 66, 0x8D).reshape(rhs_dims)
    want = (lhs_vals.reshape(1, 17, 1).astype(np.uint32) + rhs_vals.reshape(2, 1, 33)).astype(np.uint8)
    for dev in (cpu, gpu):
        l = dev.tensor(DT_U8, lhs_dims); l.view().from_host(lhs_vals)
        r = dev.tensor(DT_U8, rhs_dims); r.view().from_host(rhs_vals)
        o = dev.tensor(DT_U8, out_dims); o.view().from_host(np.full(out_dims, 0xAA, np.uint8))
        assert dev.binary(OP_ADD, l.view(), r.view(), o.view()) > 0, dev.error()
        assert np.array_equal(o.view().to_host().reshape(2, 17, 33), want)
        close(l, r, o)
