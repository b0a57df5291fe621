"""Differential test over seeded random views: the HIP library against the CPU oracle.

Every case draws a result shape of 2 to 5 axes, operands that broadcast along any subset of
them (including operands of lower rank), and for every operand an owner that is reached
through select / strided slice / permute; owners are pre-filled, so whatever a kernel writes
outside the selected window shows as a storage difference.  Binary operations and copy are
bit-exact (F64 against the binary64-carrier rule); RMSNorm is within one encoding step of the
leaf / 1e-5 relative.  The same cases run between the oracle and the compiled reference in
test_oracle_random_views.py.
"""
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


def pair(dtype, dims, salt):
    dt = iomx.DeviceTensor(dtype, dims, fill=0x5A)
    ht = iomo.HostTensor(dtype, dims, fill=0x5A)
    values = datagen.pattern_bits(LEAF_BITS[dtype], int(np.prod(dims)), salt).reshape(dims)
    if dtype == iomo.DT_BOOL:
        values = values & 1                              # BOOL host bytes are zero or one
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
    owners = [pair(dtype, dims, 0x900 + 3 * case + i) for i, (dims, _) in enumerate(operands)]
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
        g, w = got.view(np.float32), want.view(np.float32)
        assert np.all(np.abs(g - w) <= 4e-7 * np.abs(w) + 1e-37), (lead, rows, cols, operands)
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
