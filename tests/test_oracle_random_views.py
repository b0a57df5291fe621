"""The seeded random views of view_cases.py between the C restatement and the compiled
reference CPU backend (skipped where oracle/_ref was not built): binary operations and copy
bit for bit over whole owner storages, so the oracle's view, broadcast and padding rules are
pinned on the very cases the GPU tests compare against."""
import numpy as np
import pytest

import datagen
import iomo
import view_cases
from iomo import (DT_BF16, DT_F16, DT_F32, DT_F6_E2M3, DT_F8_E4M3FN, DT_I32, DT_I64, DT_I8, DT_U4, FLOAT_LEAVES,
                  LEAF_BITS, LEAF_NAME, OP_ADD, OP_DIV, OP_MUL, OP_SUB)

LEAVES = tuple(d for d in iomo.NUMERIC_LEAVES if d != iomo.DT_F64)   # F64: the x87 carrier rounds twice
CASES = 400


def both(ref, dtype, dims, salt):
    rt = ref.tensor(dtype, dims)
    ht = iomo.HostTensor(dtype, dims)
    values = datagen.pattern_bits(LEAF_BITS[dtype], int(np.prod(dims)), salt).reshape(dims)
    if dtype == iomo.DT_BOOL:
        values = values & 1                              # BOOL host bytes are zero or one
    rt.view().from_host(values)
    ht.view().from_logical(values)
    return rt, ht


def same_storage(rt, ht):
    return np.array_equal(rt.view().raw_storage().view(np.uint8), ht.storage.view(np.uint8))


@pytest.mark.parametrize("case", range(CASES))
def test_binary_on_random_views(ref, case):
    dtype = LEAVES[case % len(LEAVES)]
    op = (OP_ADD, OP_MUL, OP_SUB, OP_DIV)[(case // len(LEAVES)) % 4]
    if op == OP_DIV and dtype not in FLOAT_LEAVES:
        op = OP_SUB
    lead, rows, cols, operands = view_cases.binary_case(case)
    owners = [both(ref, dtype, dims, 0x900 + 3 * case + i) for i, (dims, _) in enumerate(operands)]
    rv = [view_cases.apply(r.view(), steps) for (r, _), (_, steps) in zip(owners, operands)]
    hv = [view_cases.apply(h.view(), steps) for (_, h), (_, steps) in zip(owners, operands)]
    assert ref.binary(op, rv[0], rv[1], rv[2]) > 0, (ref.error(), LEAF_NAME[dtype], operands)
    for ieee in (False, True):
        assert iomo.binary(op, hv[0], hv[1], hv[2], ieee) == 0
        assert same_storage(*owners[2]), (LEAF_NAME[dtype], op, ieee, lead, rows, cols, operands)


@pytest.mark.parametrize("case", range(CASES // 2))
def test_copy_on_random_views(ref, case):
    dtype = (LEAVES + (iomo.DT_BOOL, iomo.DT_F8_E8M0, iomo.DT_U2, iomo.DT_F64))[case % (len(LEAVES) + 4)]
    lead, rows, cols, operands = view_cases.unary_case(case)
    owners = [both(ref, dtype, dims, 0xA00 + 2 * case + i) for i, (dims, _) in enumerate(operands)]
    rv = [view_cases.apply(r.view(), steps) for (r, _), (_, steps) in zip(owners, operands)]
    hv = [view_cases.apply(h.view(), steps) for (_, h), (_, steps) in zip(owners, operands)]
    assert ref.copy(rv[0], rv[1]) > 0, ref.error()
    assert iomo.copy(hv[0], hv[1]) == 0
    assert same_storage(*owners[1]), (LEAF_NAME[dtype], lead, rows, cols, operands)


def finite_bits(dtype, count, salt):
    """Raw encodings with moderate exponents (no NaN / infinity patterns) for the floating leaves."""
    fmt = {13: (2, 1, 1), 14: (2, 3, 1), 15: (3, 2, 3), 16: (4, 3, 7), 17: (5, 2, 15), 19: (5, 10, 15),
           20: (8, 7, 127), 21: (8, 23, 127), 22: (11, 52, 1023)}
    v = datagen.pattern_bits(LEAF_BITS[dtype], count, salt)
    if dtype not in fmt or dtype in (13, 14, 15):
        return v
    ebits, fbits, bias = fmt[dtype]
    top = (1 << ebits) - 1
    exp = (v.astype(np.uint64) >> np.uint64(fbits)) & np.uint64(top)
    exp = exp % np.uint64(min(5, top - 1)) + np.uint64(max(bias - 2, 1))
    cleared = v.astype(np.uint64) & ~np.uint64(top << fbits)
    return (cleared | (exp << np.uint64(fbits))).astype(v.dtype)


def filled(ref, dtype, dims, values):
    rt = ref.tensor(dtype, dims)
    ht = iomo.HostTensor(dtype, dims)
    rt.view().from_host(values)
    ht.view().from_logical(values)
    return rt, ht


FLOATS = tuple(FLOAT_LEAVES)


@pytest.mark.parametrize("case", range(135))
def test_rmsnorm_and_silu_on_random_views(ref, case):
    """Bit for bit: the restatement follows the CPU backend's order of operations and calls the
    same libm (src/cpu/queue.cpp:1144-1296, src/shared/scalar_silu.hpp:69-97)."""
    dtype = FLOATS[case % len(FLOATS)]
    lead, rows, cols, operands = view_cases.unary_case(case, salt=1515)
    rx, hx = filled(ref, dtype, operands[0][0], finite_bits(dtype, int(np.prod(operands[0][0])), 0x100 + case).reshape(operands[0][0]))
    rw, hw = filled(ref, dtype, (1, cols), finite_bits(dtype, cols, 0x200 + case).reshape(1, cols))
    ro, ho = both(ref, dtype, operands[1][0], 0x300 + case)
    rxv, hxv = view_cases.apply(rx.view(), operands[0][1]), view_cases.apply(hx.view(), operands[0][1])
    rov, hov = view_cases.apply(ro.view(), operands[1][1]), view_cases.apply(ho.view(), operands[1][1])
    assert ref.rmsnorm(rxv, rw.view(), rov, 1e-5) > 0, ref.error()
    assert iomo.rmsnorm(hxv, hw.view(), hov, 1e-5) == 0
    assert same_storage(ro, ho), ("rmsnorm", LEAF_NAME[dtype], lead, rows, cols, operands)
    assert ref.silu(rxv, rov) > 0, ref.error()
    assert iomo.silu(hxv, hov) == 0
    assert same_storage(ro, ho), ("silu", LEAF_NAME[dtype], lead, rows, cols, operands)


@pytest.mark.parametrize("case", range(120))
def test_layer_movement_on_random_views(ref, case):
    """cache_append, rope and embedding through views, whole owners bit for bit."""
    rng = view_cases.Stream(case, 1616)
    dtype = (DT_BF16, DT_F32, DT_I8, DT_U4, DT_F16, DT_F6_E2M3, DT_I64, iomo.DT_BOOL)[case % 8]
    nlead = 1 + rng.below(3)
    lead = tuple(1 + rng.below(4) for _ in range(nlead))
    R = (1, 3, 16, 17, 40)[rng.below(5)]
    D = (2, 16, 24, 64, 128)[rng.below(5)]
    a = (0, 1, 15, 16, 37)[rng.below(5)]
    capacity = a + R + rng.below(20)
    so, ss = view_cases.viewed_operand(rng, lead, R, D)
    co, cs = view_cases.viewed_operand(rng, lead, capacity, D)
    rs_, hs = both(ref, dtype, so, 0x400 + case)
    rc_, hc = both(ref, dtype, co, 0x500 + case)
    assert ref.cache_append(view_cases.apply(rs_.view(), ss), view_cases.apply(rc_.view(), cs), a) > 0, ref.error()
    assert iomo.cache_append(view_cases.apply(hs.view(), ss), view_cases.apply(hc.view(), cs), a) == 0
    assert same_storage(rc_, hc), ("cache_append", LEAF_NAME[dtype], so, ss, co, cs, a)
    # rope over the floating leaves, on the source's shape
    if dtype in FLOAT_LEAVES:
        rx, hx = filled(ref, dtype, so, finite_bits(dtype, int(np.prod(so)), 0x600 + case).reshape(so))
        oo, os_ = view_cases.viewed_operand(rng, lead, R, D)
        ro, ho = both(ref, dtype, oo, 0x700 + case)
        assert ref.rope(view_cases.apply(rx.view(), ss), view_cases.apply(ro.view(), os_), a, 10000.0) > 0, ref.error()
        assert iomo.rope(view_cases.apply(hx.view(), ss), view_cases.apply(ho.view(), os_), a, 10000.0) == 0
        assert same_storage(ro, ho), ("rope", LEAF_NAME[dtype], so, ss, oo, os_, a)
    # embedding: payload of this leaf, ids of a drawn integer leaf
    index_dtype = (DT_I32, iomo.DT_U8, iomo.DT_I16, iomo.DT_U64)[rng.below(4)]
    V, F, n_ids = (1, 7, 37)[rng.below(3)], (1, 16, 33, 128)[rng.below(4)], (1, 2, 9, 21)[rng.below(4)]
    elead = lead[:rng.below(nlead + 1)]
    io, isteps = view_cases.viewed_operand(rng, elead, 1, n_ids)
    eo, esteps = view_cases.viewed_operand(rng, elead, n_ids, F)
    rt, ht = both(ref, dtype, (V, F), 0x800 + case)
    ids = (datagen.pattern_bits(32, int(np.prod(io)), 0x900 + case) % V).astype(iomo.NP_OF[index_dtype]).reshape(io)
    ri, hi = filled(ref, index_dtype, io, ids)
    re_, he = both(ref, dtype, eo, 0xA00 + case)
    token, status = ref.embedding(rt.view(), view_cases.apply(ri.view(), isteps), view_cases.apply(re_.view(), esteps))
    assert token > 0 and status == 0, ref.error()
    assert iomo.embedding(ht.view(), view_cases.apply(hi.view(), isteps), view_cases.apply(he.view(), esteps)) == 0
    assert same_storage(re_, he), ("embedding", LEAF_NAME[dtype], io, isteps, eo, esteps)


@pytest.mark.parametrize("case", range(105))
def test_linear_on_random_shapes_and_views(ref, case):
    """The scalar recurrence of the linear contract, every numeric leaf, bit for bit."""
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
    rx, hx = filled(ref, dtype, xo, finite_bits(dtype, int(np.prod(xo)), 0xB00 + case).reshape(xo))
    rw, hw = filled(ref, dtype, (H * D, inner), finite_bits(dtype, H * D * inner, 0xC00 + case).reshape(H * D, inner))
    ro, ho = both(ref, dtype, oo, 0xD00 + case)
    args = (s, R, head_planar, H if head_planar else 1, D if head_planar else H * D)
    assert ref.linear(view_cases.apply(rx.view(), xs), rw.view(), view_cases.apply(ro.view(), os_), *args) > 0, ref.error()
    assert iomo.linear(view_cases.apply(hx.view(), xs), hw.view(), view_cases.apply(ho.view(), os_), *args) == 0
    if dtype == iomo.DT_F64:
        # the CPU backend's extended carrier: one unit apart where it rounds twice
        a_, b_ = ro.view().to_host().astype(np.int64), ho.view().to_logical().astype(np.int64)
        assert np.abs(a_ - b_).max() <= 1
    else:
        assert same_storage(ro, ho), (LEAF_NAME[dtype], xo, xs, oo, os_, args)
