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
