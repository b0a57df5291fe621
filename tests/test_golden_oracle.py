"""The oracle reproduces every committed vector of the reference CPU backend."""
import numpy as np
import pytest

import golden_cases as gc
import iomo

CASES = gc.manifest()


@pytest.mark.parametrize("case", CASES, ids=gc.case_id)
def test_oracle_reproduces_reference_vector(case):
    z = gc.arrays()
    key, dtype = case["key"], case["dtype"]
    kind = case["kind"]
    if kind == "binary_directed":
        dims = tuple(case["dims"])
        a, b, o = (iomo.HostTensor(dtype, dims) for _ in range(3))
        a.view().from_logical(z[key + "_a"])
        b.view().from_logical(z[key + "_b"])
        for ieee in (False, True):
            assert iomo.binary(case["op"], a.view(), b.view(), o.view(), ieee) == 0
            assert np.array_equal(o.view().to_logical(), z[key + "_y"])
    elif kind == "binary_view":
        views = []
        for name in ("lhs", "rhs", "out"):
            dims, steps, values = gc.operand(case[name], dtype)
            t = iomo.HostTensor(dtype, dims)
            t.view().from_logical(values)
            views.append((t, gc.apply(t.view(), steps)))
        assert iomo.binary(case["op"], views[0][1], views[1][1], views[2][1]) == 0
        assert np.array_equal(views[2][0].view().to_logical(), z[key + "_y"])
    elif kind == "rmsnorm":
        R, F = case["dims"]
        x, w, o = iomo.HostTensor(dtype, (R, F)), iomo.HostTensor(dtype, (1, F)), iomo.HostTensor(dtype, (R, F))
        x.view().from_logical(z[key + "_x"])
        w.view().from_logical(z[key + "_w"].reshape(1, F))
        assert iomo.rmsnorm(x.view(), w.view(), o.view(), case["eps"]) == 0
        assert np.array_equal(o.view().to_logical(), z[key + "_y"])
    elif kind == "silu":
        dims = tuple(case["dims"])
        x, o = iomo.HostTensor(dtype, dims), iomo.HostTensor(dtype, dims)
        x.view().from_logical(z[key + "_x"])
        assert iomo.silu(x.view(), o.view()) == 0
        assert np.array_equal(o.view().to_logical(), z[key + "_y"])
    else:
        raise AssertionError(kind)
