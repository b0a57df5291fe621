"""Seeded random tensor views for differential tests.

A case describes, for every operand, an owner shape and the chain of view steps (select,
slice with a step, permute of the leading axes) that yields the operand's logical shape; the
same chain is applied to a HostTensor of the oracle, a DeviceTensor of the HIP library and an
IomTensor of the compiled reference, so all three see the same planes through the same strides.
Right-aligned broadcasting (src/device_ops_binary.cpp:121-143) is drawn per axis: an operand may
have extent 1 where the result has more, or fewer axes than the result.

Everything is derived from the case number with a hash stream: no global random state.
"""
from __future__ import annotations

import numpy as np

import datagen


class Stream:
    """Deterministic integer stream of one case."""

    def __init__(self, case: int, salt: int):
        self.values = datagen.pattern_bits(32, 512, (case * 7919 + salt) & 0x7FFFFFFF).astype(np.uint64)
        self.at = 0

    def below(self, n: int) -> int:
        v = int(self.values[self.at % self.values.size])
        self.at += 1
        return v % n

    def chance(self, num: int, den: int) -> bool:
        return self.below(den) < num


def viewed_operand(rng: Stream, lead: tuple, rows: int, cols: int):
    """(owner dims, steps) whose view has the logical shape lead + (rows, cols)."""
    n = len(lead)
    order = list(range(n))
    for i in range(n - 1, 0, -1):                        # Fisher-Yates
        j = rng.below(i + 1)
        order[i], order[j] = order[j], order[i]
    if not rng.chance(1, 2):
        order = list(range(n))
    before = [0] * n                                     # leading shape before the permute
    for i, source in enumerate(order):
        before[source] = lead[i]
    owner, steps = [], []
    for axis, extent in enumerate(before):
        step = 1 + rng.below(3) if rng.chance(1, 2) else 1
        first = rng.below(3) if rng.chance(1, 2) else 0
        spare = rng.below(2)
        owner.append(first + (extent - 1) * step + 1 + spare)
        if first or step != 1 or spare:
            steps.append(("slice", (axis, first, extent, step)))
    # an extra axis that a select removes again (rank stays within 8)
    if n + 2 < 8 and rng.chance(1, 3):
        at = rng.below(n + 1)
        size = 2 + rng.below(2)
        owner.insert(at, size)
        steps = [("select", (at, rng.below(size)))] + steps
    if order != list(range(n)):
        steps.append(("permute", (order,)))
    return tuple(owner) + (rows, cols), steps


def binary_case(case: int, max_lead: int = 3, max_extent: int = 4, salt: int = 101):
    """(result lead, rows, cols, [lhs, rhs, out]) with lhs/rhs/out = (owner dims, steps)."""
    rng = Stream(case, salt)
    nlead = rng.below(max_lead + 1)
    lead = tuple(1 + rng.below(max_extent) for _ in range(nlead))
    rows = (1, 5, 15, 16, 17, 33, 32, 48)[rng.below(8)]
    cols = (1, 7, 16, 17, 31, 48, 256, 1040)[rng.below(8)]
    # every axis of the result is held in full by at least one input (the output shape is
    # exactly the broadcast of the two); the other input may have extent 1 there
    shape = lead + (rows, cols)
    held = [[d, d] for d in shape]
    for axis in range(len(shape)):
        pick = rng.below(4)                              # 0, 1: both in full; 2: lhs is 1; 3: rhs is 1
        if pick >= 2:
            held[axis][pick - 2] = 1
    operands = []
    shorter = rng.below(2)                               # the one input that may have a lower rank
    for k in range(2):
        dims = [h[k] for h in held]
        # leading axes of extent 1 at the front may be dropped: a right-aligned input of lower rank
        drop = 0
        while k == shorter and drop < nlead and dims[drop] == 1 and rng.chance(1, 2):
            drop += 1
        dims = dims[drop:]
        operands.append(viewed_operand(rng, tuple(dims[:-2]), dims[-2], dims[-1]))
    operands.append(viewed_operand(rng, lead, rows, cols))
    return lead, rows, cols, operands


def unary_case(case: int, salt: int = 202):
    """(lead, rows, cols, [source, destination]) of identical logical shape."""
    rng = Stream(case, salt)
    nlead = rng.below(4)
    lead = tuple(1 + rng.below(4) for _ in range(nlead))
    rows = (1, 5, 15, 16, 17, 33, 32, 48)[rng.below(8)]
    cols = (2, 8, 16, 18, 32, 48, 256, 1040)[rng.below(8)]
    return lead, rows, cols, [viewed_operand(rng, lead, rows, cols), viewed_operand(rng, lead, rows, cols)]


def apply(view, steps):
    for name, args in steps:
        view = getattr(view, name)(*args)
    return view
