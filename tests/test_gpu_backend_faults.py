"""Failure paths and native-resource lifecycle of the C++ backend, driven through IOM's own
DeviceOps API with the backend's host-side fault seams (iom_amd/host/mi355x_testing.hpp).

Every fault is injected on the host: a launch that is not made, a status that is replaced.  No
test makes the GPU itself fail.  The cases follow the reference's ROCm conformance and smoke
drivers: a retained launch failure keeps owners reusable
(test/rocm/test_rocm_conformance.cpp:1906-1940), submission stays transactional across failures
before and after acceptance (:1942-2010), a fifth queue is refused before any native resource and
a failed final synchronisation retains the whole queue lease (test/rocm/test_rocm_smoke.cpp:201-296,
362-441), and a workspace dropped while its operation is in flight stays out of the allocator
(src/rocm/device.cpp:243-264)."""
import numpy as np
import pytest

import datagen
import iomo
from iomo import (COUNT_DEVICE_ALLOC, COUNT_DEVICE_FREE, COUNT_EVENT_CREATE, COUNT_EVENT_DESTROY,
                  COUNT_LINEAR_NATIVE, COUNT_LINEAR_SCALAR, COUNT_SILU, COUNT_STREAM_CREATE,
                  COUNT_STREAM_DESTROY, DT_BF16, DT_F32, DT_U8, DT_U16, FAULT_EMBEDDING_STATUS_COPY,
                  FAULT_EVENT_CREATE, FAULT_EVENT_RECORD, FAULT_EVENT_RECORD_UNPROVED, FAULT_KERNEL_LAUNCH, FAULT_NONE,
                  FAULT_QUEUE_EVENT_CREATE, FAULT_QUEUE_STREAM_CREATE, FAULT_SDPA_LAUNCH,
                  FAULT_SILU_LAUNCH, FAULT_STREAM_SYNCHRONIZE, OP_ADD)
from test_oracle_sdpa import random_case, shapes

pytestmark = pytest.mark.gpu

C_IN_FLIGHT = 4
SEQUENCE_MASK = (1 << 55) - 1          # include/iom/iom.hpp: token = queue id << 55 | sequence


@pytest.fixture()
def gpu():
    if not iomo.mi355x_available():
        pytest.skip("oracle/_ref/libiom_mi355x_shim.so not built (needs the reference headers)")
    dev = iomo.mi355x_backend(arena_bytes=1 << 28, max_in_flight=C_IN_FLIGHT)
    dev.inject(FAULT_NONE)
    yield dev
    dev.inject(FAULT_NONE)
    dev.close()


def expect_repeated_runtime_failure(dev, token):
    """Every wait on the token reports the same retained device error."""
    assert token > 0
    for _ in range(3):
        assert dev.wait(token) == -5, dev.error()
        assert "exception" in dev.error() or "runtime" in dev.error()


def u8_pattern(dims):
    n = int(np.prod(dims))
    return ((np.arange(n) * 3) & 0xFF).astype(np.uint8).reshape(dims)


def test_retained_launch_failure_keeps_owners_reusable(gpu):
    dims = (2, 16, 16)
    lhs, out = gpu.tensor(DT_U8, dims), gpu.tensor(DT_U8, dims)
    pattern = u8_pattern(dims)
    lhs.view().from_host(pattern)
    gpu.inject(FAULT_KERNEL_LAUNCH)
    failed = gpu.submit("binary", OP_ADD, lhs.view(), lhs.view(), out.view())
    expect_repeated_runtime_failure(gpu, failed)
    gpu.inject(FAULT_NONE)
    recovered = gpu.submit("binary", OP_ADD, lhs.view(), lhs.view(), out.view())
    assert recovered > 0 and gpu.wait(recovered) == 0, gpu.error()
    assert np.array_equal(out.view().to_host(), (pattern.astype(np.uint16) * 2 & 0xFF).astype(np.uint8))
    assert gpu.wait(failed) == -5                      # the failure stays retained
    assert gpu.snapshot() == (C_IN_FLIGHT, 0, 0)
    lhs.close(); out.close()


def test_submission_stays_transactional_across_failures_before_and_after_acceptance(gpu):
    src, dst = gpu.tensor(DT_U8, (3, 16, 16)), gpu.tensor(DT_U8, (3, 16, 16))
    wrong = gpu.tensor(DT_U8, (3, 16, 17))
    fill = np.full((3, 16, 16), 0x3C, np.uint8)
    src.view().from_host(fill)
    dst.view().from_host(fill)
    assert gpu.submit("copy", src.view(), wrong.view()) == -1          # rejected: no sequence used
    first = gpu.submit("copy", src.view(), dst.view())
    assert first & SEQUENCE_MASK == 1 and gpu.wait(first) == 0
    gpu.inject(FAULT_EVENT_CREATE)                                      # fails before acceptance
    assert gpu.submit("copy", src.view(), dst.view()) == -5
    second = gpu.submit("copy", src.view(), dst.view())
    assert second & SEQUENCE_MASK == 2 and gpu.wait(second) == 0
    gpu.inject(FAULT_KERNEL_LAUNCH)                                     # fails after acceptance
    third = gpu.submit("copy", src.view(), dst.view())
    assert third & SEQUENCE_MASK == 3
    expect_repeated_runtime_failure(gpu, third)
    gpu.inject(FAULT_EVENT_RECORD)
    fourth = gpu.submit("copy", src.view(), dst.view())
    assert fourth & SEQUENCE_MASK == 4
    expect_repeated_runtime_failure(gpu, fourth)
    gpu.inject(FAULT_NONE)
    fifth = gpu.submit("copy", src.view(), dst.view())
    assert fifth & SEQUENCE_MASK == 5 and gpu.wait(fifth) == 0
    assert np.array_equal(dst.view().to_host(), fill)
    assert gpu.snapshot() == (C_IN_FLIGHT, 0, 0)                         # every event came back
    for t in (src, dst, wrong):
        t.close()


def test_accepted_failures_of_silu_attention_and_the_embedding_status_copy(gpu):
    x = gpu.tensor(DT_BF16, (33, 64))
    y = gpu.tensor(DT_BF16, (33, 64))
    x.view().from_host(datagen.bf16_rne(datagen.normal_f32(33 * 64, 0, 1, 3)).reshape(33, 64))
    before = gpu.counter(COUNT_SILU)
    gpu.inject(FAULT_SILU_LAUNCH)
    failed = gpu.submit("silu", x.view(), y.view())
    expect_repeated_runtime_failure(gpu, failed)
    assert gpu.counter(COUNT_SILU) == before                            # never reached the kernel
    ok = gpu.submit("silu", x.view(), y.view())
    assert gpu.wait(ok) == 0 and gpu.counter(COUNT_SILU) == before + 1
    # attention: the request and its workspace lease are accepted, then the launch fails
    case = random_case(7, (), 4, 2, 20, 32, 40, 5, 25)
    qd, kd, od = shapes(case)
    t = [gpu.tensor(DT_BF16, d) for d in (qd, kd, kd, od)]
    for tensor, name, d in zip(t, "qkv", (qd, kd, kd)):
        tensor.view().from_host(np.array(case[name], np.uint16).reshape(d))
    need = gpu.sdpa_workspace_bytes(t[0].view(), t[1].view(), t[2].view(), t[3].view(), 5, 25)
    assert need > 0
    ws = gpu.workspace(need)
    gpu.inject(FAULT_SDPA_LAUNCH)
    failed = gpu.sdpa_submit(t[0].view(), t[1].view(), t[2].view(), t[3].view(), 5, 25, ws)
    expect_repeated_runtime_failure(gpu, failed)
    ok = gpu.sdpa_submit(t[0].view(), t[1].view(), t[2].view(), t[3].view(), 5, 25, ws)   # lease released
    assert ok > 0 and gpu.wait(ok) == 0, gpu.error()
    gpu.drop_workspace(ws)
    # embedding: the gather was launched, the copy of its status word failed
    table, ids, out = gpu.tensor(DT_F32, (37, 48)), gpu.tensor(DT_U16, (1, 9)), gpu.tensor(DT_F32, (9, 48))
    table.view().from_host(datagen.pattern_bits(32, 37 * 48, 1).reshape(37, 48))
    ids.view().from_host((np.arange(9) * 4 % 37).astype(np.uint16).reshape(1, 9))
    ws = gpu.workspace(gpu.embedding_workspace_bytes(table.view(), ids.view(), out.view()))
    gpu.inject(FAULT_EMBEDDING_STATUS_COPY)
    failed = gpu.embedding_submit(table.view(), ids.view(), out.view(), ws)
    expect_repeated_runtime_failure(gpu, failed)
    ok = gpu.embedding_submit(table.view(), ids.view(), out.view(), ws)
    assert ok > 0 and gpu.wait(ok) == 0
    gpu.drop_workspace(ws)
    assert gpu.snapshot() == (C_IN_FLIGHT, 0, 0)
    for tensor in (x, y, table, ids, out, *t):
        tensor.close()


def test_linear_counters_connect_an_accepted_oid_to_the_kernel_that_ran(gpu):
    x, w, o = gpu.tensor(DT_BF16, (40, 64)), gpu.tensor(DT_BF16, (48, 64)), gpu.tensor(DT_BF16, (40, 48))
    native, scalar = gpu.counter(COUNT_LINEAR_NATIVE), gpu.counter(COUNT_LINEAR_SCALAR)
    assert gpu.linear(x.view(), w.view(), o.view(), 0, 40, False, 1, 48) > 0
    assert (gpu.counter(COUNT_LINEAR_NATIVE), gpu.counter(COUNT_LINEAR_SCALAR)) == (native + 1, scalar)
    xf, wf, of = gpu.tensor(DT_F32, (40, 64)), gpu.tensor(DT_F32, (48, 64)), gpu.tensor(DT_F32, (40, 48))
    assert gpu.linear(xf.view(), wf.view(), of.view(), 0, 40, False, 1, 48) > 0
    assert (gpu.counter(COUNT_LINEAR_NATIVE), gpu.counter(COUNT_LINEAR_SCALAR)) == (native + 1, scalar + 1)
    for t in (x, w, o, xf, wf, of):
        t.close()


def test_one_device_allocation_and_eager_queue_resources(gpu):
    """The arena is the only device allocation; a queue creates its C events and its stream at
    construction; the fifth queue is refused before it creates anything; a failure in the
    middle of construction unwinds what was created."""
    allocs, frees = gpu.counter(COUNT_DEVICE_ALLOC), gpu.counter(COUNT_DEVICE_FREE)
    events, streams = gpu.counter(COUNT_EVENT_CREATE), gpu.counter(COUNT_STREAM_CREATE)
    tensors = [gpu.tensor(DT_F32, (64, 64)) for _ in range(8)]
    queues = [gpu.second_queue() for _ in range(3)]                      # four live with the fixture's
    assert gpu.counter(COUNT_DEVICE_ALLOC) == allocs and gpu.counter(COUNT_DEVICE_FREE) == frees
    assert gpu.counter(COUNT_EVENT_CREATE) == events + 3 * C_IN_FLIGHT
    assert gpu.counter(COUNT_STREAM_CREATE) == streams + 3
    for q in queues:
        assert q.snapshot() == (C_IN_FLIGHT, 0, 0)
    with pytest.raises(RuntimeError, match="bad_alloc"):
        gpu.second_queue()
    assert gpu.counter(COUNT_EVENT_CREATE) == events + 3 * C_IN_FLIGHT   # nothing was created
    assert gpu.counter(COUNT_STREAM_CREATE) == streams + 3
    destroyed = gpu.counter(COUNT_EVENT_DESTROY), gpu.counter(COUNT_STREAM_DESTROY)
    queues.pop().close()
    assert gpu.counter(COUNT_EVENT_DESTROY) == destroyed[0] + C_IN_FLIGHT
    assert gpu.counter(COUNT_STREAM_DESTROY) == destroyed[1] + 1
    for fault in (FAULT_QUEUE_EVENT_CREATE, FAULT_QUEUE_STREAM_CREATE):
        made = gpu.counter(COUNT_EVENT_CREATE) - gpu.counter(COUNT_EVENT_DESTROY)
        live_streams = gpu.counter(COUNT_STREAM_CREATE) - gpu.counter(COUNT_STREAM_DESTROY)
        gpu.inject(fault)
        with pytest.raises(RuntimeError):
            gpu.second_queue()
        assert gpu.counter(COUNT_EVENT_CREATE) - gpu.counter(COUNT_EVENT_DESTROY) == made
        assert gpu.counter(COUNT_STREAM_CREATE) - gpu.counter(COUNT_STREAM_DESTROY) == live_streams
    again = gpu.second_queue()                                            # the slot was given back
    again.close()
    for q in queues:
        q.close()
    for t in tensors:
        t.close()


def test_attention_keeps_its_workspace_leased_until_the_token_is_observed(gpu):
    """test/backend/backend_conformance_sdpa.hpp:562-626: a second accepted use of the same live
    range is exhaustion (-4) until the caller has waited for the first -- also when the first has
    long finished on the device -- and a queue that goes away releases what nobody observed."""
    import time
    case = random_case(23, (), 4, 2, 40, 32, 48, 3, 43)
    qd, kd, od = shapes(case)
    t = [gpu.tensor(DT_BF16, d) for d in (qd, kd, kd, od)]
    for tensor, name, d in zip(t, "qkv", (qd, kd, kd)):
        tensor.view().from_host(np.array(case[name], np.uint16).reshape(d))
    views = [x.view() for x in t]
    need = gpu.sdpa_workspace_bytes(*views, 3, 43)
    assert need > 0
    ws = gpu.workspace(need)
    first = gpu.sdpa_submit(*views, 3, 43, ws)
    assert first > 0
    assert gpu.sdpa_submit(*views, 3, 43, ws) == -4            # while it may still run
    time.sleep(0.05)                                            # finished by now, not yet observed
    assert gpu.snapshot() == (C_IN_FLIGHT, 0, 0)
    assert gpu.sdpa_submit(*views, 3, 43, ws) == -4
    assert gpu.wait(first) == 0 and gpu.wait(first) == 0
    want = t[3].view().to_host()
    again = gpu.sdpa_submit(*views, 3, 43, ws)                  # observed: the range is free again
    assert again > 0 and gpu.wait(again) == 0, gpu.error()
    assert np.array_equal(t[3].view().to_host(), want)
    # never observed: the queue's end releases it
    other = gpu.second_queue()
    unseen = other.sdpa_submit(*views, 3, 43, ws)
    assert unseen > 0
    time.sleep(0.05)
    assert gpu.sdpa_submit(*views, 3, 43, ws) == -4
    other.close()
    last = gpu.sdpa_submit(*views, 3, 43, ws)
    assert last > 0 and gpu.wait(last) == 0, gpu.error()
    gpu.drop_workspace(ws)
    for x in t:
        x.close()


def test_a_failed_final_synchronisation_retains_the_whole_queue_lease(gpu):
    a, b = gpu.tensor(DT_F32, (32, 32)), gpu.tensor(DT_F32, (32, 32))
    doomed = gpu.second_queue()
    # double fault: the event record fails, so the submission retires with a retained failure,
    # and then the covering synchronisation at destruction fails too
    gpu.inject(FAULT_EVENT_RECORD)
    unresolved = doomed.submit("copy", a.view(), b.view())
    assert unresolved > 0 and doomed.wait(unresolved) == -5
    destroyed = gpu.counter(COUNT_EVENT_DESTROY), gpu.counter(COUNT_STREAM_DESTROY)
    gpu.inject(FAULT_STREAM_SYNCHRONIZE)
    doomed.close()
    gpu.inject(FAULT_NONE)
    assert gpu.retained_leases() == 1
    assert (gpu.counter(COUNT_EVENT_DESTROY), gpu.counter(COUNT_STREAM_DESTROY)) == destroyed
    # two more queues fit beside the fixture's; live plus retained leases exhaust the four places
    others = [gpu.second_queue() for _ in range(2)]
    with pytest.raises(RuntimeError, match="bad_alloc"):
        gpu.second_queue()
    assert gpu.retained_leases() == 1
    # a live queue that drains properly gives its place back; the retained one does not
    others.pop().close()
    replacement = gpu.second_queue()
    with pytest.raises(RuntimeError, match="bad_alloc"):
        gpu.second_queue()
    # a proof that fails again keeps the lease; a covering proof on the same stream reclaims it
    gpu.inject(FAULT_STREAM_SYNCHRONIZE)
    gpu.reclaim_leases()
    assert gpu.retained_leases() == 1
    gpu.reclaim_leases()
    assert gpu.retained_leases() == 0
    assert gpu.counter(COUNT_EVENT_DESTROY) == destroyed[0] + 2 * C_IN_FLIGHT    # doomed's and the drained one's
    assert gpu.counter(COUNT_STREAM_DESTROY) == destroyed[1] + 2
    reclaimed = gpu.second_queue()
    token = reclaimed.submit("copy", a.view(), b.view())
    assert token > 0 and reclaimed.wait(token) == 0
    for q in (reclaimed, replacement, *others):
        q.close()
    a.close(); b.close()


def test_a_workspace_dropped_before_the_wait_stays_out_of_the_allocator(gpu):
    """Attention keeps packed K / V in its workspace while it runs.  The caller drops the
    workspace owner right after submission: the range is quarantined, the next tensor does not
    get it (and is not zero-filled over the running kernel's data), and the result is the one a
    patient caller gets."""
    case = random_case(17, (2,), 8, 2, 300, 64, 320, 10, 310)
    qd, kd, od = shapes(case)
    t = [gpu.tensor(DT_BF16, d) for d in (qd, kd, kd, od)]
    for tensor, name, d in zip(t, "qkv", (qd, kd, kd)):
        tensor.view().from_host(np.array(case[name], np.uint16).reshape(d))
    views = [x.view() for x in t]
    need = gpu.sdpa_workspace_bytes(*views, 10, 310)
    assert need > 0
    patient = gpu.workspace(need)
    token = gpu.sdpa_submit(*views, 10, 310, patient)
    assert token > 0 and gpu.wait(token) == 0
    want = t[3].view().to_host()
    gpu.drop_workspace(patient)
    t[3].view().from_host(np.zeros(od, np.uint16))
    # where does a workspace of this size land?  (the arena hands out the first fit)
    probe = gpu.tensor(DT_U8, (need // 256, 16, 16))
    address = gpu.l.iomc_view_native_handle(probe.view().h)
    probe.close()
    hasty = gpu.workspace(need)
    token = gpu.sdpa_submit(*views, 10, 310, hasty)
    assert token > 0
    gpu.drop_workspace(hasty)                                             # before the wait
    successor = gpu.tensor(DT_U8, (need // 256, 16, 16))                  # zero-filled at creation
    assert gpu.l.iomc_view_native_handle(successor.view().h) != address
    assert gpu.wait(token) == 0, gpu.error()
    assert np.array_equal(t[3].view().to_host(), want)
    assert not successor.view().to_host().any()
    successor.close()
    for x in t:
        x.close()


def test_a_failed_submission_without_proof_of_completion_keeps_its_workspace_range(gpu):
    """The completion event of an accepted attention request cannot be recorded, and the stream
    synchronisation that would still prove the kernel finished fails as well: the operation
    retires as failed, and its workspace range -- which the kernel may still be writing for all
    the host knows -- is never handed out again.  With the proof (the plain event_record fault)
    the range returns to the allocator."""
    case = random_case(19, (2,), 8, 2, 300, 64, 320, 10, 310)
    qd, kd, od = shapes(case)
    t = [gpu.tensor(DT_BF16, d) for d in (qd, kd, kd, od)]
    for tensor, name, d in zip(t, "qkv", (qd, kd, kd)):
        tensor.view().from_host(np.array(case[name], np.uint16).reshape(d))
    views = [x.view() for x in t]
    need = gpu.sdpa_workspace_bytes(*views, 10, 310)
    assert need > 0

    def first_fit():
        probe = gpu.tensor(DT_U8, (need // 256, 16, 16))
        address = gpu.l.iomc_view_native_handle(probe.view().h)
        probe.close()
        return address

    # proved: the failed operation's range is free again once its owner goes away
    address = first_fit()
    ws = gpu.workspace(need)
    gpu.inject(FAULT_EVENT_RECORD)
    token = gpu.sdpa_submit(*views, 10, 310, ws)
    assert token > 0 and gpu.wait(token) == -5
    gpu.drop_workspace(ws)
    assert first_fit() == address
    # unproved: the same range stays out of the allocator
    ws = gpu.workspace(need)
    gpu.inject(FAULT_EVENT_RECORD_UNPROVED)
    token = gpu.sdpa_submit(*views, 10, 310, ws)
    gpu.inject(FAULT_NONE)
    assert token > 0 and gpu.wait(token) == -5
    assert gpu.wait(token) == -5                                          # the failure repeats
    gpu.drop_workspace(ws)
    assert first_fit() != address
    # the queue goes on working, with a workspace elsewhere in the arena
    ws = gpu.workspace(need)
    token = gpu.sdpa_submit(*views, 10, 310, ws)
    assert token > 0 and gpu.wait(token) == 0, gpu.error()
    gpu.drop_workspace(ws)
    for x in t:
        x.close()
