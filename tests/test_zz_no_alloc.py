"""GPU test of iomx_launch_sdpa_static, the attention entry point that allocates nothing:
its workspace is the library's fixed per-GPU array instead of a caller buffer.

Every case runs the existing entry point (iomx_launch_sdpa with a freshly allocated,
poisoned workspace) and the new one on the same operands and asks for the same bits.  Calls
come in rows -- a large request first, then smaller ones that reuse the array with the earlier
call's contents still in it -- and cover both uses of the workspace: the packed K / V of a
prefill and the shares' statistics of a decode step against a long prefix.
"""
import numpy as np
import pytest

import iomo
from iom_amd import iomx
from iomo import DT_BF16
from test_oracle_sdpa import random_case, shapes

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    assert iomx.device_count() >= 1
    iomx.check(iomx.lib().iomx_set_device(0))
    yield


def operands(case, fill=0x5A):
    qd, kd, od = shapes(case)
    t = [iomx.DeviceTensor(DT_BF16, d, fill=fill) for d in (qd, kd, kd, od)]
    t[0].view().from_host(np.array(case["q"], np.uint16).reshape(qd))
    t[1].view().from_host(np.array(case["k"], np.uint16).reshape(kd))
    t[2].view().from_host(np.array(case["v"], np.uint16).reshape(kd))
    return t


def with_caller_workspace(case, path=0):
    """Raw output storage from iomx_launch_sdpa, and the workspace bytes it asked for."""
    q, k, v, o = operands(case)
    rc, nbytes, _ = iomx.sdpa_workspace(q.view(), k.view(), v.view(), o.view(), case["a"], case["L"])
    assert rc == 0
    ws = iomx.Buffer(nbytes) if nbytes and path == 0 else None
    if ws:
        ws.fill(0xEE)
    iomx.check(iomx.sdpa(q.view(), k.view(), v.view(), o.view(), case["a"], case["L"], ws, path), "sdpa")
    iomx.synchronize()
    kernel = iomx.last_launch().kernel.decode()
    raw = o.raw().copy()
    for t in (q, k, v, o):
        t.free()
    if ws:
        ws.free()
    return raw, nbytes, kernel


def with_static_scratch(case, path=0):
    q, k, v, o = operands(case)
    iomx.check(iomx.sdpa_static(q.view(), k.view(), v.view(), o.view(), case["a"], case["L"], path),
               "sdpa_static")
    iomx.synchronize()
    kernel = iomx.last_launch().kernel.decode()
    raw = o.raw().copy()
    for t in (q, k, v, o):
        t.free()
    return raw, kernel


# (leading, Hq, Hkv, R, D, C, a, L): a large request, then smaller ones on the same array
PREFILL_ROW = [((2,), 8, 2, 300, 64, 320, 10, 310), ((), 4, 4, 33, 128, 64, 10, 43),
               ((), 8, 2, 40, 64, 100, 50, 90), ((2,), 4, 2, 17, 16, 40, 20, 37)]
DECODE_ROW = [((3,), 16, 2, 2, 128, 2100, 2050, 2052), ((), 8, 2, 1, 64, 2200, 2199, 2200)]


def test_prefill_calls_in_a_row_each_smaller_than_the_last():
    used = []
    for i, spec in enumerate(PREFILL_ROW):
        case = random_case(300 + i, *spec)
        want, nbytes, kernel = with_caller_workspace(case)
        got, kernel_static = with_static_scratch(case)
        assert kernel == kernel_static == "sdpa_mfma"
        assert 0 < nbytes <= iomx.SDPA_STATIC_BYTES
        assert np.array_equal(got, want), spec
        used.append(nbytes)
    assert used == sorted(used, reverse=True) and used[0] > used[-1]


def test_decode_steps_in_shares_then_a_prefill_on_the_same_array():
    for i, spec in enumerate(DECODE_ROW):
        case = random_case(400 + i, *spec)
        want, nbytes, kernel = with_caller_workspace(case)
        got, kernel_static = with_static_scratch(case)
        assert kernel == kernel_static == "sdpa_decode" and nbytes > 0
        assert np.array_equal(got, want), spec
    case = random_case(410, *PREFILL_ROW[2])
    want, _, _ = with_caller_workspace(case)
    got, _ = with_static_scratch(case)
    assert np.array_equal(got, want)


def test_requests_that_need_no_workspace():
    """A short decode step and the reference-order path keep nothing outside their operands."""
    case = random_case(420, (2,), 8, 2, 1, 64, 70, 69, 70)
    want, nbytes, kernel = with_caller_workspace(case)
    got, kernel_static = with_static_scratch(case)
    assert nbytes == 0 and kernel == kernel_static == "sdpa_decode"
    assert np.array_equal(got, want)
    case = random_case(421, *PREFILL_ROW[3])
    want, _, kernel = with_caller_workspace(case, path=1)
    got, kernel_static = with_static_scratch(case, path=1)
    assert kernel == kernel_static == "sdpa_rows"
    assert np.array_equal(got, want)


def test_a_request_beyond_the_array_is_rejected_before_any_launch():
    # one sequence, 32 KV heads of 128 features, 4096 tokens: 2 x 32 MiB of packed K and V
    dims_q, dims_kv, dims_o = (32, 17, 128), (32, 4096, 128), (17, 32 * 128)
    q, k, v, o = (iomx.DeviceTensor(DT_BF16, d, fill=0x3C) for d in (dims_q, dims_kv, dims_kv, dims_o))
    rc, nbytes, _ = iomx.sdpa_workspace(q.view(), k.view(), v.view(), o.view(), 4000, 4017)
    assert rc == 0 and nbytes > iomx.SDPA_STATIC_BYTES
    before = o.raw().copy()
    rc = iomx.sdpa_static(q.view(), k.view(), v.view(), o.view(), 4000, 4017)
    assert rc == -4 and b"scratch" in iomx.lib().iomx_error_string(rc)
    iomx.synchronize()
    assert np.array_equal(o.raw(), before)
    # invalid requests keep their own classes
    assert iomx.sdpa_static(q.view(), k.view(), v.view(), o.view(), 4000, 5000) == -1
    for t in (q, k, v, o):
        t.free()


def test_captured_into_a_graph_after_an_eager_call_and_replayed():
    """One eager call first (it looks the array's address up), then the entry point recorded into a
    graph on a stream of its own and replayed twice, with eager work on the same array and a
    synchronisation between the replays: every replay gives the bits of iomx_launch_sdpa."""
    spec = PREFILL_ROW[2]
    case = random_case(430, *spec)
    want, _, _ = with_caller_workspace(case)
    got, _ = with_static_scratch(case)                       # the eager call
    assert np.array_equal(got, want)
    q, k, v, o = operands(case)
    st = iomx.Stream()
    st.begin_capture()
    rc = iomx.sdpa_static(q.view(), k.view(), v.view(), o.view(), case["a"], case["L"], 0, st)
    graph = st.end_capture()
    assert rc == 0
    other = random_case(431, *PREFILL_ROW[1])
    for replay in range(2):
        o.buf.fill(0x5A)
        iomx.synchronize()
        graph.launch(st)
        st.synchronize()
        assert np.array_equal(o.raw(), want), replay
        # eager work that overwrites the array between the replays
        got_other, _ = with_static_scratch(other)
        want_other, _, _ = with_caller_workspace(other)
        assert np.array_equal(got_other, want_other)
    graph.close()
    st.close()
    for t in (q, k, v, o):
        t.free()
