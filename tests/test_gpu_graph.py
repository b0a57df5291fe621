"""A recorded sequence of launches replays to the same bits as the eager sequence.

The sequence is a small decode step (rmsnorm, projection, rope, cache append, attention,
residual add) recorded once on a stream and replayed several times; between replays the
inputs are changed by ordinary eager work and the stream is synchronised, and every replay
is compared with the eager result for the same inputs.
"""
import numpy as np
import pytest

import datagen
from iom_amd import iomx
from iomo import DT_BF16

pytestmark = pytest.mark.gpu
ADD = 0


def test_recorded_decode_step_replays_to_the_eager_result():
    assert iomx.device_count() >= 1
    iomx.check(iomx.lib().iomx_set_device(0))
    B, H, Hq, Hkv, D, C, a = 4, 128, 4, 2, 32, 48, 20
    st = iomx.Stream()
    rnd = lambda n, s, sd=1.0: datagen.bf16_rne(datagen.normal_f32(n, 0, sd, s))
    x = iomx.DeviceTensor(DT_BF16, (B, 1, H))
    wn = iomx.DeviceTensor(DT_BF16, (1, H)); wn.view().from_host(rnd(H, 1).reshape(1, H))
    wq = iomx.DeviceTensor(DT_BF16, (Hq * D, H)); wq.view().from_host(rnd(Hq * D * H, 2, 0.1).reshape(Hq * D, H))
    wk = iomx.DeviceTensor(DT_BF16, (Hkv * D, H)); wk.view().from_host(rnd(Hkv * D * H, 3, 0.1).reshape(Hkv * D, H))
    kc = iomx.DeviceTensor(DT_BF16, (B, Hkv, C, D)); kc.view().from_host(rnd(B * Hkv * C * D, 4).reshape(B, Hkv, C, D))
    vc = iomx.DeviceTensor(DT_BF16, (B, Hkv, C, D)); vc.view().from_host(rnd(B * Hkv * C * D, 5).reshape(B, Hkv, C, D))
    n1 = iomx.DeviceTensor(DT_BF16, (B, 1, H))
    q, qr = iomx.DeviceTensor(DT_BF16, (B, Hq, 1, D)), iomx.DeviceTensor(DT_BF16, (B, Hq, 1, D))
    k, kr = iomx.DeviceTensor(DT_BF16, (B, Hkv, 1, D)), iomx.DeviceTensor(DT_BF16, (B, Hkv, 1, D))
    attn, out = iomx.DeviceTensor(DT_BF16, (B, 1, Hq * D)), iomx.DeviceTensor(DT_BF16, (B, 1, Hq * D))
    rc, nbytes, _ = iomx.sdpa_workspace(qr.view(), kc.view(), vc.view(), attn.view(), a, a + 1)
    assert rc == 0
    ws = iomx.Buffer(nbytes)

    def step():
        assert iomx.rmsnorm(x.view(), wn.view(), n1.view(), 1e-5, st) == 0
        assert iomx.linear(n1.view(), wq.view(), q.view(), 0, 1, True, Hq, D, 0, st) == 0
        assert iomx.linear(n1.view(), wk.view(), k.view(), 0, 1, True, Hkv, D, 0, st) == 0
        assert iomx.rope(q.view(), qr.view(), a, 10000.0, st) == 0
        assert iomx.rope(k.view(), kr.view(), a, 10000.0, st) == 0
        assert iomx.cache_append(kr.view(), kc.view(), a, st) == 0
        assert iomx.sdpa(qr.view(), kc.view(), vc.view(), attn.view(), a, a + 1, ws, 0, st) == 0
        assert iomx.binary(ADD, attn.view(), attn.view(), out.view(), st) == 0

    x.view().from_host(rnd(B * H, 10).reshape(B, 1, H))
    st.begin_capture()
    step()
    graph = st.end_capture()
    for replay in range(4):
        x.view().from_host(rnd(B * H, 11 + replay).reshape(B, 1, H))     # eager work between replays
        out.view().from_host(np.zeros((B, 1, Hq * D), np.uint16))
        graph.launch(st)
        st.synchronize()
        replayed = out.view().to_host().copy()
        cache_after = kc.view().to_host().copy()
        out.view().from_host(np.zeros((B, 1, Hq * D), np.uint16))
        step()
        st.synchronize()
        assert np.array_equal(out.view().to_host(), replayed), replay
        assert np.array_equal(kc.view().to_host(), cache_after), replay
        assert replayed.any()
    graph.close()
    # capturing needs a stream of its own
    assert iomx.lib().iomx_stream_begin_capture(None) == -1
    for t in (x, wn, wq, wk, kc, vc, n1, q, qr, k, kr, attn, out, ws):
        t.free()
    st.close()


def test_completion_word_arrives_after_the_work_before_it():
    """iomx_stream_write_word: the host polls a page-locked word; once it holds the value,
    everything submitted to the stream before it has finished and its results are visible."""
    import ctypes as C
    import time
    L = iomx.lib()
    iomx.check(L.iomx_set_device(0))
    st = iomx.Stream()
    cells = C.c_void_p()
    iomx.check(L.iomx_host_alloc(C.byref(cells), 64))
    word = C.cast(cells, C.POINTER(C.c_uint32))
    word[0] = 0
    on_device = C.c_void_p()
    iomx.check(L.iomx_host_device_address(cells, C.byref(on_device)))
    dims = (32, 512, 2048)                                  # 64 MiB per operand: tens of microseconds
    n = int(np.prod(dims))
    a, b, o = (iomx.DeviceTensor(DT_BF16, dims) for _ in range(3))
    va = datagen.bf16_rne(datagen.normal_f32(n, 0, 1, 7)).reshape(dims)
    vb = datagen.bf16_rne(datagen.normal_f32(n, 0, 1, 8)).reshape(dims)
    a.view().from_host(va)
    b.view().from_host(vb)
    after_add = iomx.Event(timing=False)
    for ticket in (1, 2, 0xFFFFFFFF):
        o.view().from_host(np.zeros(dims, np.uint16))
        assert iomx.binary(ADD, a.view(), b.view(), o.view(), st) == 0
        after_add.record(st)
        iomx.check(L.iomx_stream_write_word(st.h, on_device, ticket))
        deadline = time.monotonic() + 10.0
        while word[0] != ticket:
            assert time.monotonic() < deadline, "the completion word never arrived"
        # the moment the word is seen, the work before it must already be complete: an event
        # recorded between the ADD and the word reports done without anybody waiting for it
        done = C.c_int(-1)
        iomx.check(L.iomx_event_query(after_add.h, C.byref(done)))
        assert done.value == 1, "the word arrived before the work recorded ahead of it"
        # (the download below runs on the null stream, which does not wait for `st`:
        # iomx_stream_create makes non-blocking streams)
        got = o.buf.download(np.uint16)
        want = iomx.DeviceTensor(DT_BF16, dims)
        assert iomx.binary(ADD, a.view(), b.view(), want.view()) == 0
        assert np.array_equal(got, want.raw())
        want.free()
    # a misaligned or null word is refused before anything is submitted
    assert L.iomx_stream_write_word(st.h, None, 1) == -1
    assert L.iomx_stream_write_word(st.h, C.c_void_p(on_device.value + 2), 1) == -1
    assert L.iomx_host_device_address(None, C.byref(on_device)) == -1
    st.synchronize()
    for t in (a, b, o):
        t.free()
    iomx.check(L.iomx_host_free(cells))
    st.close()
