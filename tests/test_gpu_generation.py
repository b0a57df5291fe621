"""Greedy generation with a whole (small) TinyLlama-shaped model through IOM's DeviceOps API on
the MI355X backend, next to the reference CPU backend in the same process: the forward pass in
the session's order (src/session.cpp:3430-3515: token ids to the device, embedding lookup, the
decoder layers, the final normalisation over the run, the output projection of the last row
into the [1,V] logits) and the host-side greedy rule (src/token_selection.cpp:133-154: the
first largest BF16 logit, non-finite logits refused), a prefill and then decode steps against
the growing caches.

Three layers at the width of tests/test_gpu_decoder_layer.py (hidden 128, 4 query / 2 KV heads
of 32 features, FFN 352), vocabulary 320, BF16, random-init weights.  The CPU backend generates;
the MI355X backend is fed the same tokens, so both see the same context at every step, and is
held to two things per step: its logits lie within the end-to-end distance that the rounding of
fifty-odd operations allows, and the token it would select is the CPU's or one whose CPU logit
is within two BF16 steps of the CPU's largest (a tie that rounding may break either way).
"""
import numpy as np
import pytest

import datagen
import iomo
from iomo import DT_BF16, DT_U32

from test_gpu_decoder_layer import CAP, D, EPS, FF, HID, HKV, HQ, Layer, bf16, f64, steps, submit

pytestmark = pytest.mark.gpu

LAYERS, VOCAB = 3, 320


@pytest.fixture(scope="module")
def devices():
    if not iomo.mi355x_available():
        pytest.skip("oracle/_ref/libiom_mi355x_shim.so not built (needs the reference headers)")
    gpu = iomo.mi355x_backend(arena_bytes=1 << 28, max_in_flight=4)
    cpu = iomo.cpu_backend_beside_mi355x()
    yield cpu, gpu
    gpu.close()
    cpu.close()


def layer_weights(index):
    def mat(rows, cols, seed):
        return bf16(datagen.normal_f32(rows * cols, 0.0, 1.0, 100 * index + seed) / np.sqrt(cols)).reshape(rows, cols)
    return {
        "attn_scale": bf16(datagen.uniform_f32(HID, 0.5, 1.5, 100 * index + 11)).reshape(1, HID),
        "post_scale": bf16(datagen.uniform_f32(HID, 0.5, 1.5, 100 * index + 12)).reshape(1, HID),
        "wq": mat(HQ * D, HID, 13), "wk": mat(HKV * D, HID, 14), "wv": mat(HKV * D, HID, 15),
        "wo": mat(HID, HQ * D, 16), "wg": mat(FF, HID, 17), "wu": mat(FF, HID, 18), "wd": mat(HID, FF, 19),
    }


class Model:
    """Weights and caches of the model on one device; forward() is one run of the session."""

    def __init__(self, dev):
        self.dev = dev
        self.layers = [Layer(dev, layer_weights(i)) for i in range(LAYERS)]
        self.fixed = {}
        for name, value in (("table", bf16(datagen.normal_f32(VOCAB * HID, 0.0, 1.0, 901)).reshape(VOCAB, HID)),
                            ("final_scale", bf16(datagen.uniform_f32(HID, 0.5, 1.5, 902)).reshape(1, HID)),
                            ("head", bf16(datagen.normal_f32(VOCAB * HID, 0.0, 1.0, 903) / np.sqrt(HID)).reshape(VOCAB, HID))):
            self.fixed[name] = dev.tensor(DT_BF16, value.shape)
            self.fixed[name].view().from_host(value)
        self.logits = dev.tensor(DT_BF16, (1, VOCAB))

    def forward(self, ids, a):
        """Logits [V] (BF16 bits) of the last of the rows `ids` placed at positions a.."""
        dev, R = self.dev, len(ids)
        tokens = dev.tensor(DT_U32, (1, 1, R))
        tokens.view().from_host(np.asarray(ids, np.uint32).reshape(1, 1, R))
        for layer in self.layers:
            layer.rows(R)
        token, status = dev.embedding(self.fixed["table"].view(), tokens.view(), self.layers[0].v("x"))
        assert token > 0 and status == 0, (token, status, dev.error())
        for index, layer in enumerate(self.layers):
            for step in steps(a, R):
                submit(layer, step, R)
            if index + 1 < LAYERS:
                assert dev.copy(layer.v("next"), self.layers[index + 1].v("x")) > 0, dev.error()
        # the session's final-normalisation bank is the [R,F] matrix itself (src/session.cpp:413)
        final = dev.tensor(DT_BF16, (R, HID))
        run = self.layers[-1].v("next").select(0, 0)
        assert dev.rmsnorm(run, self.fixed["final_scale"].view(), final.view(), EPS) > 0, dev.error()
        assert dev.linear(final.view(), self.fixed["head"].view(), self.logits.view(), R - 1, 1, False, 1, VOCAB) > 0, \
            dev.error()
        tokens.close()
        final.close()
        return self.logits.view().to_host().reshape(-1)

    def close(self):
        for layer in self.layers:
            layer.close()
        for tensor in self.fixed.values():
            tensor.close()
        self.logits.close()


def greedy(logits):
    """src/token_selection.cpp:133-154."""
    assert not ((logits & 0x7F80) == 0x7F80).any()
    return int(np.argmax(datagen.bf16_to_f32(logits)))          # the first of equal maxima


def ordered(bits):
    bits = bits.astype(np.int64)
    return np.where(bits & 0x8000, -(bits & 0x7FFF), bits)


def test_greedy_generation_follows_the_reference_cpu_backend(devices):
    cpu, gpu = devices
    reference, candidate = Model(cpu), Model(gpu)
    prompt = [int(v) for v in datagen.pattern_bits(32, 48, 77) % VOCAB]
    generated, same_choice, report = [], 0, []
    ids, a = prompt, 0
    for step in range(9):
        want = reference.forward(ids, a)
        got = candidate.forward(ids, a)
        w, g = f64(want), f64(got)
        rms = np.sqrt(np.mean(w * w))
        assert np.abs(g - w).max() <= 2.0 ** -3 * rms, (step, float(np.abs(g - w).max() / rms))
        chosen, would = greedy(want), greedy(got)
        # the candidate's choice is the reference's, or a token the reference scored within two
        # BF16 steps of its largest
        assert ordered(want)[chosen] - ordered(want)[would] <= 2, (step, chosen, would)
        same_choice += chosen == would
        report.append((step, len(ids), chosen, would, float(np.abs(g - w).max() / rms)))
        generated.append(chosen)
        a += len(ids)
        ids = [chosen]
    print()
    for step, rows, chosen, would, rel in report:
        print(f"  step {step}: {rows:2d} rows  reference token {chosen:3d}  candidate token {would:3d}  "
              f"max |logit difference| / rms {rel:.2e}")
    print(f"  generated {generated}; same greedy choice in {same_choice} of {len(report)} steps")
    assert same_choice >= len(report) - 2
    assert a == len(prompt) + 8 and a <= CAP
    reference.close()
    candidate.close()
