"""One whole decoder layer through IOM's DeviceOps API on the MI355X backend, next to the
reference CPU backend in the same process: the session's own order of operations
(src/session.cpp:2842-2879 normalisation, Q / K / V projections, rotations; :2451-2503 cache
appends, attention, output projection, first residual; :1996-2046 second normalisation, gate /
up, SiLU, product, down projection, second residual), a prefill of 512 rows and then two
decode steps against the growing cache.

TinyLlama's architecture at a width the scalar CPU backend finishes in seconds (hidden 128,
4 query / 2 KV heads of 32 features, FFN 352; BF16, random-init weights).  Two comparisons:

* per operation: the CPU backend repeats every operation on the inputs the GPU operation had,
  and the two outputs are held to that operation's own bar -- bit-exact for add / mul / cache
  append, 1 BF16 ulp for RMSNorm and SiLU, the contract's native-BF16 bound for the
  projections, the reference's rotation rule for RoPE, the float64 budget for attention;
* end to end: the CPU backend runs the whole layer on its own intermediates; the distance of
  the two layer outputs is reported (max ulp, mismatch count) and bounded.
"""
import numpy as np
import pytest

import datagen
import iomo
from iomo import DT_BF16, OP_ADD, OP_MUL

pytestmark = pytest.mark.gpu

HID, HQ, HKV, D, FF, CAP = 128, 4, 2, 32, 352, 528
THETA, EPS = 10000.0, 1e-5


@pytest.fixture(scope="module")
def devices():
    if not iomo.mi355x_available():
        pytest.skip("oracle/_ref/libiom_mi355x_shim.so not built (needs the reference headers)")
    gpu = iomo.mi355x_backend(arena_bytes=1 << 28, max_in_flight=4)
    cpu = iomo.cpu_backend_beside_mi355x()
    yield cpu, gpu
    gpu.close()
    cpu.close()


def bf16(values):
    return datagen.bf16_rne(np.ascontiguousarray(values, dtype=np.float32).reshape(-1))


def f64(bits):
    return datagen.bf16_to_f32(np.ascontiguousarray(bits).reshape(-1)).astype(np.float64).reshape(bits.shape)


def weights():
    def mat(rows, cols, seed):
        return bf16(datagen.normal_f32(rows * cols, 0.0, 1.0, seed) / np.sqrt(cols)).reshape(rows, cols)
    return {
        "attn_scale": bf16(datagen.uniform_f32(HID, 0.5, 1.5, 11)).reshape(1, HID),
        "post_scale": bf16(datagen.uniform_f32(HID, 0.5, 1.5, 12)).reshape(1, HID),
        "wq": mat(HQ * D, HID, 13), "wk": mat(HKV * D, HID, 14), "wv": mat(HKV * D, HID, 15),
        "wo": mat(HID, HQ * D, 16), "wg": mat(FF, HID, 17), "wu": mat(FF, HID, 18), "wd": mat(HID, FF, 19),
    }


class Layer:
    """The layer's tensors on one device, and the session's sequence of submissions."""

    def __init__(self, dev, w):
        self.dev = dev
        self.t = {}
        for name, value in w.items():
            self.t[name] = dev.tensor(DT_BF16, value.shape)
            self.t[name].view().from_host(value)
        for name in ("k_cache", "v_cache"):
            self.t[name] = dev.tensor(DT_BF16, (1, HKV, CAP, D))
            self.t[name].view().from_host(np.zeros((1, HKV, CAP, D), np.uint16))

    def rows(self, R):
        shapes = {"x": (1, R, HID), "n1": (1, R, HID), "q": (1, HQ, R, D), "k": (1, HKV, R, D),
                  "v": (1, HKV, R, D), "rq": (1, HQ, R, D), "rk": (1, HKV, R, D),
                  "merged": (1, R, HQ * D), "attn": (1, R, HID), "x2": (1, R, HID), "n2": (1, R, HID),
                  "gate": (1, R, FF), "up": (1, R, FF), "act": (1, R, FF), "prod": (1, R, FF),
                  "down": (1, R, HID), "next": (1, R, HID)}
        for name, dims in shapes.items():
            if name in self.t:
                self.t[name].close()
            self.t[name] = self.dev.tensor(DT_BF16, dims)

    def put(self, name, bits):
        self.t[name].view().from_host(bits)

    def get(self, name):
        return self.t[name].view().to_host()

    def v(self, name):
        return self.t[name].view()

    def close(self):
        for tensor in self.t.values():
            tensor.close()


def steps(a, R):
    """(operation, inputs, output, arguments) in the session's order; L = a + R."""
    return [
        ("rmsnorm", ("x", "attn_scale"), "n1", ()),
        ("linear", ("n1", "wq"), "q", (True, HQ, D)),
        ("linear", ("n1", "wk"), "k", (True, HKV, D)),
        ("linear", ("n1", "wv"), "v", (True, HKV, D)),
        ("rope", ("q",), "rq", (a,)),
        ("rope", ("k",), "rk", (a,)),
        ("cache_append", ("rk",), "k_cache", (a,)),
        ("cache_append", ("v",), "v_cache", (a,)),
        ("sdpa", ("rq", "k_cache", "v_cache"), "merged", (a, a + R)),
        ("linear", ("merged", "wo"), "attn", (False, 1, HID)),
        ("add", ("x", "attn"), "x2", ()),
        ("rmsnorm", ("x2", "post_scale"), "n2", ()),
        ("linear", ("n2", "wg"), "gate", (False, 1, FF)),
        ("linear", ("n2", "wu"), "up", (False, 1, FF)),
        ("silu", ("gate",), "act", ()),
        ("mul", ("act", "up"), "prod", ()),
        ("linear", ("prod", "wd"), "down", (False, 1, HID)),
        ("add", ("x2", "down"), "next", ()),
    ]


def submit(layer, step, R):
    op, ins, out, args = step
    dev, v = layer.dev, layer.v
    if op == "rmsnorm":
        token = dev.rmsnorm(v(ins[0]), v(ins[1]), v(out), EPS)
    elif op == "linear":
        planar, heads, width = args
        token = dev.linear(v(ins[0]), v(ins[1]), v(out), 0, R, planar, heads, width)
    elif op == "rope":
        token = dev.rope(v(ins[0]), v(out), args[0], THETA)
    elif op == "cache_append":
        token = dev.cache_append(v(ins[0]), v(out), args[0])
    elif op == "sdpa":
        token = dev.sdpa(v(ins[0]), v(ins[1]), v(ins[2]), v(out), args[0], args[1])
    elif op == "add":
        token = dev.binary(OP_ADD, v(ins[0]), v(ins[1]), v(out))
    elif op == "mul":
        token = dev.binary(OP_MUL, v(ins[0]), v(ins[1]), v(out))
    elif op == "silu":
        token = dev.silu(v(ins[0]), v(out))
    else:
        raise ValueError(op)
    assert token > 0, (op, out, token, dev.error())


def ulp_distance(a, b):
    """Distance in BF16 steps on the ordered encoding (sign-magnitude -> two's complement)."""
    def ordered(bits):
        bits = bits.astype(np.int64)
        return np.where(bits & 0x8000, 0x8000 - bits, bits)
    return np.abs(ordered(a) - ordered(b))


def steps_apart(got, want):
    """|got - want| in BF16 steps at the larger magnitude of the pair, with magnitudes below
    2^-7 of the tensor's rms counted as that (a sign flip between two values next to zero is
    then a fraction of a step, not thousands of encodings)."""
    g, c = f64(got), f64(want)
    floor = 2.0 ** -7 * max(np.sqrt(np.mean(c * c)), 1e-30)
    size = np.maximum(np.maximum(np.abs(g), np.abs(c)), floor)
    return np.abs(g - c) / 2.0 ** (np.floor(np.log2(size)) - 7)


def check_step(step, got, want, inputs, a, R):
    """The GPU output `got` against the CPU output `want` of the same operation on the same inputs."""
    op, ins, out, args = step
    where = f"{op} -> {out} (a={a}, R={R})"
    if op in ("add", "mul", "cache_append"):
        assert np.array_equal(got, want), where
        return 0.0, 0
    dist = ulp_distance(got, want)
    if op in ("rmsnorm", "silu"):
        assert dist.max() <= 1, (where, int(dist.max()))
    elif op == "linear":
        g, c = f64(got), f64(want)
        step_size = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(c), 1e-30))) - 7)
        assert np.all(np.abs(g - c) <= np.maximum(np.maximum(step_size, 2.0 ** -7), 2.0 ** -6 * np.abs(c))), where
    elif op == "rope":
        from test_gpu_layer_ops import rope64, ulp_at
        ref, norm = rope64(f64(inputs[0]), a, THETA)
        g, c = f64(got), f64(want)
        assert np.all(np.abs(g - ref) <= ulp_at(ref, DT_BF16) + np.ldexp(norm, -9)), where
        assert np.all(np.abs(g - c) <= 2 * ulp_at(ref, DT_BF16) + np.ldexp(norm, -12)), where
    elif op == "sdpa":
        from test_gpu_sdpa import float64_attention
        L = a + R
        case = {"leading": [1], "Hq": HQ, "Hkv": HKV, "R": R, "D": D, "C": CAP, "a": a, "L": L,
                "q": inputs[0].reshape(-1), "k": inputs[1].reshape(-1), "v": inputs[2].reshape(-1)}
        ref64, budget = float64_attention(case)
        assert np.all(np.abs(f64(got).reshape(ref64.shape) - ref64) <= budget), where
        assert np.all(np.abs(f64(want).reshape(ref64.shape) - ref64) <= budget), where
    return float(steps_apart(got, want).max()), int((dist != 0).sum())


def run_phase(cpu_forced, cpu_free, gpu, x_bits, a, R, report):
    for layer in (cpu_forced, cpu_free, gpu):
        layer.rows(R)
    gpu.put("x", x_bits)
    cpu_free.put("x", x_bits)
    for step in steps(a, R):
        op, ins, out, args = step
        # what the GPU operation is about to read (the caches before the append included)
        inputs = [gpu.get(name) for name in ins]
        before = gpu.get(out) if op == "cache_append" else None
        submit(gpu, step, R)
        got = gpu.get(out)
        for name, bits in zip(ins, inputs):
            cpu_forced.put(name, bits)
        if before is not None:
            cpu_forced.put(out, before)
        submit(cpu_forced, step, R)
        worst, differing = check_step(step, got, cpu_forced.get(out), inputs, a, R)
        report.append((f"a={a:3d} R={R:3d} {op:12s} -> {out:8s}", worst, differing, got.size))
        submit(cpu_free, step, R)
    return gpu.get("next"), cpu_free.get("next")


def test_prefill_of_512_rows_then_two_decode_steps(devices):
    cpu, gpu = devices
    w = weights()
    layers = [Layer(cpu, w), Layer(cpu, w), Layer(gpu, w)]
    report, ends = [], []
    x = bf16(datagen.normal_f32(514 * HID, 0.0, 1.0, 21)).reshape(514, HID)
    for a, R in ((0, 512), (512, 1), (513, 1)):
        got, want = run_phase(*layers, x[a:a + R].reshape(1, R, HID), a, R, report)
        dist = ulp_distance(got, want)
        g, c = f64(got), f64(want)
        scale = np.sqrt(np.mean(c * c))
        ends.append((a, R, float(steps_apart(got, want).max()), int((dist != 0).sum()), got.size,
                     float(np.abs(g - c).max() / scale)))
        # end to end: eighteen operations of independent rounding apart, still the same layer
        assert np.abs(g - c).max() <= 2.0 ** -4 * scale, ends[-1]
        assert np.median(dist) <= 1, ends[-1]
    print()
    for line, worst, differing, size in report:
        print(f"  per operation  {line}  max steps {worst:5.2f}  differing {differing:6d} of {size}")
    for a, R, worst, differing, size, rel in ends:
        print(f"  end to end     a={a:3d} R={R:3d}  max steps {worst:.2f}  differing {differing} of {size}  "
              f"max |diff| / rms {rel:.2e}")
    # the caches the two devices built are the same tokens (K rotated, V as projected) within the bars
    for name in ("k_cache", "v_cache"):
        g, c = f64(layers[2].get(name))[0, :, :514], f64(layers[1].get(name))[0, :, :514]
        assert np.abs(g - c).max() <= 2.0 ** -4 * np.sqrt(np.mean(c * c))
        assert not layers[2].get(name)[0, :, 514:].any()          # nothing past the prefix was written
    for layer in layers:
        layer.close()
