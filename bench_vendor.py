"""Vendor yardsticks for bench.py: kernels this repository did not write, timed on the same box.

    python3 bench_vendor.py stream STEPS    elementwise kernels of the importable torch on the headline
                                            shapes (broadcast ADD BF16 [32768,2048]+[2048], a 128 MiB
                                            Tensor.copy_, ADD F32 [4096,4096]; row-major tensors, six
                                            rotating sets so the footprint exceeds the Infinity Cache)
    python3 bench_vendor.py gemm STEPS      the vendor GEMM library (torch.nn.functional.linear, BF16) on
                                            the two prefill shapes of the linear workload

One JSON line per workload.  bench.py runs this file as a child process (torch carries a HIP runtime
of its own, which finds no device in a process where the system's runtime already holds it); it can
also be run by itself, e.g. under `rocprofv3 --kernel-trace --stats -- python3 bench_vendor.py stream 200`.
Nothing of the product imports it.
"""
import json
import sys
import time

import torch


def stream(steps):
    ROT = 6
    def timed(name, kernel, alg_bytes, launch):
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.03:
            for i in range(ROT):
                launch(i)
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(steps):
            launch(i)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        gbs = alg_bytes / (ms * 1e-3) / 1e9
        print(json.dumps({"workload": name, "kernel": kernel, "algorithmic_bytes": alg_bytes,
                          "ms_per_launch": round(ms, 5), "GB_per_s": round(gbs, 1),
                          "hbm_frac": round(gbs / 8000.0, 4)}), flush=True)

    # broadcast ADD BF16 [64*512, 2048] + [2048], row-major, out-of-place into preallocated outputs
    M, F = 64 * 512, 2048
    xs = [torch.randn(M, F, device="cuda", dtype=torch.bfloat16) for _ in range(ROT)]
    os_ = [torch.empty(M, F, device="cuda", dtype=torch.bfloat16) for _ in range(ROT)]
    b = torch.randn(F, device="cuda", dtype=torch.bfloat16) * 0.02
    timed("vendor_stream_torch_add_bf16_[32768,2048]+[2048]", "torch.add(out=) elementwise kernel",
          (2 * M * F + F) * 2, lambda i: torch.add(xs[i % ROT], b, out=os_[i % ROT]))
    # copy of 128 MiB through the same tensors
    timed("vendor_stream_torch_copy_128MiB", "Tensor.copy_ (same dtype, contiguous)",
          2 * M * F * 2, lambda i: os_[i % ROT].copy_(xs[i % ROT]))
    del xs, os_
    # ADD F32 [4096,4096]
    N = 4096
    a = [torch.rand(N, N, device="cuda") * 2 - 1 for _ in range(ROT)]
    c = [torch.rand(N, N, device="cuda") * 2 - 1 for _ in range(ROT)]
    o = [torch.empty(N, N, device="cuda") for _ in range(ROT)]
    timed("vendor_stream_torch_add_f32_[4096,4096]", "torch.add(out=) elementwise kernel",
          3 * N * N * 4, lambda i: torch.add(a[i % ROT], c[i % ROT], out=o[i % ROT]))


def gemm(steps):
    M, K = 64 * 512, 2048
    x = torch.randn(M, K, device="cuda", dtype=torch.bfloat16)
    for N, name in ((2048, "o_proj"), (5632, "gate_proj")):
        w = torch.randn(N, K, device="cuda", dtype=torch.bfloat16) * 0.02
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.03:
            for _ in range(5):
                torch.nn.functional.linear(x, w)
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            torch.nn.functional.linear(x, w)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        tf = 2.0 * M * K * N / (ms * 1e-3) / 1e12
        print(json.dumps({"workload": "vendor_gemm_bf16_%s_[32768,2048]x[%d,2048]" % (name, N),
                          "kernel": "torch.nn.functional.linear (hipBLASLt / rocBLAS)",
                          "ms_per_launch": round(ms, 5), "TFLOP_per_s": round(tf, 1),
                          "mfma_frac_of_2500": round(tf / 2500.0, 4)}), flush=True)


if __name__ == "__main__":
    which, steps = sys.argv[1], int(sys.argv[2])
    {"stream": stream, "gemm": gemm}[which](steps)
