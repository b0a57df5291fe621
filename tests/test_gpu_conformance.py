"""IOM's own backend-agnostic conformance scenarios, run once against this backend.

The binary oracle/_ref/mi355x_conformance is tests/conformance/mi355x_conformance.cpp compiled
together with the reference's scenario headers (test/backend/backend_conformance_*.hpp, in place)
and linked against iom::make_rocm_device of iom_amd/host and the reference CPU backend.  Every
assertion that decides the outcome is the reference's; this test runs the binary, prints the
assertion count of every scenario and fails on any failed assertion or missing scenario.

Skipped where the binary was not built (it needs the reference sources at build time)."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "oracle", "_ref", "mi355x_conformance")

# scenario -> the shared runner(s) of the reference it calls
SCENARIOS = {
    "MI355X: supported_data_types is the standard 23-entry span": "require_standard_capabilities",
    "MI355X: storage and host transfers for every leaf type": "run_storage_and_transfer_conformance",
    "MI355X: storage oracle tells a perturbed tile map from the true one": "run_storage_oracle_conformance",
    "MI355X: raw tiled storage of every leaf width and padded shape": "run_storage_oracle_conformance",
    "MI355X: asynchronous copies against the CPU reference": "run_async_copy_conformance",
    "MI355X: copy validation fails before writes and sequences": "run_copy_error_conformance",
    "MI355X: transfer failures keep metadata and ownership": "run_transfer_error_conformance",
    "MI355X: sub-byte odd-length host reads": "require_logical_bytes",
    "MI355X: deferred queue lifetime and stability": "run_lifetime_conformance",
    "MI355X: compute methods reject capability without submitting": "run_compute_capability_conformance",
    "MI355X: rank-eight owners accepted, rank nine rejected": "run_accelerator_rank_boundary_conformance",
    "MI355X: ADD MUL SUB DIV on the real queue, values, mappings and exact aliases":
        "run_gpu_eltwise_conformance, run_gpu_eltwise_mapping_conformance, run_gpu_exact_alias_conformance",
    "MI355X: binary rank boundary": "run_binary_rank_boundary_conformance",
    "MI355X: RMSNorm reference, admission and lifetime": "run_rmsnorm_conformance",
    "MI355X: SiLU reference, admission and lifetime": "run_silu_conformance",
    "MI355X: cache append reference, admission, ordering and lifetime": "run_cache_append_conformance",
    "MI355X: embedding lookup reference, admission and lifetime": "run_embedding_conformance",
    "MI355X: RoPE reference, admission and lifetime": "rope_reference::run_rope_conformance",
    "MI355X: linear projection reference, admission and lifetime": "run_linear_conformance",
    "MI355X: SDPA admission and BF16 attention on the matrix cores": "run_sdpa_conformance",
    "MI355X: full shared suite with the RoPE contract": "run_backend_conformance",
}

# behaviours the reference's own accelerator driver asserts through backend seams
# (test/rocm/test_rocm_conformance.cpp:374-540, 798-838, 1242-1288, 1366-1492, 1906-2221, 2314-2407),
# asked of this backend through its seams with the reference's shared helpers for data and values
BACKEND_CASES = {
    "MI355X backend: a launch that fails after acceptance repeats its failure and the owners serve the next one":
        "ROCm ADD retained launch failure keeps owners reusable",
    "MI355X backend: only accepted submissions take a sequence, and a failed one's operands are not recycled":
        "ROCm submission remains transactional across post-enqueue failures",
    "MI355X backend: queue destruction drains pending copies around a failed one":
        "ROCm queue destruction fences pending copies",
    "MI355X backend: a source destroyed before the wait stays intact until both of its copies are done":
        "ROCm pre-wait source destruction / shared-operand copies",
    "MI355X backend: operands of work nobody waited for are quarantined once their queue is gone":
        "ROCm operands destroyed after queue teardown remain quarantined",
    "MI355X backend: cache append failures retire, a new queue appends correctly, pending operands are quarantined":
        "ROCm cache append retained event / launch failure, queue teardown, source retention",
    "MI355X backend: an embedding whose status word cannot be fetched retires as failed and the queue goes on":
        "ROCm embedding status transfer failure retires safely",
    "MI355X backend: SiLU launch evidence, accepted failure, recovery, and quarantine after an unrecorded completion":
        "ROCm SiLU accepted native failure / failed drain",
    "MI355X backend: SiLU submitted through views that die before the wait, input owner destroyed first":
        "ROCm SiLU retains snapshot and owners across temporary views",
    "MI355X backend: one SiLU kernel per accepted request of every floating leaf, none for a rejected one, negative subnormal tails kept":
        "ROCm SiLU native launch evidence and negative subnormal tails",
    "MI355X backend: TinyLlama-shaped attention, prefill of 17 rows and the decode step that follows it":
        "ROCm TinyLlama SDPA native QK/PV decode and prefill",
    "MI355X backend: workspaces are ranges of the one arena, and requirement queries are pure":
        "ROCm raw workspace suballocates the arena / workspace requirement queries",
}
SCENARIOS.update(BACKEND_CASES)

CASE_LINE = re.compile(r"^\[ (?: ok |FAIL) \] (.*): (\d+) assertions, (\d+) failed$")
DONE_LINE = re.compile(r"^\[ done \] (\d+) cases, (\d+) failed; (\d+) assertions, (\d+) failed$")


def test_reference_conformance_scenarios_pass_on_the_backend():
    if not os.path.exists(BINARY):
        pytest.skip("oracle/_ref/mi355x_conformance not built (needs the reference sources)")
    proc = subprocess.run([BINARY], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=900)
    seen, done = {}, None
    for line in proc.stdout.splitlines():
        m = CASE_LINE.match(line)
        if m:
            seen[m.group(1)] = (int(m.group(2)), int(m.group(3)))
        m = DONE_LINE.match(line)
        if m:
            done = tuple(int(g) for g in m.groups())
    for name, (asserts, failed) in seen.items():
        print(f"{asserts:>9} assertions, {failed} failed  {name}  [{SCENARIOS.get(name, '?')}]")
    failures = [l for l in proc.stdout.splitlines() if "FAILED" in l]
    assert proc.returncode == 0 and not failures, "\n".join(failures[:40]) or proc.stdout[-4000:]
    assert done is not None, proc.stdout[-2000:]
    assert set(seen) == set(SCENARIOS), sorted(set(SCENARIOS) ^ set(seen))
    assert done[1] == 0 and done[3] == 0
    # every scenario evaluated something: an empty pass would be a harness fault
    assert all(asserts > 0 for asserts, _ in seen.values())
    print("total", done[2], "assertions in", done[0], "scenarios")
