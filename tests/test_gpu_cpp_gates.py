"""Runs the C++ gates of the reference-signature shim headers (tests/cpp), built ahead of time by
`make -C tests/cpp` (which __graft_entry__.build() drives): the swizzled GEMV / dual-GEMV entry
points, run_moe_grouped_expert_batch against the per-token trio, the resident-expert
executor behind the V4RoutedExpertExecutor seam, and the two-tier (HBM slots over pinned host
copies) executor behind the same seam against the resident one."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "bin")


@pytest.mark.parametrize("gate", ["test_swizzled_gemv", "test_grouped_batch_parity",
                                  "test_resident_executor", "test_resident_pool",
                                  "test_elementwise_controls", "test_tiered_executor"])
def test_cpp_gate(gate):
    path = os.path.join(BIN, gate)
    assert os.path.exists(path), "tests/cpp is not built: run __graft_entry__.build()"
    run = subprocess.run([path], capture_output=True, text=True, timeout=300)
    print(run.stdout)
    print(run.stderr)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-2000:]
    assert "[PASS]" in run.stdout
