"""The reference's own acceptance programs for a physical backend (its tools/test/gpu-trunk-mapped-test.c and
gpu-moe-shared-mapped-test.c, Makefile targets test-gpu-trunk and test-gpu-moe-shared), built in the authoring container
from the reference's sources where they lie and linked against this repository's library (oracle/Makefile, target
ref-gpu-tests).  The first drives resident_trunk_map, q4_batch, q4_matvec, the engine's mixed CPU/GPU projection over
proj_batch_indexed, the batch counters, mapped-only rejections and a free / init / second-lifecycle cycle; the second
is the whole engine (every source of its Makefile's SRC) running a MoE layer step whose trunk projections go to the
backend, synchronously and deferred.  Both compare every output byte for byte with the reference's CPU kernels.

A third program is this repository's own (tests/residency_engine_path.c) over the reference's packed expert pool, expert
cache with its resource hooks, and residency ledger: the trunk becomes permanent spans of the residency arena, every
expert of a 30-layer pool takes a seat in HBM through the cache's bind hook, and the trunk projections and the selected
expert chain are compared with the reference's CPU kernels; then again with sixteen seats, so that the cache evicts."""
import os
import subprocess
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
PROGRAMS = ROOT / "oracle" / "_ref"


@pytest.mark.parametrize("name,verdict", [("gpu-trunk-mapped-test", "gpu-trunk mapped projection: PASS"),
                                          ("gpu-moe-shared-mapped-test", "gpu-moe shared mapped: PASS"),
                                          ("residency-engine-path", "residency-engine-path: PASS")])
def test_reference_acceptance_program_passes(name, verdict):
    program = PROGRAMS / name
    if not program.exists():
        pytest.skip("the reference tree was not mounted where the checker was built")
    print(name, flush=True)
    env = dict(os.environ, SALT_REQUIRE_GPU="1")
    run = subprocess.run([str(program)], env=env, capture_output=True, text=True, timeout=300)
    print(run.stdout, run.stderr, flush=True)
    assert run.returncode == 0, run.stderr
    assert verdict in run.stdout
