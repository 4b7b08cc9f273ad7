"""The reference's own acceptance program for a physical backend's trunk path (its tools/test/gpu-trunk-mapped-test.c,
Makefile target test-gpu-trunk), built in the authoring container from the reference's sources where they lie and
linked against this repository's library (oracle/Makefile, target ref-gpu-tests).  It drives resident_trunk_map, q4_batch,
q4_matvec, the engine's mixed CPU/GPU projection over proj_batch_indexed, the batch counters, mapped-only rejections and
a free / init / second-lifecycle cycle, and compares every output byte for byte with the reference's CPU kernels."""
import os
import subprocess
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
PROGRAM = ROOT / "oracle" / "_ref" / "gpu-trunk-mapped-test"


@pytest.mark.skipif(not PROGRAM.exists(), reason="the reference tree was not mounted where the checker was built")
def test_reference_trunk_acceptance_program_passes():
    env = dict(os.environ, SALT_REQUIRE_GPU="1")
    run = subprocess.run([str(PROGRAM)], env=env, capture_output=True, text=True, timeout=120)
    print(run.stdout, run.stderr, flush=True)
    assert run.returncode == 0, run.stderr
    assert "gpu-trunk mapped projection: PASS" in run.stdout
