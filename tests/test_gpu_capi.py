"""The C ABI without Python in the way: tests/capi_decode_step.cpp (a plain HIP program, built by
`python -m retrievalattention_amd.build`) allocates its own device buffers, runs a decode step through
ri_score_select + ri_wave_attention (+ the no-allocation variant) and compares every group with a direct fp64
evaluation on the host."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_decode_step_from_a_plain_hip_program(dev):
    exe = os.path.join(ROOT, "tests", "capi_decode_step")
    assert os.path.exists(exe), "build it first: python -m retrievalattention_amd.build"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, (r.returncode, r.stdout[-500:], r.stderr[-1500:])
    assert r.stdout.strip().endswith("ok"), r.stdout
