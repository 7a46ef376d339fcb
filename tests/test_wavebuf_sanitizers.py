"""The host wave buffer (csrc/wavebuf.cpp: worker pool, block cache manager, K/V re-organisation) under
ThreadSanitizer and under AddressSanitizer + UndefinedBehaviorSanitizer: tests/host_wavebuf_driver.cpp is compiled
together with wavebuf.cpp by g++ and run as a program of its own (host code only; the GPU kernels are not involved).
The update of the block cache runs on the workers behind the caller, which is what the thread sanitizer is for."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCES = [os.path.join(ROOT, "tests", "host_wavebuf_driver.cpp"),
           os.path.join(ROOT, "retrievalattention_amd", "csrc", "wavebuf.cpp")]


@pytest.mark.parametrize("name,flags,env", [
    ("thread", ["-fsanitize=thread"], {"TSAN_OPTIONS": "halt_on_error=1 exitcode=66"}),
    ("address+undefined", ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined"],
     {"ASAN_OPTIONS": "detect_leaks=1 exitcode=67"}),
])
def test_wave_buffer_is_clean_under(tmp_path, name, flags, env):
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    exe = str(tmp_path / "driver")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-pthread"] + flags + ["-I", os.path.join(ROOT, "include")] + SOURCES + ["-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    if r.returncode != 0 and "cannot find" in r.stderr:
        pytest.skip("sanitizer runtime not installed: " + r.stderr.strip().splitlines()[-1])
    assert r.returncode == 0, r.stderr[-2000:]
    run_env = {k: v for k, v in os.environ.items() if k != "LD_PRELOAD"}
    run_env.update(env)
    outs = []
    for threads in ("1", "4", "7"):
        r = subprocess.run([exe, threads], capture_output=True, text=True, timeout=300, env=run_env)
        assert r.returncode == 0, (threads, r.stdout[-500:], r.stderr[-3000:])
        assert "Sanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-3000:]
        outs.append(r.stdout.strip())
    assert len(set(outs)) == 1, outs          # the lists do not depend on how many workers share the groups
