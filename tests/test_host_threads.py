"""The host code of libacchip under ThreadSanitizer, eight threads on one context, against an in-process stand-in for
the HIP runtime (tests/tsan): no GPU, no device code, the real hiprtc.  What is checked is the absence of data races in
the scratch pool, the skeleton instances, the scan ordering, guards, the memory table and the launch trace."""
import os
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tsan")


def test_many_threads_on_one_context_race_free():
    build = subprocess.run(["make", "-C", HERE], capture_output=True, text=True)
    assert build.returncode == 0, build.stdout[-3000:] + build.stderr[-3000:]
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=0 second_deadlock_stack=1")
    run = subprocess.run([os.path.join(HERE, "host_threads"), "8", "150"], capture_output=True, text=True, env=env, timeout=600)
    text = run.stdout + run.stderr
    if "FATAL: ThreadSanitizer" in text:              # the sanitizer itself cannot run here (address-space layout)
        pytest.skip(text.strip().splitlines()[0])
    assert "WARNING: ThreadSanitizer" not in text, text[-6000:]
    assert run.returncode == 0 and "failures 0" in run.stdout, text[-3000:]
