"""AddressSanitizer + UndefinedBehaviorSanitizer over the host code: the C oracle, the product's host RNNT loss
(speech_amd/csrc/mi_cpu.cpp) and the host-side planning of the GPU library (speech_amd/csrc/mi_plan.h), driven with
random shapes by tests/native/fuzz_host.cpp.  Host code only: nothing here touches a GPU."""

import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_sanitized_fuzz_of_host_code_finds_nothing():
    build = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "_asan/fuzz_host"], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    run = subprocess.run([os.path.join(ROOT, "oracle", "_asan", "fuzz_host"), "400", "7"], capture_output=True, text=True,
                         env=env, timeout=600)  # fmt: skip
    assert run.returncode == 0, (run.stdout[-2000:], run.stderr[-2000:])
    assert "0 failure(s)" in run.stdout
