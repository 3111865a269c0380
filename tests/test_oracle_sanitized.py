"""The CPU oracle once more under AddressSanitizer + UndefinedBehaviorSanitizer (host code only): the pin and golden
tests are run in a child interpreter against ``oracle/libnesbin_oracle_asan.so``, so an out-of-bounds index or a
signed overflow in the C restatement fails a test instead of silently shaping the expected values."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_pins_hold_under_asan_and_ubsan():
    asan = subprocess.run(["gcc", "-print-file-name=libasan.so"], capture_output=True, text=True).stdout.strip()
    if not asan or not os.path.isabs(asan) or not os.path.exists(asan):
        pytest.skip("gcc has no libasan.so here")
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "libnesbin_oracle_asan.so"])
    env = dict(os.environ)
    # the sanitizer runtime has to come first in the preload list; anything already listed stays
    env["LD_PRELOAD"] = " ".join([asan] + env.get("LD_PRELOAD", "").split())
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=0"          # CPython itself is not leak-clean
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    env["NESBIN_ORACLE_LIB"] = os.path.join(ROOT, "oracle", "libnesbin_oracle_asan.so")
    r = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider",
                        os.path.join(ROOT, "tests", "test_oracle_pins.py"),
                        os.path.join(ROOT, "tests", "test_oracle_golden.py")],
                       cwd=ROOT, env=env, capture_output=True, text=True, timeout=900)
    tail = (r.stdout + r.stderr)[-4000:]
    assert r.returncode == 0, tail
    assert "runtime error" not in tail and "AddressSanitizer" not in tail, tail
