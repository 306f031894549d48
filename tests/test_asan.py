"""Host code under the address and undefined-behaviour sanitizers (tests/asan/Makefile, target `asan`): the C
oracle, the range permutation of the forward kernel, and the argument validation of the C ABI.  Needs no GPU; any finding aborts a program."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_make_asan(tmp_path):
    out = subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "asan"), "asan", "OUT=" + str(tmp_path)],
                         capture_output=True, text=True)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:]
    assert out.stdout.count("\nok") >= 3
