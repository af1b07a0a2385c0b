"""Runs the C++ harness (tests/harness/mixed_gemv_test.cpp, the counterpart of the reference's
main()) as a child process: seeded inputs, 20 launches through the C++ host mirror, HOST_CHECK
comparison, exit code 0 only on a pass."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "harness", "mixed_gemv_test")

CASES = [
    ["151936", "2048", "128", "3", "4", "0"],  # the problem the reference's main() ships with (mixed_gemv_test.cu:187), at full size
    ["11008", "2048", "128", "3", "4", "0"],   # one of the reference's own shapes (mixed_gemv_test.cu:189), mode as shipped
    ["2048", "11008", "128", "3", "4", "1"],   # the other one (:188), with the bias epilogue
    ["4096", "4096", "128", "2", "4", "1"],
    ["4096", "4096", "0", "1", "8", "1"],
]


@pytest.mark.gpu
@pytest.mark.parametrize("args", CASES, ids=["x".join(a) for a in CASES])
def test_cpp_harness(gpu, args):
    if not os.path.exists(BINARY):
        pytest.fail(f"{BINARY} is not built (run __graft_entry__.build())")
    proc = subprocess.run([BINARY] + args, capture_output=True, text=True, timeout=240)
    print(proc.stdout[-2000:], proc.stderr[-1000:])
    assert proc.returncode == 0, proc.stdout[-2000:]
    assert "PASS" in proc.stdout
