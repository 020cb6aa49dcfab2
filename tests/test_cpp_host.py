"""The C++ host layer (include/dsx_moe.hpp: the reference's Rust wrapper API -- Stream,
DeviceBuffer, RouterTopk, Q8KQuantize, MoeGroupBuilder, het::dispatch, MoeExecutor -- over the C
ABI) driven by tests/cpp/host_mirror_test.cpp, which checks every result against the CPU oracle.
The binary is built by __graft_entry__.build() (make -C tests/cpp); one process runs all cases."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "_build", "host_mirror_test")


def _run(args, timeout):
    if not os.path.exists(BIN):
        pytest.fail(f"{BIN} is not built: run `python __graft_entry__.py`")
    res = subprocess.run([BIN, *args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                         timeout=timeout)
    print(res.stdout)
    return res


def test_cpp_wrappers_refuse_bad_arguments_before_any_launch():
    res = _run(["--host-only"], 60)
    assert res.returncode == 0, res.stdout
    assert "PASS" in res.stdout and "0 failed" in res.stdout


@pytest.mark.gpu
def test_cpp_host_layer_against_the_oracle():
    res = _run([], 110)
    assert res.returncode == 0, res.stdout
    last = res.stdout.strip().splitlines()[-1]
    assert last.startswith("PASS") and "(host only)" not in last, last
    for case in ("mxfp4 sigmoid group-limited", "mxfp4 sqrt-softplus", "q8_0 softmax"):
        assert f"== {case}" in res.stdout
