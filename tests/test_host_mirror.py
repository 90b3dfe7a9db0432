"""The C++ host mirror of the axonml-quant API (include/axonml_quant.hpp), through its own test program
(tests/cpp/host_mirror_test.cpp, which reads like the reference crate's unit tests)."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "cpp", "host_mirror_test")


def _run():
    return subprocess.run([EXE], capture_output=True, text=True, timeout=120)


def test_host_mirror_compiles_and_fails_loudly_without_a_gpu():
    subprocess.run(["make", "-C", os.path.join(HERE, "cpp"), "-s"], check=True, timeout=300)
    r = _run()
    # 0 on a GPU box, 77 = "no usable GPU" everywhere else; anything else is a failed check or a crash
    assert r.returncode in (0, 77), r.stdout + r.stderr
    if r.returncode == 77:
        assert "no usable GPU" in r.stdout


@pytest.mark.gpu
def test_host_mirror_on_gpu():
    assert os.path.exists(EXE), "tests/cpp/host_mirror_test is not built (run __graft_entry__.build())"
    r = _run()
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout
