"""Host sanitizer runs (address + undefined behaviour) of the CPU side: the oracle's sources with their driver
(`make -C oracle asan`: codecs on whole, tail and odd-length inputs, the matmul composition, a small decode model over its
whole cache, the sampler, the GGUF block conversion), and the C++ host mirror's test program on its host-only paths
(`make -C tests/cpp asan`).  A finding aborts the run with a non-zero status."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_is_clean_under_asan_and_ubsan():
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-s", "asan"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert r.stdout.strip().endswith("asan driver: ok")
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr


def test_host_mirror_is_clean_under_asan_and_ubsan():
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"), "-s", "asan"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr
