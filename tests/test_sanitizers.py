"""AddressSanitizer + UBSan over the host-side code, CPU only: the oracle's own
self-test (oracle/selftest.c: every oracle function on exactly sized heap buffers at
its edge shapes) and the C++ operator interface's host tests (the model file reader
with its mutation loop, tensors, attribute parsing, the base-class checks) rebuilt
with -fsanitize=address,undefined.  A report from either sanitizer ends the program
with a non-zero status."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _make(directory, timeout):
    r = subprocess.run(["make", "-C", os.path.join(ROOT, directory), "asan"], capture_output=True, text=True, timeout=timeout)
    print(r.stdout[-4000:])
    print(r.stderr[-4000:])
    assert r.returncode == 0
    assert "ERROR: AddressSanitizer" not in r.stderr and "runtime error:" not in r.stderr
    assert " 0 failed" in r.stdout
    return r


def test_oracle_under_asan_ubsan():
    _make("oracle", 300)


def test_host_layer_and_model_reader_under_asan_ubsan():
    r = _make(os.path.join("vkop_amd", "host"), 900)
    assert "Model file mutations" in r.stdout
