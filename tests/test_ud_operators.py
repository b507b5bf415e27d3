"""Runs the C++ operator-level tests (tests/ud_op_test.cpp): the Hip*
operator classes, tensors and buffer manager that mirror the reference's operator API,
checked bit for bit against the CPU oracle inside the test program."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "ud_op_test")


def _binary():
    if not os.path.exists(BIN):
        import importlib
        importlib.import_module("cl-eden-kernel_amd.build").build_all()
        importlib.import_module("build_native").build_ud_test()
    return BIN


def test_host_side_buffer_pool_and_types():
    r = subprocess.run([_binary(), "--host-only"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    print(r.stdout)
    assert r.returncode == 0, r.stdout
    assert "0 of 5 host-only tests failed" in r.stdout


@pytest.mark.gpu
def test_operator_classes_on_gpu():
    r = subprocess.run([_binary()], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(r.stdout, flush=True)
    # on failure show what is not a plain RUN / OK line: the failed expectations and the first mismatching bytes
    notable = "\n".join(l for l in r.stdout.splitlines() if not l.startswith(("[ RUN", "[  OK")))
    assert r.returncode == 0, notable[-4000:]
    assert "FAIL" not in r.stdout, notable[-4000:]
    assert "GPU operator tests failed" in r.stdout
