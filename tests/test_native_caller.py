"""The C ABI from a caller that has no PyTorch: tests/native/cabi_check.cpp, built by
torch-xpu-ops_amd/build.py next to the libraries, opens libmi355x_rownorm.so with dlopen and
calls it on hipMalloc memory.  Also: the header is valid C99 on its own."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "torch-xpu-ops_amd", "lib", "libmi355x_rownorm.so")
CHECK = os.path.join(ROOT, "torch-xpu-ops_amd", "lib", "cabi_check")


def _run(mode):
    assert os.path.exists(CHECK) and os.path.exists(LIB), \
        "run torch-xpu-ops_amd/build.py first: %s or %s is missing" % (CHECK, LIB)
    p = subprocess.run([CHECK, LIB, mode], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=120)
    print(p.stdout, flush=True)
    return p


def test_header_is_plain_c():
    header = os.path.join(ROOT, "include", "mi355x_rownorm.h")
    p = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-fsyntax-only", "-x", "c", header],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert p.returncode == 0 and not p.stdout.strip(), p.stdout


def test_symbols_and_validation_without_a_gpu():
    p = _run("symbols")
    assert p.returncode == 0 and "cabi_check: ok" in p.stdout, p.stdout


@pytest.mark.gpu
def test_every_family_on_hipmalloc_memory():
    p = _run("gpu")
    assert p.returncode == 0 and "cabi_check: ok" in p.stdout, p.stdout
    for what in ("rms_norm forward", "rms_norm backward dx", "rms_norm backward dweight", "layer_norm forward",
                 "softmax forward", "softmax forward, dim 1 of 3", "group_norm forward"):
        assert what in p.stdout
