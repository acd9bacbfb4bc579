"""The C++ mirror of the reference's operator classes (include/mfmoe.hpp), driven by a C++
program that reads like the reference's own operator tests: grouping KATs and thrown errors on
the CPU, one layer (decode, two-phase, ragged prefill) against the CPU checker on the GPU."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CPP = os.path.join(HERE, "cpp")
BIN = os.path.join(CPP, "mirror_test")


def _binary():
    if not os.path.exists(BIN):  # normally built by __graft_entry__.build()
        from mference_amd import _capi
        from oracle import mf_oracle
        _capi.lib()
        mf_oracle.lib()
        subprocess.run(["make", "-C", CPP, "mirror_test"], check=True, capture_output=True)
    return BIN


def _run(mode):
    r = subprocess.run([_binary(), mode], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "mirror_test: ok" in r.stdout
    return r.stdout


def test_cpp_mirror_grouping_and_errors():
    _run("cpu")


@pytest.mark.gpu
def test_cpp_mirror_layer_on_gpu():
    out = _run("gpu")
    assert "ragged prefill layer" in out and "decode layer" in out
