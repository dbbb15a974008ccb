"""Runs the C++ test program of the drop-in classes (tests/cpp/test_host_classes.cpp,
built by vkllama_amd/host/Makefile): its host-only part here, everything on a GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "vkllama_amd", "lib", "test_host_classes")


def _run(args):
    assert os.path.exists(BIN), "build it with __graft_entry__.build()"
    r = subprocess.run([BIN] + args, capture_output=True, text=True, timeout=300)
    print(r.stdout[-2000:], r.stderr[-4000:])
    return r


def test_host_only_checks():
    r = _run(["--cpu"])
    assert r.returncode == 0, r.stderr[-2000:]
    assert "0 failed" in r.stdout


@pytest.mark.gpu
def test_operator_classes_on_the_gpu():
    r = _run([])
    assert r.returncode == 0, r.stderr[-2000:]
    assert "0 failed" in r.stdout
