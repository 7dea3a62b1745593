"""Runs the C++ tests of the host mirror (tests/cpp/hip_provider_test.cc, built by
hyle_amd.build.build_host_tests): schema/admission on the CPU, execution against the oracle on a GPU."""
from __future__ import annotations

import os
import subprocess

import pytest

BINARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "hip_provider_test")


def _run(mode: str) -> None:
    if not os.path.exists(BINARY):
        pytest.fail("tests/cpp/hip_provider_test is not built: run __graft_entry__.build()")
    done = subprocess.run([BINARY, mode], capture_output=True, text=True, timeout=300)
    print(done.stdout)
    assert done.returncode == 0, done.stdout[-4000:] + done.stderr[-2000:]
    assert " 0 failed expectations" in done.stdout


def test_host_mirror_schema_and_admission():
    _run("--host")


@pytest.mark.gpu
def test_host_mirror_executes_against_oracle():
    _run("--device")
