"""Reports the C++ tests of the host mirror (tests/cpp/hip_provider_test.cc, built by
hyle_amd.build.build_host_tests): schema/admission on the CPU, execution against the oracle on a GPU.

The tests are a separate program.  tests/conftest.py starts it when collection ends, before anything
in the session opens the GPU, because a process that holds the GPU must not start another program;
the tests here read the outcome recorded there, so it does not matter where in the session they run."""
from __future__ import annotations

import pytest

import conftest


def _report(mode: str) -> None:
    outcome = conftest.host_mirror_runs.get(mode)
    if outcome is None:
        pytest.fail(f"hip_provider_test {mode} was not started when collection ended "
                    "(tests/conftest.py: pytest_collection_finish did not see this test)")
    if "error" in outcome:
        pytest.fail(outcome["error"])
    print(outcome["stdout"])
    assert outcome["returncode"] == 0, outcome["stdout"][-4000:] + outcome["stderr"][-2000:]
    assert " 0 failed expectations" in outcome["stdout"]


def test_host_mirror_schema_and_admission():
    _report("--host")


@pytest.mark.gpu
def test_host_mirror_executes_against_oracle():
    _report("--device")
