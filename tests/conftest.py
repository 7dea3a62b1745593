import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HOST_MIRROR_BINARY = os.path.join(ROOT, "tests", "cpp", "hip_provider_test")
# test name -> mode of tests/cpp/hip_provider_test it reports on
HOST_MIRROR_TESTS = {
    "test_host_mirror_schema_and_admission": "--host",
    "test_host_mirror_executes_against_oracle": "--device",
}

# Outcomes of the hip_provider_test runs, filled in before the first test of the session runs:
# mode -> {"returncode", "stdout", "stderr"} or {"error": text}.
host_mirror_runs = {}


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def process_holds_gpu() -> bool:
    """True once this process has opened the GPU's compute device."""
    try:
        return any(os.path.realpath(os.path.join("/proc/self/fd", fd)) == "/dev/kfd"
                   for fd in os.listdir("/proc/self/fd"))
    except OSError:
        return False


def pytest_collection_finish(session):
    """The C++ tests of the host mirror are a program of their own.  A process that already holds
    the GPU must not start another program, so the binary runs here: after collection has settled
    which tests are selected and before any of them (or any fixture) touches the device.  The
    tests themselves only read the recorded outcome, whatever position they run at."""
    if session.config.getoption("collectonly", False):
        return
    for item in session.items:
        mode = HOST_MIRROR_TESTS.get(item.name)
        if mode is None or mode in host_mirror_runs:
            continue
        if process_holds_gpu():
            host_mirror_runs[mode] = {"error": (
                "the test process opened the GPU before the session's tests started (a module touches "
                f"the device at import time): hip_provider_test {mode} cannot be started from here")}
        elif not os.path.exists(HOST_MIRROR_BINARY):
            host_mirror_runs[mode] = {"error": "tests/cpp/hip_provider_test is not built: run __graft_entry__.build()"}
        else:
            try:
                done = subprocess.run([HOST_MIRROR_BINARY, mode], capture_output=True, text=True, timeout=300)
                host_mirror_runs[mode] = {"returncode": done.returncode, "stdout": done.stdout, "stderr": done.stderr}
            except (OSError, subprocess.SubprocessError) as error:
                host_mirror_runs[mode] = {"error": f"hip_provider_test {mode} did not run: {error}"}
