"""The host side of the library (API, recorder, planner, serializer) under
AddressSanitizer and UndefinedBehaviorSanitizer: `make sanitize` builds the
library with those files instrumented, and the device-less tests - ABI checks,
stored computations with corrupted records, host-only lowering of the benchmark
graphs - run against it in a child process with the sanitizer runtimes
preloaded.  Any report ends the child with a non-zero status.
"""
import os
import subprocess
import sys

import pytest

import __graft_entry__ as entry

CSRC = os.path.join(entry.PKG_DIR, "csrc")
SAN_LIB = os.path.join(entry.PKG_DIR, "libodla_hip_san.so")
CASES = ["tests/test_abi_cpu.py", "tests/test_stored_computation_cpu.py", "tests/test_plan_summary_cpu.py"]


def runtime(name):
    path = subprocess.run(["gcc", "-print-file-name=" + name], capture_output=True, text=True).stdout.strip()
    return path if os.path.isabs(path) and os.path.exists(path) else None


def test_cpu_suites_are_clean_under_asan_and_ubsan():
    asan, ubsan = runtime("libasan.so"), runtime("libubsan.so")
    if asan is None or ubsan is None:
        pytest.skip("gcc's sanitizer runtimes are not installed")
    subprocess.check_call(["make", "-C", CSRC, "-j", str(min(8, os.cpu_count() or 1)), "sanitize"],
                          stdout=subprocess.DEVNULL)
    env = dict(os.environ)
    preload = [asan, ubsan] + [p for p in env.get("LD_PRELOAD", "").split(":") if p]
    env.update(LD_PRELOAD=":".join(preload), ODLA_HIP_LIBRARY=SAN_LIB,
               ASAN_OPTIONS="detect_leaks=0:halt_on_error=1",       # the interpreter itself is not instrumented
               UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    # -s: a report is written to stderr just before the process ends, past pytest's capture
    run = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-s", "-p", "no:cacheprovider"] + CASES,
                         cwd=entry.ROOT, env=env, capture_output=True, text=True, timeout=900)
    out = run.stdout + run.stderr
    reports = [l for l in out.splitlines() if "runtime error:" in l or "ERROR: AddressSanitizer" in l]
    assert run.returncode == 0 and not reports, "\n".join(reports or out.splitlines()[-30:])
    assert " passed" in out
