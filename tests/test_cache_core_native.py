"""The cache core checked without Python in between: a C++ program (tests/cpp/core_check.cpp)
that counts allocations on the per-step path and runs a random workload against a model,
built once as the module is built and once with the address and undefined-behaviour
sanitizers; every compiler warning is an error in both builds
(the reference: tests/cpp/test_no_alloc.cpp:79-144, CMakeLists.txt:15-18,50-54)."""

from __future__ import annotations

import subprocess
from pathlib import Path

import pytest

from prefixserve_amd.build import build_core_program

SOURCE = Path(__file__).resolve().parent / "cpp" / "core_check.cpp"


@pytest.mark.parametrize("sanitize", [False, True], ids=["plain", "sanitizers"])
def test_core_check_program(sanitize, tmp_path):
    exe = build_core_program(SOURCE, tmp_path / "core_check", sanitize=sanitize)
    env = {"ASAN_OPTIONS": "detect_leaks=1:abort_on_error=0", "UBSAN_OPTIONS": "print_stacktrace=1", "PATH": "/usr/bin:/bin"}
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300, env=env)
    assert run.returncode == 0, run.stdout + run.stderr
    out = run.stdout
    assert "the counter counts" in out and "allocated 0 times" in out and "all core checks passed" in out
    assert out.count("ok: random workload") == 5
    assert "runtime error" not in run.stderr and "AddressSanitizer" not in run.stderr


def test_core_benchmark_runs_and_meets_the_reference_bar(tmp_path):
    """The core's micro-benchmark (the reference: bench/micro_core.cpp, whose bar for looking up a
    held 2,048-token prompt is 10 microseconds): it builds with every warning an error, runs, and
    the lookup is under the bar (the program's exit status says so); the figures it prints parse."""
    from prefixserve_amd.build import CSRC

    exe = build_core_program(CSRC / "core" / "core_bench.cpp", tmp_path / "core_bench", what="core benchmark")
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    lines = run.stdout.strip().splitlines()
    assert len(lines) == 4 and lines[0].startswith("lookup of 2048 held tokens")
    figures = [float(line.split(": ")[1].split(" ns/call")[0]) for line in lines]
    assert all(0 < f < 1e6 for f in figures) and figures[0] < 10000
