"""The C++ host layer (deepnet_amd/cpp/hip_tensor.hpp) through its own test driver, tests/cpp/host_cpp_test.cpp.

The driver is built beforehand by __graft_entry__.build(); it links libtensor_hip.so and the CPU oracle and prints one PASS/FAIL
line per case.  `layout` mode needs no GPU; `gpu` mode runs every frontend operation on the device against the oracle.
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "_build", "host_cpp_test")


def _run(mode):
    if not os.path.exists(EXE):
        import __graft_entry__
        __graft_entry__.build_cpp_host_test()
    p = subprocess.run([EXE, mode], capture_output=True, text=True, timeout=110)
    failed = [l for l in p.stdout.splitlines() if l.startswith("FAIL")]
    assert p.returncode == 0 and not failed, "\n".join(failed) + "\n" + p.stdout[-2000:] + p.stderr[-2000:]
    return p.stdout


def test_cpp_layout_algebra():
    out = _run("layout")
    assert "0 failed" in out


@pytest.mark.gpu
def test_cpp_frontend_against_oracle():
    out = _run("gpu")
    assert "0 failed" in out
    assert out.count("PASS parity.") >= 30 and out.count("PASS doc.") >= 40


@pytest.mark.gpu
def test_cpp_reference_benchmark_loop_runs():
    """deepnet_amd/cpp/bench_suite.cpp (the reference's benchmark loop through the compiled host layer) runs every method at every
    shape and type and prints the reference's CSV columns."""
    exe = os.path.join(ROOT, "deepnet_amd", "cpp", "_build", "bench_suite")
    if not os.path.exists(exe):
        import __graft_entry__
        __graft_entry__.build_cpp_bench()
    p = subprocess.run([exe, "1", "0"], capture_output=True, text=True, timeout=110)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = p.stdout.strip().splitlines()
    assert lines[0] == "Method,Shape,Type,Dev,Mean [ms],StdDev [ms]"
    rows = [l.split(",") for l in lines[1:]]
    assert all(len(r) == 6 and r[3] == "Hip" and float(r[4]) > 0 for r in rows)
    assert {r[1] for r in rows} == {"1000x1000", "2000x2000", "4000x4000"}
    assert {r[2] for r in rows} == {"single", "double", "int32"}
    assert {"Add", "SumAxis", "ArgMaxAxis", "MaskedGet", "Dot", "Invert"} <= {r[0] for r in rows}
