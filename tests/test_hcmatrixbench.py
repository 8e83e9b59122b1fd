"""The C++ HCMatrixBench (honeycrisp_amd/cpp/HCMatrixBench.cpp, built by build()) as a child
process: the counterpart of the reference's benchmark executable
(Sources/HCMatrixBench/Entrypoint.swift:12-27) driving the backend through the C++ mirror of
the Backend interface. Checks that every line parses, that every self-check of the program
passed, and that the figures are plausible for the device (lower bounds far below the measured
rates, so that only a kernel that did not run, or ran on the wrong path, trips them)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "honeycrisp_amd", "cpp", "HCMatrixBench")


def test_hcmatrixbench_runs_and_reports():
    assert os.path.exists(BINARY), "build it with `python -m honeycrisp_amd.csrc.build`"
    print("running", BINARY, flush=True)
    proc = subprocess.run([BINARY, "5", "4096"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=170)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    lines = [dict(kv.split("=", 1) for kv in line.split()) for line in proc.stdout.strip().splitlines()]
    assert lines[0]["backend"] == "HIPBackend" and lines[-1] == {"failures": "0"}
    ops = lines[1:-1]
    assert all(r["check"] == "ok" for r in ops), proc.stdout
    matmuls = {(r["dtype"], r["layout"], int(r["size"])): float(r["gflops"]) for r in ops if r["op"] == "matmul"}
    assert set(matmuls) == {(d, l, n) for d in ("float16", "float32") for l in ("NN", "NT") for n in (512, 1024, 2048, 4096)}
    assert matmuls[("float16", "NN", 4096)] > 300e3 and matmuls[("float16", "NT", 4096)] > 300e3   # GFLOP/s
    assert matmuls[("float32", "NN", 4096)] > 50e3
    bandwidth = {r["op"]: float(r["gbs"]) for r in ops if r["op"] != "matmul"}
    assert set(bandwidth) == {"bias_add", "gelu", "sum_axis1", "argmax_axis1", "max_axis1", "embedding_gather"}
    assert min(bandwidth.values()) > 1000.0   # GB/s
