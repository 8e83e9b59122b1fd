"""The C++ HCMatrixBench (honeycrisp_amd/cpp/HCMatrixBench.cpp, built by build()) as a child
process: the counterpart of the reference's benchmark executable
(Sources/HCMatrixBench/Entrypoint.swift:10-27) driving BOTH backends on the same seeded inputs:
the MI355X backend through the C++ mirror of the Backend interface, and the reference CPUBackend's
algorithms on the host cores. Checks that every line parses, that both legs report, that the
program's own self-checks and its HIP-against-CPU comparisons passed, and that the figures are
plausible for the device (floors at about half of the measured rates). The eager forward pass of
the benchmark's transformer, issued from native host code, must reproduce the logits of the same
model driven through the Python mirror bit for bit (same backend calls in the same order)."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "honeycrisp_amd", "cpp", "HCMatrixBench")


def run(args, timeout=170):
    assert os.path.exists(BINARY), "build it with `python -m honeycrisp_amd.csrc.build`"
    print("running", BINARY, *args, flush=True)
    # (the program sets its own batching: a setting meant for this process's context stays here)
    env = {k: v for k, v in os.environ.items() if k != "HCHIP_BATCHING"}
    proc = subprocess.run([BINARY] + args, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout, env=env)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    return [dict(kv.split("=", 1) for kv in line.split()) for line in proc.stdout.strip().splitlines()], proc.stdout


OPS = {"bias_add", "gelu", "sum_axis1", "argmax_axis1", "max_axis1", "embedding_gather"}


def test_cpu_leg_alone_needs_no_gpu():
    """`--backend cpu`: the reference algorithms only (no context is created)."""
    lines, out = run(["--backend", "cpu", "--max-size", "512", "--cpu-seconds", "0.05"])
    assert lines[0]["backends"] == "CPUBackend" and lines[-1] == {"failures": "0"}
    ops = lines[1:-1]
    assert {r["op"] for r in ops} == OPS | {"matmul"}
    assert all("hip_us" not in r and float(r["cpu_us"]) > 0 for r in ops), out
    paths = {(r["dtype"], r["layout"]): r["cpu_path"] for r in ops if r["op"] == "matmul"}
    # BackendCPU.swift:1245: only the fp32 product without transposes goes to vDSP_mmul
    assert paths == {("float16", "NN"): "literal_loop", ("float16", "NT"): "literal_loop",
                     ("float32", "NN"): "vDSP_mmul", ("float32", "NT"): "literal_loop"}


@pytest.mark.gpu
def test_both_backends_report_and_agree():
    lines, out = run(["--backend", "both", "--iters", "5", "--max-size", "4096", "--cpu-seconds", "0.5"])
    assert lines[0]["backends"] == "HIPBackend+CPUBackend" and lines[-1] == {"failures": "0"}
    ops = lines[1:-1]
    assert all(r["check"] == "ok" and r["parity"] == "ok" for r in ops), out
    assert all(float(r["ratio"]) > 1.0 for r in ops), out
    matmuls = {(r["dtype"], r["layout"], int(r["size"])): r for r in ops if r["op"] == "matmul"}
    assert set(matmuls) == {(d, l, n) for d in ("float16", "float32") for l in ("NN", "NT") for n in (512, 1024, 2048, 4096)}
    for r in matmuls.values():
        assert float(r["cpu_gflops"]) > 0.05 and int(r["cpu_threads"]) >= 1
        done, total = map(int, r["cpu_rows"].split("/"))
        assert 2 <= done <= total == int(r["size"])
    # floors: about half of what the device measures through this program (host-timed, 5 calls and a wait)
    assert float(matmuls[("float16", "NN", 4096)]["hip_gflops"]) > 600e3
    assert float(matmuls[("float16", "NT", 4096)]["hip_gflops"]) > 600e3
    assert float(matmuls[("float32", "NN", 4096)]["hip_gflops"]) > 70e3
    bandwidth = {r["op"]: r for r in ops if r["op"] != "matmul"}
    assert set(bandwidth) == OPS
    floors = {"bias_add": 3000.0, "gelu": 3000.0, "sum_axis1": 2500.0, "argmax_axis1": 2500.0, "max_axis1": 2000.0,
              "embedding_gather": 3000.0}   # GB/s
    for op, r in bandwidth.items():
        assert float(r["hip_gbs"]) > floors[op], (op, r)
        assert int(r["cpu_threads"]) == 1 and float(r["cpu_gbs"]) > 0.05


def export_weights(model, path):
    """The model's parameters as float32, in the order honeycrisp_amd/cpp/transformer.hpp reads them."""
    def f32(t):
        return t.numpy().astype(np.float32).reshape(-1)

    def linear(l):
        return [f32(l.weight), f32(l.bias)]
    parts = [f32(model.table), f32(model.pos)]
    for b in model.blocks:
        parts += [f32(b.ln1.gain), f32(b.ln1.bias)] + linear(b.q) + linear(b.k) + linear(b.v) + linear(b.o)
        parts += [f32(b.ln2.gain), f32(b.ln2.bias)] + linear(b.fc1) + linear(b.fc2)
    parts += [f32(model.ln_f.gain), f32(model.ln_f.bias)] + linear(model.unembed)
    np.concatenate(parts).tofile(path)


@pytest.mark.gpu
@pytest.mark.parametrize("batching", [0, 128], ids=["eager", "batched"])
@pytest.mark.parametrize("dtype_name", ["f16", "f32"])
def test_native_eager_transformer_reproduces_the_python_path(hip_backend, tmp_path, dtype_name, batching):
    from honeycrisp_amd.descriptors import DType
    from honeycrisp_amd.nn import Transformer
    from honeycrisp_amd.tensor import Tensor
    dtype = DType.float16 if dtype_name == "f16" else DType.float32
    ids = np.random.default_rng(11).integers(0, 8192, size=(8, 256))
    with hip_backend.use():
        model = Transformer(dtype=dtype)
        want = model(Tensor(data=ids)).numpy()
        export_weights(model, str(tmp_path / "weights.bin"))
    ids.astype(np.int64).tofile(str(tmp_path / "ids.bin"))
    lines, out = run(["--transformer", "--dtype", dtype_name, "--iters", "5", "--weights", str(tmp_path / "weights.bin"),
                      "--ids", str(tmp_path / "ids.bin"), "--logits-out", str(tmp_path / "logits.bin"),
                      "--batching", str(batching)])
    (r,) = lines
    assert r["op"] == "transformer_forward" and int(r["tokens"]) == 2048
    assert r["mode"] == ("batched_native_host" if batching else "eager_native_host")
    if batching:    # the same calls, listed and rewritten batch by batch: fewer launches, the same bits
        assert int(r["launches_listed"]) == (256 if dtype_name == "f16" else 193)
        assert int(r["launches_enqueued"]) < int(r["launches_listed"]) // 3
    assert float(r["tokens_per_s"]) > 2.0e5, out
    got = np.fromfile(str(tmp_path / "logits.bin"), dtype=want.dtype).reshape(want.shape)
    assert np.array_equal(got.view(np.uint16 if dtype_name == "f16" else np.uint32),
                          want.view(np.uint16 if dtype_name == "f16" else np.uint32))
