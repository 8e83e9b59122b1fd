// HCMatrixBench extended to drive both backends (reference: Sources/HCMatrixBench/
// Entrypoint.swift, which is hard-wired to MPSBackend). Same method: one untimed warm-up call,
// then a timed call ending in `try await result.wait()`, FLOPs = 2*M*N*K, GFLOP/s printed per
// backend plus the ratio, followed by the bandwidth-bound ops of a forward pass with GB/s. The
// input tensors are created once and reused under both backends (foreign Tensor.Data is legal
// input), so both see identical values. Not compiled anywhere yet (no Swift toolchain at hand).
import Foundation
import Honeycrisp
import HoneycrispHIP

@main
struct Main {
  static func time(_ backend: Backend, _ m1: Tensor, _ m2: Tensor) async throws -> Double {
    try await backend.use {
      let warm = m1 &* m2
      try await warm.wait()
      let t0 = DispatchTime.now()
      let result = m1 &* m2
      try await result.wait()
      let t1 = DispatchTime.now()
      return Double(t1.uptimeNanoseconds - t0.uptimeNanoseconds)
    }
  }

  static func main() async {
    do {
      let hip = try HIPBackend()
      let cpu = CPUBackend.global
      print("host cores: \(ProcessInfo.processInfo.activeProcessorCount) (CPUBackend runs one worker thread)")
      for dtype: Tensor.DType in [.float16, .float32] {
        for size in [256, 512, 1024, 2048, 4096] {
          let (m1, m2) = cpu.use {
            cpu.defaultRandom().seed(size)
            return (
              Tensor(randn: [size, size], dtype: dtype) * (1 / Float(size).squareRoot()),
              Tensor(randn: [size, size], dtype: dtype)
            )
          }
          let flops = 2.0 * Double(size) * Double(size) * Double(size)
          let hipNs = try await time(hip, m1, m2)
          // the scalar CPU path is minutes at 4096^3 for fp16: cap the CPU leg at 1024
          let cpuNs = size <= 1024 ? try await time(cpu, m1, m2) : Double.nan
          print(
            "\(dtype) size=\(size) hip_gflops=\(flops / hipNs) cpu_gflops=\(flops / cpuNs) "
              + "speedup=\(cpuNs / hipNs)")
        }
      }
      try await bandwidthOps(hip: hip, cpu: cpu)
    } catch {
      print("FATAL ERROR: \(error)")
    }
  }

  /// Seconds for `fn` under `backend`: one untimed call, then one timed call ending in wait().
  static func time(_ backend: Backend, _ fn: () -> Tensor) async throws -> Double {
    try await backend.use {
      try await fn().wait()
      let t0 = DispatchTime.now()
      try await fn().wait()
      return Double(DispatchTime.now().uptimeNanoseconds - t0.uptimeNanoseconds) / 1e9
    }
  }

  /// The bandwidth-bound ops of a forward pass at [8192, 4096] fp32 and an int64 row gather from a
  /// [32000, 1024] table: GB/s = algorithmic bytes / time, per backend, and the ratio. The same
  /// tensors (created once under the CPU backend) feed both; foreign Tensor.Data is legal input.
  static func bandwidthOps(hip: HIPBackend, cpu: Backend) async throws {
    let (rows, cols) = (8192, 4096)
    let (x, bias, table, ids) = cpu.use {
      cpu.defaultRandom().seed(7)
      return (
        Tensor(randn: [rows, cols]), Tensor(randn: [1, cols]), Tensor(randn: [32000, 1024]),
        Tensor(data: (0..<65536).map { ($0 * 7919) % 32000 }, shape: [65536])
      )
    }
    // uploaded once, so that the timed calls do not measure the PCIe copy
    let onHIP = hip.use { (x + 0, bias + 0, table + 0, ids + 0) }
    let nb = Double(rows * cols * 4)
    let ops: [(String, Double, (Tensor, Tensor, Tensor, Tensor) -> Tensor)] = [
      ("bias_add", 2 * nb + Double(cols * 4), { x, b, _, _ in x + b }),
      ("gelu", 2 * nb, { x, _, _, _ in x.gelu() }),
      ("sum_axis1", nb + Double(rows * 4), { x, _, _, _ in x.sum(axis: 1) }),
      ("argmax_axis1", nb + Double(rows * 8), { x, _, _, _ in x.argmax(axis: 1) }),
      ("max_axis1", nb + Double(rows * 24), { x, _, _, _ in x.max(axis: 1) }),
      ("embedding_gather", Double(65536 * 8 + 2 * 65536 * 1024 * 4), { _, _, t, i in t.gather(axis: 0, indices: i) }),
    ]
    for (name, bytes, op) in ops {
      let hipS = try await time(hip) { op(onHIP.0, onHIP.1, onHIP.2, onHIP.3) }
      let cpuS = try await time(cpu) { op(x, bias, table, ids) }
      print("\(name) hip_gbs=\(bytes / hipS / 1e9) cpu_gbs=\(bytes / cpuS / 1e9) speedup=\(cpuS / hipS)")
    }
  }
}
