// HCMatrixBench extended to drive both backends (reference: Sources/HCMatrixBench/
// Entrypoint.swift, which is hard-wired to MPSBackend). Same method: one untimed warm-up call,
// then a timed call ending in `try await result.wait()`, FLOPs = 2*M*N*K, GFLOP/s printed per
// backend plus the ratio. The input tensors are created once and reused under both backends
// (foreign Tensor.Data is legal input), so both see identical values.
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
    } catch {
      print("FATAL ERROR: \(error)")
    }
  }
}
