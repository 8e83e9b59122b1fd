// Counterpart of the reference's HCMatrixBench (Sources/HCMatrixBench/Entrypoint.swift) for
// the MI355X backend: square fp16 / fp32 matmuls, one untimed warm-up call and then timed
// calls that end in wait(), FLOPs = 2 * M * N * K (Entrypoint.swift:16-26), printed as
// GFLOP/s per size. Inputs are seeded on the host; the CPUBackend leg of the comparison is
// run by bench.py (it times the CPU restatement of the reference algorithm).
//
// Build: g++ -O2 -std=c++17 HCMatrixBench.cpp -I../../include -L../csrc -lhchip -Wl,-rpath,'$ORIGIN/../csrc'
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "hip_backend.hpp"

static uint16_t to_half(float f) {
  // round-to-nearest-even conversion of a finite, moderate value (inputs are N(0,1)/sqrt(K))
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u, absx = x & 0x7fffffffu;
  if (absx < 0x38800000u) return (uint16_t)sign;  // below the normal half range: flush
  uint32_t res = (((absx >> 23) - 112u) << 10) | ((absx & 0x7fffffu) >> 13);
  const uint32_t rem = absx & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (res & 1u))) res++;
  return (uint16_t)(sign | res);
}

int main(int argc, char** argv) {
  const int iters = argc > 1 ? std::atoi(argv[1]) : 10;
  try {
    hc::HIPBackend backend(0);
    for (hc::DType dtype : {hc::DType::float16, hc::DType::float32}) {
      const std::vector<int> sizes = dtype == hc::DType::float16 ? std::vector<int>{512, 1024, 2048, 4096, 8192}
                                                                  : std::vector<int>{512, 1024, 2048, 4096};
      for (int n : sizes) {
        std::mt19937_64 gen(1);
        std::normal_distribution<float> dist(0.0f, 1.0f / std::sqrt((float)n));
        hc::Data a, b;
        if (dtype == hc::DType::float16) {
          std::vector<uint16_t> ha((size_t)n * n), hb((size_t)n * n);
          for (auto& v : ha) v = to_half(dist(gen));
          for (auto& v : hb) v = to_half(dist(gen));
          a = backend.upload(ha.data(), ha.size() * 2);
          b = backend.upload(hb.data(), hb.size() * 2);
        } else {
          std::vector<float> ha((size_t)n * n), hb((size_t)n * n);
          for (auto& v : ha) v = dist(gen);
          for (auto& v : hb) v = dist(gen);
          a = backend.upload(ha.data(), ha.size() * 4);
          b = backend.upload(hb.data(), hb.size() * 4);
        }
        backend.matmul(a, false, b, false, false, n, n, n, dtype);  // warm-up
        backend.wait();
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < iters; i++) backend.matmul(a, false, b, false, false, n, n, n, dtype);
        backend.wait();
        const auto t1 = std::chrono::steady_clock::now();
        const double ns = std::chrono::duration<double, std::nano>(t1 - t0).count() / iters;
        const double flops = 2.0 * n * n * (double)n;
        std::printf("%s size=%d gflops=%.1f\n", dtype == hc::DType::float16 ? "float16" : "float32", n, flops / ns);
      }
    }
  } catch (const hc::BackendError& e) {
    std::fprintf(stderr, "backend error (kind %d): %s\n", (int)e.kind, e.what());
    return 1;
  }
  return 0;
}
