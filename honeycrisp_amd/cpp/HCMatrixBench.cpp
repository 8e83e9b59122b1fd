// Counterpart of the reference's HCMatrixBench (Sources/HCMatrixBench/Entrypoint.swift) for
// the MI355X backend, through the C++ mirror of the Backend interface (hip_backend.hpp):
//   * square fp16 / fp32 matmuls in the NN and NT layouts: one untimed warm-up call, then `iters`
//     timed calls ending in wait(), FLOPs = 2 * M * N * K (Entrypoint.swift:16-26), GFLOP/s;
//   * the bandwidth-bound ops of a forward pass at [8192, 4096] fp32 (broadcast bias add, GELU,
//     sum and argmax over axis 1, max = argmax + gather) and an int64 row gather of 65536 ids from
//     a [32000, 1024] table, timed the same way, GB/s = algorithmic bytes / time.
// Inputs are seeded on the host. Every result line is `key=value` pairs so that a caller can
// parse it; a one-line self-check of each result (known sums / identities) guards against a
// benchmark of a kernel that did nothing. The CPUBackend leg of the comparison needs the
// reference's Swift code: the Swift HCMatrixBench of this package runs both backends, and
// bench.py times the CPU restatement next to the GPU figures.
//
// Usage: HCMatrixBench [iters=10] [max_size=8192]
// Build: g++ -O2 -std=c++17 HCMatrixBench.cpp -L../csrc -lhchip -Wl,-rpath,'$ORIGIN/../csrc'
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>
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

static float from_half(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 1023u;
  float out;
  if (e == 0) {
    out = std::ldexp((float)m, -24);
  } else {
    const uint32_t bits = ((e + 112u) << 23) | (m << 13);
    std::memcpy(&out, &bits, 4);
  }
  return sign ? -out : out;
}

// seconds per call: one untimed call, then `iters` calls and one wait
static double time_calls(hc::HIPBackend& backend, int iters, const std::function<void()>& call) {
  call();
  backend.wait();
  const auto t0 = std::chrono::steady_clock::now();
  for (int i = 0; i < iters; i++) call();
  backend.wait();
  const auto t1 = std::chrono::steady_clock::now();
  return std::chrono::duration<double>(t1 - t0).count() / iters;
}

static int bench_matmul(hc::HIPBackend& backend, int iters, int max_size) {
  int failures = 0;
  for (hc::DType dtype : {hc::DType::float16, hc::DType::float32}) {
    const bool f16 = dtype == hc::DType::float16;
    for (int n : {512, 1024, 2048, 4096, 8192}) {
      if (n > max_size || (!f16 && n > 4096)) continue;
      std::mt19937_64 gen(1);
      std::normal_distribution<float> dist(0.0f, 1.0f / std::sqrt((float)n));
      // B is the identity scaled by 2 in the self-check launch, random in the timed ones
      std::vector<float> ha((size_t)n * n), hb((size_t)n * n), eye((size_t)n * n, 0.0f);
      for (auto& v : ha) v = dist(gen);
      for (auto& v : hb) v = dist(gen);
      for (int i = 0; i < n; i++) eye[(size_t)i * n + i] = 2.0f;
      auto up = [&](const std::vector<float>& h) {
        if (!f16) return backend.upload(h.data(), h.size() * 4);
        std::vector<uint16_t> hh(h.size());
        for (size_t i = 0; i < h.size(); i++) hh[i] = to_half(h[i]);
        return backend.upload(hh.data(), hh.size() * 2);
      };
      hc::Data a = up(ha), b = up(hb), e = up(eye);
      // self-check: A x 2I == 2A exactly (doubling is exact in both types)
      hc::Data c = backend.matmul(a, false, e, false, false, n, n, n, dtype);
      const size_t probe = (size_t)(n / 2) * n + n / 3;
      float got, want;
      if (f16) {
        std::vector<uint16_t> all((size_t)n * n);
        backend.download(c, all.data(), all.size() * 2);
        got = from_half(all[probe]);
        want = 2.0f * from_half(to_half(ha[probe]));
      } else {
        std::vector<float> all((size_t)n * n);
        backend.download(c, all.data(), all.size() * 4);
        got = all[probe];
        want = 2.0f * ha[probe];
      }
      const bool ok = got == want;
      failures += !ok;
      for (bool transB : {false, true}) {
        const double s = time_calls(backend, iters, [&] { backend.matmul(a, false, b, transB, false, n, n, n, dtype); });
        const double flops = 2.0 * n * n * (double)n;
        std::printf("op=matmul dtype=%s layout=%s size=%d us=%.2f gflops=%.1f check=%s\n", f16 ? "float16" : "float32",
                    transB ? "NT" : "NN", n, s * 1e6, flops / s / 1e9, ok ? "ok" : "FAILED");
      }
    }
  }
  return failures;
}

static int bench_bandwidth(hc::HIPBackend& backend, int iters) {
  const int64_t R = 8192, C = 4096;
  const hc::DType F32 = hc::DType::float32;
  int failures = 0;
  std::mt19937_64 gen(7);
  std::normal_distribution<float> dist(0.0f, 1.0f);
  std::vector<float> hx((size_t)(R * C)), hbias((size_t)C);
  for (auto& v : hx) v = dist(gen);
  for (auto& v : hbias) v = dist(gen);
  // plant known extrema: row r has its maximum 100 + r % 7 at column (37 r) % C
  for (int64_t r = 0; r < R; r++) hx[(size_t)(r * C + (37 * r) % C)] = 100.0f + (float)(r % 7);
  hc::Data x = backend.upload(hx.data(), hx.size() * 4), bias = backend.upload(hbias.data(), hbias.size() * 4);
  const hc::BroadcastStrides xs{{R, C}, {C, 1}}, bs{{R, C}, {0, 1}};
  const hc::ReduceDims dims{R, C, 1};
  const double nb = (double)(R * C * 4);
  auto line = [&](const char* op, double seconds, double bytes, bool ok) {
    failures += !ok;
    std::printf("op=%s dtype=float32 shape=%lldx%lld us=%.2f gbs=%.1f check=%s\n", op, (long long)R, (long long)C,
                seconds * 1e6, bytes / seconds / 1e9, ok ? "ok" : "FAILED");
  };
  {
    hc::Data out = backend.binaryOp({xs, x}, {bs, bias}, HC_ADD, F32);
    std::vector<float> row((size_t)C);
    backend.download(out, row.data(), row.size() * 4);
    bool ok = true;
    for (int64_t j = 0; j < C; j++) ok = ok && row[(size_t)j] == hx[(size_t)j] + hbias[(size_t)j];
    line("bias_add", time_calls(backend, iters, [&] { backend.binaryOp({xs, x}, {bs, bias}, HC_ADD, F32); }),
         2 * nb + C * 4.0, ok);
  }
  {
    hc::Data out = backend.elemwise(x, HC_GELU_APPROX, nullptr, (size_t)(R * C), F32);
    std::vector<float> row((size_t)C);
    backend.download(out, row.data(), row.size() * 4);
    bool ok = true;  // gelu(x) lies between min(x, 0) - 0.2 and max(x, 0)
    for (int64_t j = 0; j < C; j++)
      ok = ok && row[(size_t)j] <= std::max(hx[(size_t)j], 0.0f) + 1e-6f && row[(size_t)j] >= std::min(hx[(size_t)j], 0.0f) - 0.2f;
    line("gelu", time_calls(backend, iters, [&] { backend.elemwise(x, HC_GELU_APPROX, nullptr, (size_t)(R * C), F32); }),
         2 * nb, ok);
  }
  {
    hc::Data out = backend.reduce(x, HC_SUM, dims, F32);
    std::vector<float> sums((size_t)R);
    backend.download(out, sums.data(), sums.size() * 4);
    double ref = 0.0;
    for (int64_t j = 0; j < C; j++) ref += hx[(size_t)j];
    line("sum_axis1", time_calls(backend, iters, [&] { backend.reduce(x, HC_SUM, dims, F32); }), nb + R * 4.0,
         std::fabs(sums[0] - ref) <= 1e-3 * std::max(1.0, std::fabs(ref)) + 1e-2);
  }
  {
    hc::Data out = backend.reduce(x, HC_ARGMAX, dims, F32);
    std::vector<int64_t> idx((size_t)R);
    backend.download(out, idx.data(), idx.size() * 8);
    bool ok = true;
    for (int64_t r = 0; r < R; r++) ok = ok && idx[(size_t)r] == (37 * r) % C;
    line("argmax_axis1", time_calls(backend, iters, [&] { backend.reduce(x, HC_ARGMAX, dims, F32); }), nb + R * 8.0, ok);
    // Tensor.max(axis:) = argmax + gather (ReduceRepeat.swift:201-209)
    auto max_axis1 = [&] {
      hc::Data i = backend.reduce(x, HC_ARGMAX, dims, F32);
      return backend.gather(x, hc::ScatterGatherIndices{{R, C}, 1, {hc::BroadcastStrides{{R, 1}, {1, 0}}, i}}, F32);
    };
    hc::Data mx = max_axis1();
    std::vector<float> vals((size_t)R);
    backend.download(mx, vals.data(), vals.size() * 4);
    ok = true;
    for (int64_t r = 0; r < R; r++) ok = ok && vals[(size_t)r] == 100.0f + (float)(r % 7);
    line("max_axis1", time_calls(backend, iters, [&] { max_axis1(); }), nb + R * 8.0 + R * 8.0 + R * 4.0 + R * 4.0, ok);
  }
  {
    const int64_t V = 32000, D = 1024, N = 65536;
    std::vector<float> table((size_t)(V * D));
    for (int64_t v = 0; v < V; v++)
      for (int64_t d = 0; d < D; d++) table[(size_t)(v * D + d)] = (float)v + (float)d / 2048.0f;
    std::vector<int64_t> ids((size_t)N);
    std::mt19937_64 g9(9);
    for (auto& v : ids) v = (int64_t)(g9() % (uint64_t)V);
    hc::Data t = backend.upload(table.data(), table.size() * 4), di = backend.upload(ids.data(), ids.size() * 8);
    const hc::ScatterGatherIndices emb{{V, D}, 0, {hc::BroadcastStrides{{N, D}, {1, 0}}, di}};
    hc::Data out = backend.gather(t, emb, F32);
    std::vector<float> rows((size_t)(N * D));
    backend.download(out, rows.data(), rows.size() * 4);
    bool ok = true;
    for (int64_t i = 0; i < N; i += 997) ok = ok && rows[(size_t)(i * D + 5)] == (float)ids[(size_t)i] + 5.0f / 2048.0f;
    const double s = time_calls(backend, iters, [&] { backend.gather(t, emb, F32); });
    failures += !ok;
    std::printf("op=embedding_gather dtype=float32 shape=%lldx%lld ids=%lld us=%.2f gbs=%.1f check=%s\n", (long long)V,
                (long long)D, (long long)N, s * 1e6, (N * 8.0 + 2.0 * N * D * 4.0) / s / 1e9, ok ? "ok" : "FAILED");
  }
  return failures;
}

int main(int argc, char** argv) {
  const int iters = argc > 1 ? std::atoi(argv[1]) : 10;
  const int max_size = argc > 2 ? std::atoi(argv[2]) : 8192;
  try {
    hc::HIPBackend backend(0);
    std::printf("backend=HIPBackend iters=%d\n", iters);
    int failures = bench_matmul(backend, iters, max_size);
    failures += bench_bandwidth(backend, iters);
    std::printf("failures=%d\n", failures);
    return failures == 0 ? 0 : 1;
  } catch (const hc::BackendError& e) {
    std::fprintf(stderr, "backend error (kind %d): %s\n", (int)e.kind, e.what());
    return 2;
  }
}
