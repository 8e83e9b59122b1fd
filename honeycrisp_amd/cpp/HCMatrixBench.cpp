// Counterpart of the reference's HCMatrixBench (Sources/HCMatrixBench/Entrypoint.swift:10-27: pick a
// backend, one untimed warm-up call, `iters` timed calls ending in wait(), FLOPs = 2 * M * N * K,
// GFLOP/s per backend) extended to drive BOTH backends on identical seeded inputs:
//   hip  the MI355X backend through the C++ mirror of the Backend interface (hip_backend.hpp);
//   cpu  the reference CPUBackend's algorithms on this machine's host cores (cpu_backend.hpp: one
//        thread, literal loops, Accelerate calls through the Linux stand-in; fp32 NN products go to
//        vDSP_mmul, i.e. an OpenBLAS sgemm when one is found, with its thread count printed).
// Workloads: square fp16 / fp32 products in the NN and NT layouts (config 1 and 2 sizes); the
// bandwidth-bound ops of a forward pass at [8192, 4096] fp32 (broadcast bias add, GELU, sum, argmax and
// max = argmax + gather over axis 1) and an int64 row gather of 65536 ids from a [32000, 1024] table
// (config 4); with --transformer, the eager forward pass of the 6-layer transformer (config 5) issued
// from native host code, tokens/s (--batching N: the same calls with the library's batching on).
// One `key=value` line per op with both rates, the ratio, a self-check of the HIP result (known sums /
// identities) and, when both backends ran, the parity of the two results on the rows the CPU computed.
// The scalar CPU loop takes minutes at 4096^3, so the CPU leg computes a slab of output rows sized to
// --cpu-seconds per product (cpu_rows=<computed>/<all>); its rate per row does not depend on the row.
//
// Usage: HCMatrixBench [--backend cpu|hip|both] [--iters N] [--max-size S] [--cpu-seconds T]
//                      [--transformer [--dtype f16|f32] [--batching N [--idle-after M]] [--weights FILE --ids FILE --logits-out FILE]]
// Build: see honeycrisp_amd/csrc/build.py (g++ -O2, links libhchip.so and the Accelerate stand-in).
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <functional>
#include <memory>
#include <random>
#include <string>
#include <vector>

#include "cpu_backend.hpp"
#include "hip_backend.hpp"
#include "transformer.hpp"

typedef std::chrono::steady_clock Clock;
static double seconds_since(Clock::time_point t0) { return std::chrono::duration<double>(Clock::now() - t0).count(); }

struct Options {
  bool hip = true, cpu = true, transformer = false;
  int iters = 10, max_size = 8192, batching = 0, idle_after = 0;
  double cpu_seconds = 2.0;
  std::string dtype = "f16", weights, ids, logits_out;
};

// seconds per call: one untimed call, then `iters` calls and one wait (Entrypoint.swift:16-24)
static double time_calls(hc::HIPBackend& backend, int iters, const std::function<void()>& call) {
  call();
  backend.wait();
  const auto t0 = Clock::now();
  for (int i = 0; i < iters; i++) call();
  backend.wait();
  return seconds_since(t0) / iters;
}

// |a - b| <= tol or |a / b - 1| <= tol (HCTestUtils/Assertions.swift:16)
static bool close(float a, float b, float tol) { return std::fabs(a - b) <= tol || (b != 0.0f && std::fabs(a / b - 1.0f) <= tol); }

static int bench_matmul(hc::HIPBackend* backend, const Options& opt) {
  int failures = 0;
  for (hc::DType dtype : {hc::DType::float16, hc::DType::float32}) {
    const bool f16 = dtype == hc::DType::float16;
    const size_t el = f16 ? 2 : 4;
    for (int n : {512, 1024, 2048, 4096, 8192}) {
      if (n > opt.max_size || (!f16 && n > 4096)) continue;
      std::mt19937_64 gen(1);
      std::normal_distribution<float> dist(0.0f, 1.0f / std::sqrt((float)n));
      std::vector<float> ha((size_t)n * n), hb((size_t)n * n);
      for (auto& v : ha) v = dist(gen);
      for (auto& v : hb) v = dist(gen);
      // the operands in the element type, as both backends receive them (same bytes)
      std::vector<char> a_bytes(ha.size() * el), b_bytes(hb.size() * el);
      hc::CPUBackend::writeFloats(ha.data(), ha.size(), dtype, a_bytes.data());
      hc::CPUBackend::writeFloats(hb.data(), hb.size(), dtype, b_bytes.data());
      hc::Data a, b;
      bool ok = true;
      if (backend) {
        a = backend->upload(a_bytes.data(), a_bytes.size());
        b = backend->upload(b_bytes.data(), b_bytes.size());
        // self-check: A x 2I == 2A exactly (doubling is exact in both types)
        std::vector<float> eye((size_t)n * n, 0.0f);
        for (int i = 0; i < n; i++) eye[(size_t)i * n + i] = 2.0f;
        std::vector<char> e_bytes(eye.size() * el);
        hc::CPUBackend::writeFloats(eye.data(), eye.size(), dtype, e_bytes.data());
        hc::Data e = backend->upload(e_bytes.data(), e_bytes.size());
        hc::Data c = backend->matmul(a, false, e, false, false, n, n, n, dtype);
        std::vector<char> c_bytes(a_bytes.size());
        backend->download(c, c_bytes.data(), c_bytes.size());
        const std::vector<float> got = hc::CPUBackend::readFloats(c_bytes.data(), ha.size(), dtype);
        const std::vector<float> src = hc::CPUBackend::readFloats(a_bytes.data(), ha.size(), dtype);
        for (size_t i = 0; i < got.size() && ok; i += 977) ok = got[i] == 2.0f * src[i];
        failures += !ok;
      }
      for (bool transB : {false, true}) {
        // B as the layout stores it: [K, N], or [N, K] for the NT layout (same product either way)
        std::vector<char> bt_bytes;
        hc::Data b_dev = b;
        const char* b_host = b_bytes.data();
        if (transB) {
          std::vector<float> t((size_t)n * n);
          const std::vector<float> bf = hc::CPUBackend::readFloats(b_bytes.data(), hb.size(), dtype);
          for (int i = 0; i < n; i++)
            for (int j = 0; j < n; j++) t[(size_t)j * n + i] = bf[(size_t)i * n + j];
          bt_bytes.resize(b_bytes.size());
          hc::CPUBackend::writeFloats(t.data(), t.size(), dtype, bt_bytes.data());
          b_host = bt_bytes.data();
          if (backend) b_dev = backend->upload(bt_bytes.data(), bt_bytes.size());
        }
        const double flops = 2.0 * n * n * (double)n;
        double hip_s = 0.0, cpu_s = 0.0;
        std::vector<float> hip_rows;
        int64_t rows_done = 0;
        if (backend) {
          hip_s = time_calls(*backend, opt.iters, [&] { backend->matmul(a, false, b_dev, transB, false, n, n, n, dtype); });
        }
        std::string parity = "n/a";
        const char* cpu_path = "";
        int cpu_threads = 1;
        if (opt.cpu) {
          // the reference's sequence: read both operands as Float (whole buffers), product, write back
          const auto t0 = Clock::now();
          const std::vector<float> af = hc::CPUBackend::readFloats(a_bytes.data(), ha.size(), dtype);
          const std::vector<float> bf = hc::CPUBackend::readFloats(b_host, hb.size(), dtype);
          const double convert_s = seconds_since(t0);
          const bool vdsp = !f16 && !transB;   // BackendCPU.swift:1245: vDSP_mmul only for fp32 without transposes
          std::vector<float> out;
          double loop_s;
          if (vdsp) {
            out.resize((size_t)n * n);
            hc::CPUBackend::matmulRows(af.data(), false, bf.data(), false, n, n, n, 0, n, true, out.data());   // (library warm-up)
            const auto t1 = Clock::now();
            hc::CPUBackend::matmulRows(af.data(), false, bf.data(), false, n, n, n, 0, n, true, out.data());
            loop_s = seconds_since(t1);
            rows_done = n;
            cpu_path = "vDSP_mmul";
            cpu_threads = std::max(1, hc_accelerate_blas_threads());
          } else {
            // rows in chunks of 2 until the budget is spent; the time per row does not depend on the row
            out.resize((size_t)n * n);
            const auto t1 = Clock::now();
            while (rows_done < n && (rows_done < 2 || seconds_since(t1) < opt.cpu_seconds)) {
              const int64_t r1 = std::min<int64_t>(n, rows_done + 2);
              hc::CPUBackend::matmulRows(af.data(), false, bf.data(), transB, n, n, n, rows_done, r1, false, out.data() + (size_t)rows_done * n);
              rows_done = r1;
            }
            loop_s = seconds_since(t1) * (double)n / (double)rows_done;   // all rows at the measured rate per row
            cpu_path = "literal_loop";
          }
          std::vector<char> out_bytes((size_t)rows_done * n * el);
          const auto t2 = Clock::now();
          hc::CPUBackend::writeFloats(out.data(), (size_t)rows_done * n, dtype, out_bytes.data());
          const double write_s = seconds_since(t2) * (double)n / (double)rows_done;
          cpu_s = convert_s + loop_s + write_s;
          if (backend) {
            hc::Data c = backend->matmul(a, false, b_dev, transB, false, n, n, n, dtype);
            std::vector<char> c_bytes((size_t)rows_done * n * el);
            backend->download(c, c_bytes.data(), c_bytes.size());
            const std::vector<float> got = hc::CPUBackend::readFloats(c_bytes.data(), (size_t)rows_done * n, dtype);
            const std::vector<float> want = hc::CPUBackend::readFloats(out_bytes.data(), (size_t)rows_done * n, dtype);
            bool same = true;
            for (size_t i = 0; i < got.size() && same; i++) same = close(got[i], want[i], f16 ? 1e-2f : 1e-4f);
            parity = same ? "ok" : "FAILED";
            failures += !same;
          }
        }
        std::printf("op=matmul dtype=%s layout=%s size=%d", f16 ? "float16" : "float32", transB ? "NT" : "NN", n);
        if (backend) std::printf(" hip_us=%.2f hip_gflops=%.1f", hip_s * 1e6, flops / hip_s / 1e9);
        if (opt.cpu)
          std::printf(" cpu_us=%.1f cpu_gflops=%.3f cpu_path=%s cpu_threads=%d cpu_rows=%lld/%d", cpu_s * 1e6, flops / cpu_s / 1e9,
                      cpu_path, cpu_threads, (long long)rows_done, n);
        if (backend && opt.cpu) std::printf(" ratio=%.1f parity=%s", cpu_s / hip_s, parity.c_str());
        if (backend) std::printf(" check=%s", ok ? "ok" : "FAILED");
        std::printf("\n");
        std::fflush(stdout);
      }
    }
  }
  return failures;
}

static int bench_bandwidth(hc::HIPBackend* backend, const Options& opt) {
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
  hc::Data x, bias;
  if (backend) x = backend->upload(hx.data(), hx.size() * 4), bias = backend->upload(hbias.data(), hbias.size() * 4);
  const hc::BroadcastStrides xs{{R, C}, {C, 1}}, bs{{R, C}, {0, 1}};
  const hc::ReduceDims dims{R, C, 1};
  const double nb = (double)(R * C * 4);
  // one line per op: `hip` and `cpu` each run the op once more than they time it and leave their result
  // in the vectors `compare` looks at
  auto line = [&](const char* op, const char* shape, double bytes, const std::function<void()>& hip_call,
                  const std::function<bool()>& hip_check, const std::function<void()>& cpu_call,
                  const std::function<bool()>& compare) {
    double hip_s = 0.0, cpu_s = 0.0;
    bool ok = true, same = true;
    if (backend) {
      hip_s = time_calls(*backend, opt.iters, hip_call);
      ok = hip_check();
      failures += !ok;
    }
    if (opt.cpu) {
      const auto t0 = Clock::now();
      cpu_call();
      cpu_s = seconds_since(t0);
    }
    std::printf("op=%s dtype=float32 shape=%s", op, shape);
    if (backend) std::printf(" hip_us=%.2f hip_gbs=%.1f", hip_s * 1e6, bytes / hip_s / 1e9);
    if (opt.cpu) std::printf(" cpu_us=%.1f cpu_gbs=%.3f cpu_threads=1", cpu_s * 1e6, bytes / cpu_s / 1e9);
    if (backend && opt.cpu) {
      same = compare();
      failures += !same;
      std::printf(" ratio=%.1f parity=%s", cpu_s / hip_s, same ? "ok" : "FAILED");
    }
    if (backend) std::printf(" check=%s", ok ? "ok" : "FAILED");
    std::printf("\n");
    std::fflush(stdout);
  };
  std::vector<float> hip_f((size_t)(R * C)), cpu_f((size_t)(R * C));
  std::vector<int64_t> hip_i((size_t)R), cpu_i((size_t)R);
  auto all_close = [&](size_t n, float tol) {
    for (size_t i = 0; i < n; i++)
      if (!close(hip_f[i], cpu_f[i], tol)) return false;
    return true;
  };
  line("bias_add", "8192x4096", 2 * nb + C * 4.0, [&] { backend->binaryOp({xs, x}, {bs, bias}, HC_ADD, F32); },
       [&] {
         backend->download(backend->binaryOp({xs, x}, {bs, bias}, HC_ADD, F32), hip_f.data(), hip_f.size() * 4);
         for (int64_t j = 0; j < C; j++)
           if (hip_f[(size_t)j] != hx[(size_t)j] + hbias[(size_t)j]) return false;
         return true;
       },
       [&] { hc::CPUBackend::add(hx.data(), xs, hbias.data(), bs, cpu_f.data()); },
       [&] { return std::memcmp(hip_f.data(), cpu_f.data(), hip_f.size() * 4) == 0; });   // an IEEE addition: same bits
  line("gelu", "8192x4096", 2 * nb, [&] { backend->elemwise(x, HC_GELU_APPROX, nullptr, (size_t)(R * C), F32); },
       [&] {
         backend->download(backend->elemwise(x, HC_GELU_APPROX, nullptr, (size_t)(R * C), F32), hip_f.data(), hip_f.size() * 4);
         for (int64_t j = 0; j < C; j++)   // gelu(x) lies between min(x, 0) - 0.2 and max(x, 0)
           if (!(hip_f[(size_t)j] <= std::max(hx[(size_t)j], 0.0f) + 1e-6f && hip_f[(size_t)j] >= std::min(hx[(size_t)j], 0.0f) - 0.2f))
             return false;
         return true;
       },
       [&] { hc::CPUBackend::geluApprox(hx.data(), R * C, cpu_f.data()); }, [&] { return all_close((size_t)(R * C), 1e-4f); });
  line("sum_axis1", "8192x4096", nb + R * 4.0, [&] { backend->reduce(x, HC_SUM, dims, F32); },
       [&] {
         backend->download(backend->reduce(x, HC_SUM, dims, F32), hip_f.data(), (size_t)R * 4);
         double ref = 0.0;
         for (int64_t j = 0; j < C; j++) ref += hx[(size_t)j];
         return std::fabs(hip_f[0] - ref) <= 1e-3 * std::max(1.0, std::fabs(ref)) + 1e-2;
       },
       [&] { hc::CPUBackend::sum(hx.data(), dims, cpu_f.data()); },
       [&] {   // the order of an fp32 sum is not fixed: 1e-4 of the row's sum of magnitudes
         for (int64_t r = 0; r < R; r++) {
           double mag = 0.0;
           for (int64_t j = 0; j < C; j++) mag += std::fabs(hx[(size_t)(r * C + j)]);
           if (std::fabs((double)hip_f[(size_t)r] - (double)cpu_f[(size_t)r]) > 1e-4 * mag) return false;
         }
         return true;
       });
  line("argmax_axis1", "8192x4096", nb + R * 8.0, [&] { backend->reduce(x, HC_ARGMAX, dims, F32); },
       [&] {
         backend->download(backend->reduce(x, HC_ARGMAX, dims, F32), hip_i.data(), hip_i.size() * 8);
         for (int64_t r = 0; r < R; r++)
           if (hip_i[(size_t)r] != (37 * r) % C) return false;
         return true;
       },
       [&] { hc::CPUBackend::argmax(hx.data(), dims, cpu_i.data()); }, [&] { return hip_i == cpu_i; });
  {
    // Tensor.max(axis:) = argmax + gather (ReduceRepeat.swift:201-209)
    const hc::BroadcastStrides pick{{R, 1}, {1, 0}};
    auto hip_max = [&] {
      hc::Data i = backend->reduce(x, HC_ARGMAX, dims, F32);
      return backend->gather(x, hc::ScatterGatherIndices{{R, C}, 1, {pick, i}}, F32);
    };
    line("max_axis1", "8192x4096", nb + R * 8.0 + R * 8.0 + R * 4.0 + R * 4.0, [&] { hip_max(); },
         [&] {
           backend->download(hip_max(), hip_f.data(), (size_t)R * 4);
           for (int64_t r = 0; r < R; r++)
             if (hip_f[(size_t)r] != 100.0f + (float)(r % 7)) return false;
           return true;
         },
         [&] {
           hc::CPUBackend::argmax(hx.data(), dims, cpu_i.data());
           hc::CPUBackend::gather(hx.data(), cpu_i.data(), pick, R, C, 1, 1, cpu_f.data());
         },
         [&] { return std::memcmp(hip_f.data(), cpu_f.data(), (size_t)R * 4) == 0; });
  }
  {
    const int64_t V = 32000, D = 1024, N = 65536;
    std::vector<float> table((size_t)(V * D));
    for (int64_t v = 0; v < V; v++)
      for (int64_t d = 0; d < D; d++) table[(size_t)(v * D + d)] = (float)v + (float)d / 2048.0f;
    std::vector<int64_t> ids((size_t)N);
    std::mt19937_64 g9(9);
    for (auto& v : ids) v = (int64_t)(g9() % (uint64_t)V);
    hc::Data t, di;
    if (backend) t = backend->upload(table.data(), table.size() * 4), di = backend->upload(ids.data(), ids.size() * 8);
    const hc::BroadcastStrides is{{N, D}, {1, 0}};
    std::vector<float> hip_rows((size_t)(N * D)), cpu_rows((size_t)(N * D));
    line("embedding_gather", "32000x1024_ids=65536", N * 8.0 + 2.0 * N * D * 4.0,
         [&] { backend->gather(t, hc::ScatterGatherIndices{{V, D}, 0, {is, di}}, F32); },
         [&] {
           backend->download(backend->gather(t, hc::ScatterGatherIndices{{V, D}, 0, {is, di}}, F32), hip_rows.data(), hip_rows.size() * 4);
           for (int64_t i = 0; i < N; i += 997)
             if (hip_rows[(size_t)(i * D + 5)] != (float)ids[(size_t)i] + 5.0f / 2048.0f) return false;
           return true;
         },
         [&] { hc::CPUBackend::gather(table.data(), ids.data(), is, 1, V, N, D, cpu_rows.data()); },
         [&] { return std::memcmp(hip_rows.data(), cpu_rows.data(), hip_rows.size() * 4) == 0; });
  }
  return failures;
}

template <typename T> static std::vector<T> read_file(const std::string& path) {
  std::ifstream f(path, std::ios::binary | std::ios::ate);
  if (!f) throw std::runtime_error("cannot open " + path);
  const std::streamsize bytes = f.tellg();
  f.seekg(0);
  std::vector<T> out((size_t)bytes / sizeof(T));
  f.read((char*)out.data(), bytes);
  return out;
}

// Config 5, eager: every op of a forward pass is a call into the backend from this program, the way a
// compiled Honeycrisp program issues them; tokens/s = 2048 / wall time of a pass ending in wait().
static int bench_transformer(hc::HIPBackend& backend, const Options& opt) {
  const hc::DType dtype = opt.dtype == "f32" ? hc::DType::float32 : hc::DType::float16;
  const hc::TransformerConfig cfg;
  const int64_t B = 8, T = cfg.seq;
  std::vector<float> weights;
  if (!opt.weights.empty()) {
    weights = read_file<float>(opt.weights);
    if ((int64_t)weights.size() != cfg.parameterCount()) {
      std::fprintf(stderr, "%s holds %zu values, the model has %lld\n", opt.weights.c_str(), weights.size(), (long long)cfg.parameterCount());
      return 1;
    }
  }
  std::vector<int64_t> ids;
  if (!opt.ids.empty()) {
    ids = read_file<int64_t>(opt.ids);
  } else {
    std::mt19937_64 g(11);
    ids.resize((size_t)(B * T));
    for (auto& v : ids) v = (int64_t)(g() % (uint64_t)cfg.vocab);
  }
  if ((int64_t)ids.size() != B * T) {
    std::fprintf(stderr, "expected %lld token ids\n", (long long)(B * T));
    return 1;
  }
  hc::Transformer model(backend, dtype, cfg, weights);
  hc::Data tokens = backend.upload(ids.data(), ids.size() * 8);
  backend.setBatching((size_t)opt.batching, (size_t)opt.idle_after);
  const auto stats0 = backend.batchingStats();
  hc::Data logits = model.forward(tokens, B);
  backend.wait();
  const auto stats1 = backend.batchingStats();
  if (!opt.logits_out.empty()) {
    std::vector<char> host((size_t)(B * T * cfg.vocab) * hc::byteSize(dtype));
    backend.download(logits, host.data(), host.size());
    std::ofstream(opt.logits_out, std::ios::binary).write(host.data(), (std::streamsize)host.size());
  }
  for (int i = 0; i < 3; i++) model.forward(tokens, B);
  backend.wait();
  const auto t0 = Clock::now();
  for (int i = 0; i < opt.iters; i++) {
    logits = model.forward(tokens, B);
    backend.wait();
  }
  const double s = seconds_since(t0) / opt.iters;
  // the same passes without a wait in between (the host runs ahead of the device): the enqueue rate
  const auto t1 = Clock::now();
  for (int i = 0; i < opt.iters; i++) logits = model.forward(tokens, B);
  const double enqueue_s = seconds_since(t1) / opt.iters;
  backend.wait();
  const double back_to_back_s = seconds_since(t1) / opt.iters;
  std::printf("op=transformer_forward mode=%s dtype=%s tokens=%lld us=%.1f tokens_per_s=%.1f "
              "us_back_to_back=%.1f tokens_per_s_back_to_back=%.1f host_enqueue_us=%.1f launches_listed=%llu launches_enqueued=%llu\n",
              opt.batching > 0 ? "batched_native_host" : "eager_native_host",
              dtype == hc::DType::float32 ? "float32" : "float16", (long long)(B * T), s * 1e6, (double)(B * T) / s,
              back_to_back_s * 1e6, (double)(B * T) / back_to_back_s, enqueue_s * 1e6,
              (unsigned long long)(stats1.first - stats0.first), (unsigned long long)(stats1.second - stats0.second));
  return 0;
}

int main(int argc, char** argv) {
  Options opt;
  for (int i = 1; i < argc; i++) {
    const std::string a = argv[i];
    auto value = [&]() -> std::string {
      if (i + 1 >= argc) {
        std::fprintf(stderr, "%s needs a value\n", a.c_str());
        std::exit(2);
      }
      return argv[++i];
    };
    if (a == "--backend") {
      const std::string b = value();
      if (b != "cpu" && b != "hip" && b != "both") {
        std::fprintf(stderr, "--backend cpu|hip|both\n");
        return 2;
      }
      opt.hip = b != "cpu", opt.cpu = b != "hip";
    } else if (a == "--iters") opt.iters = std::atoi(value().c_str());
    else if (a == "--max-size") opt.max_size = std::atoi(value().c_str());
    else if (a == "--cpu-seconds") opt.cpu_seconds = std::atof(value().c_str());
    else if (a == "--transformer") opt.transformer = true;
    else if (a == "--dtype") opt.dtype = value();
    else if (a == "--weights") opt.weights = value();
    else if (a == "--ids") opt.ids = value();
    else if (a == "--logits-out") opt.logits_out = value();
    else if (a == "--batching") opt.batching = std::atoi(value().c_str());
    else if (a == "--idle-after") opt.idle_after = std::atoi(value().c_str());
    else {
      std::fprintf(stderr, "unknown argument %s\n", a.c_str());
      return 2;
    }
  }
  try {
    std::unique_ptr<hc::HIPBackend> backend;
    if (opt.hip) backend.reset(new hc::HIPBackend(0));
    if (opt.transformer) {
      if (!backend) {
        std::fprintf(stderr, "--transformer runs on the HIP backend\n");
        return 2;
      }
      return bench_transformer(*backend, opt);
    }
    std::printf("backends=%s%s%s iters=%d cpu_blas=%s\n", opt.hip ? "HIPBackend" : "", opt.hip && opt.cpu ? "+" : "",
                opt.cpu ? "CPUBackend" : "", opt.iters, opt.cpu ? hc_accelerate_blas_backend() : "n/a");
    int failures = bench_matmul(backend.get(), opt);
    failures += bench_bandwidth(backend.get(), opt);
    std::printf("failures=%d\n", failures);
    return failures == 0 ? 0 : 1;
  } catch (const hc::BackendError& e) {
    std::fprintf(stderr, "backend error (kind %d): %s\n", (int)e.kind, e.what());
    return 2;
  } catch (const std::exception& e) {
    std::fprintf(stderr, "error: %s\n", e.what());
    return 2;
  }
}
