// The benchmark's decoder-only transformer (6 layers, d_model 512, 8 heads, MLP 2048, vocab 8192,
// batch 8 x seq 256, causal mask) as the sequence of backend calls that a Honeycrisp program
// written with `Linear` (Trainable.swift:508-547), `LayerNorm` (:787-829) and Tensor ops emits, issued
// eagerly from native host code through the C++ mirror of the Backend interface. Same calls, in the
// same order, with the same shapes and strides as honeycrisp_amd/nn.py issues through the Python
// mirror, so the two produce the same bits from the same weights; what differs is the cost of the
// host code between two backend calls.
#pragma once

#include <cmath>
#include <cstdio>
#include <random>
#include <vector>

#include "hip_backend.hpp"

namespace hc {

struct TransformerConfig {
  int64_t layers = 6, d_model = 512, heads = 8, mlp = 2048, vocab = 8192, seq = 256;
  // float32 values a weight file holds, in the order Transformer reads them
  int64_t parameterCount() const {
    const int64_t d = d_model;
    const int64_t block = 2 * d + 4 * (d * d + d) + 2 * d + (d * mlp + mlp) + (mlp * d + d);
    return vocab * d + seq * d + layers * block + 2 * d + (d * vocab + vocab);
  }
};

class Transformer {
 public:
  // `weights`: parameterCount() float32 values (table, positions, per block: ln1 gain, ln1 bias, q, k, v,
  // o as weight then bias, ln2 gain, ln2 bias, fc1, fc2; final LayerNorm; unembedding), or empty for
  // seeded random values with Linear's initialisation.
  Transformer(HIPBackend& backend, DType dtype, const TransformerConfig& cfg, const std::vector<float>& weights)
      : be_(backend), dtype_(dtype), c_(cfg) {
    std::vector<float> generated;
    const float* w = weights.data();
    if (weights.empty()) {
      generated = randomWeights();
      w = generated.data();
    }
    size_t at = 0;
    auto take = [&](int64_t n, bool model_dtype) {
      Data d = be_.upload(w + at, (size_t)n * 4);
      at += (size_t)n;
      return model_dtype && dtype_ != DType::float32 ? be_.cast(d, (size_t)n, DType::float32, dtype_) : d;
    };
    auto linear = [&](int64_t in, int64_t out) {
      LinearP l;
      l.in = in, l.out = out;
      l.w = take(in * out, true);
      l.b = take(out, false);   // biases stay fp32 and are cast at call time (castParams)
      return l;
    };
    const int64_t d = c_.d_model;
    table_ = take(c_.vocab * d, true);
    pos_ = take(c_.seq * d, true);
    for (int64_t i = 0; i < c_.layers; i++) {
      BlockP b;
      b.ln1 = {take(d, false), take(d, false)};
      b.q = linear(d, d), b.k = linear(d, d), b.v = linear(d, d), b.o = linear(d, d);
      b.ln2 = {take(d, false), take(d, false)};
      b.fc1 = linear(d, c_.mlp), b.fc2 = linear(c_.mlp, d);
      blocks_.push_back(b);
    }
    lnf_ = {take(d, false), take(d, false)};
    unembed_ = linear(d, c_.vocab);
    // causal mask [T, T]: 0 on and below the diagonal, -1e4 above (finite in fp16); built once
    const int64_t T = c_.seq;
    std::vector<float> m((size_t)(T * T));
    for (int64_t i = 0; i < T; i++)
      for (int64_t j = 0; j < T; j++) m[(size_t)(i * T + j)] = i >= j ? 0.0f : -1e4f;
    Data m32 = be_.upload(m.data(), m.size() * 4);
    mask_ = dtype_ == DType::float32 ? m32 : be_.cast(m32, m.size(), DType::float32, dtype_);
  }

  // ids: int64 [B, T] on the device, T == seq. Returns logits [B, T, vocab] in the model's dtype.
  Data forward(const Data& ids, int64_t B) {
    const int64_t T = c_.seq, D = c_.d_model, H = c_.heads, hd = D / H, rows = B * T;
    const ScatterGatherIndices emb{{c_.vocab, D}, 0, {BroadcastStrides{{rows, D}, {1, 0}}, ids}};
    Data x = be_.gather(table_, emb, dtype_);
    x = be_.binaryOp({dense({B, T, D}), x}, {BroadcastStrides{{B, T, D}, {0, D, 1}}, pos_}, HC_ADD, dtype_);
    for (const BlockP& b : blocks_) {
      Data h = layerNorm(b.ln1, x, B, T);
      Data q = splitHeads(linear(b.q, h, rows), B, T, H, hd);
      Data k = splitHeads(linear(b.k, h, rows), B, T, H, hd);
      Data v = splitHeads(linear(b.v, h, rows), B, T, H, hd);
      const size_t n_scores = (size_t)(B * H * T * T);
      Data scores = be_.batchedMatmul(B * H, q, false, k, true, false, T, hd, T, dtype_);
      scores = be_.binaryOp(scores, 1.0f / std::sqrt((float)hd), HC_MUL, n_scores, dtype_);
      scores = be_.binaryOp({dense({B, H, T, T}), scores}, {BroadcastStrides{{B, H, T, T}, {0, 0, T, 1}}, mask_}, HC_ADD, dtype_);
      Data probs = be_.elemwise(be_.logSoftmax(scores, ReduceDims{B * H * T, T, 1}, dtype_), HC_EXP, nullptr, n_scores, dtype_);
      Data ctx = be_.batchedMatmul(B * H, probs, false, v, false, false, T, T, hd, dtype_);
      ctx = swapAxes(ctx, B, H, T, hd);
      x = be_.binaryOp({dense({B, T, D}), x}, {dense({B, T, D}), linear(b.o, ctx, rows)}, HC_ADD, dtype_);
      Data f = linear(b.fc1, layerNorm(b.ln2, x, B, T), rows);
      f = be_.elemwise(f, HC_GELU_APPROX, nullptr, (size_t)(rows * c_.mlp), dtype_);
      x = be_.binaryOp({dense({B, T, D}), x}, {dense({B, T, D}), linear(b.fc2, f, rows)}, HC_ADD, dtype_);
    }
    return linear(unembed_, layerNorm(lnf_, x, B, T), rows);
  }

  // (rand - 0.5) * (sqrt(3) / 0.5 / sqrt(in)) for Linear weights, zero biases (Trainable.swift:520-527),
  // small random LayerNorm parameters so that the affine part is exercised
  std::vector<float> randomWeights() const {
    std::vector<float> w((size_t)c_.parameterCount());
    std::mt19937_64 gen(12);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    std::normal_distribution<float> normal(0.0f, 1.0f);
    size_t at = 0;
    auto fill = [&](int64_t n, const std::function<float()>& f) {
      for (int64_t i = 0; i < n; i++) w[at++] = f();
    };
    auto linear = [&](int64_t in, int64_t out) {
      const float scale = std::sqrt(3.0f) / 0.5f / std::sqrt((float)in);
      fill(in * out, [&] { return (uni(gen) - 0.5f) * scale; });
      fill(out, [] { return 0.0f; });
    };
    const int64_t d = c_.d_model;
    fill(c_.vocab * d, [&] { return 0.02f * normal(gen); });
    fill(c_.seq * d, [&] { return 0.02f * normal(gen); });
    for (int64_t i = 0; i < c_.layers; i++) {
      fill(2 * d, [&] { return 0.1f * normal(gen); });
      linear(d, d), linear(d, d), linear(d, d), linear(d, d);
      fill(2 * d, [&] { return 0.1f * normal(gen); });
      linear(d, c_.mlp), linear(c_.mlp, d);
    }
    fill(2 * d, [&] { return 0.1f * normal(gen); });
    linear(d, c_.vocab);
    return w;
  }

 private:
  struct LinearP {
    Data w, b;
    int64_t in = 0, out = 0;
  };
  struct LayerNormP {
    Data gain, bias;
  };
  struct BlockP {
    LayerNormP ln1, ln2;
    LinearP q, k, v, o, fc1, fc2;
  };
  static BroadcastStrides dense(const std::vector<int64_t>& shape) { return BroadcastStrides::contiguous(shape); }

  // Linear.callAsFunction: matmul, then + bias cast to the activations' type
  Data linear(const LinearP& l, const Data& x, int64_t rows) {
    Data h = be_.matmul(x, false, l.w, false, false, rows, l.in, l.out, dtype_);
    Data bias = dtype_ == DType::float32 ? l.b : be_.cast(l.b, (size_t)l.out, DType::float32, dtype_);
    return be_.binaryOp({dense({rows, l.out}), h}, {BroadcastStrides{{rows, l.out}, {0, 1}}, bias}, HC_ADD, dtype_);
  }
  // LayerNorm.callAsFunction: cast to fp32, normalize, (gain + 1) * x + bias, cast back
  Data layerNorm(const LayerNormP& p, const Data& x, int64_t B, int64_t T) {
    const int64_t D = c_.d_model, rows = B * T;
    Data x32 = dtype_ == DType::float32 ? x : be_.cast(x, (size_t)(rows * D), dtype_, DType::float32);
    Data n = be_.normalize(x32, ReduceDims{rows, D, 1}, 1e-5f, DType::float32);
    Data gain1 = be_.binaryOp(p.gain, 1, HC_ADD, (size_t)D, DType::float32);
    const BroadcastStrides row{{B, T, D}, {0, 0, 1}};
    Data y = be_.mulAdd({dense({B, T, D}), n}, {row, gain1}, {row, p.bias}, DType::float32);
    return dtype_ == DType::float32 ? y : be_.cast(y, (size_t)(rows * D), DType::float32, dtype_);
  }
  // [B, T, H, hd] -> [B, H, T, hd]: .swap(axis: 1, with: 2), i.e. axisPermutation + a gather of hd-element
  // rows (Index.swift:238-266, 365-376)
  Data splitHeads(const Data& x, int64_t B, int64_t T, int64_t H, int64_t hd) { return swapAxes(x, B, T, H, hd); }
  Data swapAxes(const Data& x, int64_t B, int64_t a1, int64_t a2, int64_t inner) {
    Data perm = be_.axisPermutation({1, 0}, {a1, a2});
    const ScatterGatherIndices s{{B, a1 * a2, inner}, 1, {BroadcastStrides{{B, a1 * a2, inner}, {0, 1, 0}}, perm}};
    return be_.gather(x, s, dtype_);
  }

  HIPBackend& be_;
  DType dtype_;
  TransformerConfig c_;
  Data table_, pos_, mask_;
  std::vector<BlockP> blocks_;
  LayerNormP lnf_;
  LinearP unembed_;
};

}  // namespace hc
