// C++ mirror of Honeycrisp's `Backend` op interface for the MI355X backend: same method names
// and argument meaning as the open class in Sources/Honeycrisp/Backend.swift:170-815, errors
// mapped onto the BackendError cases of Backend.swift:6-16. Header-only, on top of the C ABI
// (include/hchip.h); every method enqueues on the context's in-order stream and returns a
// device buffer (`Data`, the counterpart of Tensor.Data, Tensor.swift:69-85) immediately.
#pragma once

#include <cstdint>
#include <cstring>
#include <functional>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/hchip.h"

namespace hc {

enum class DType : int { int64 = HC_I64, boolean = HC_BOOL, float16 = HC_F16, float32 = HC_F32 };
inline size_t byteSize(DType t) {
  switch (t) {
    case DType::int64: return 8;
    case DType::boolean: return 1;
    case DType::float16: return 2;
    default: return 4;
  }
}

struct BackendError : std::runtime_error {
  enum Kind { notImplemented, allocationFailed, kernelFailed, failedToLoadKernels } kind;
  BackendError(Kind k, const std::string& msg) : std::runtime_error(msg), kind(k) {}
};

// BroadcastStrides (Broadcast.swift:9-30).
struct BroadcastStrides {
  std::vector<int64_t> shape, strides;
  static BroadcastStrides contiguous(const std::vector<int64_t>& shape) {
    BroadcastStrides s{shape, std::vector<int64_t>(shape.size())};
    int64_t acc = 1;
    for (size_t i = shape.size(); i-- > 0;) {
      s.strides[i] = acc;
      acc *= shape[i];
    }
    return s;
  }
  int64_t count() const {
    int64_t n = 1;
    for (int64_t d : shape) n *= d;
    return n;
  }
  hc_strides c() const {
    if (shape.size() > HC_MAX_DIMS) throw BackendError(BackendError::kernelFailed, "more than 8 axes");
    hc_strides s;
    std::memset(&s, 0, sizeof(s));
    s.ndim = (uint32_t)shape.size();
    for (size_t i = 0; i < shape.size(); i++) {
      s.shape[i] = shape[i];
      s.strides[i] = strides[i];
    }
    return s;
  }
};

struct ReduceDims {
  int64_t outerCount, reduceCount, innerCount;
  int64_t inCount() const { return outerCount * reduceCount * innerCount; }
  int64_t outCount() const { return outerCount * innerCount; }
};

class HIPBackend;

// Device buffer; freed (stream-ordered) when the last reference goes away.
class Buffer {
 public:
  Buffer(hc_ctx* ctx, void* ptr, size_t bytes) : ctx_(ctx), ptr_(ptr), bytes_(bytes) {}
  // A buffer whose contents are produced on first use of its pointer (`fill` allocates and writes)
  Buffer(hc_ctx* ctx, size_t bytes, std::function<void*()> fill) : ctx_(ctx), ptr_(nullptr), bytes_(bytes), fill_(std::move(fill)) {}
  ~Buffer() { hc_free(ctx_, ptr_); }
  Buffer(const Buffer&) = delete;
  Buffer& operator=(const Buffer&) = delete;
  void* ptr() {
    if (!ptr_ && fill_) {
      ptr_ = fill_();
      fill_ = nullptr;
    }
    return ptr_;
  }
  size_t byteCount() const { return bytes_; }
  // set by axisPermutation: what this index vector permutes (lets gather copy directly)
  std::vector<int64_t> permutation, permutedShape;

 private:
  hc_ctx* ctx_;
  void* ptr_;
  size_t bytes_;
  std::function<void*()> fill_;
};
typedef std::shared_ptr<Buffer> Data;

struct BroadcastData {
  BroadcastStrides strides;
  Data data;
};

// ScatterGatherIndices (ScatterGather.swift:4-46).
struct ScatterGatherIndices {
  std::vector<int64_t> valueShape;
  int axis;
  BroadcastData indices;
  bool indicesAreUnique = false;
  int64_t outer() const { return prod(0, axis); }
  int64_t middle() const { return valueShape[axis]; }
  int64_t inner() const { return prod(axis + 1, (int)valueShape.size()); }
  int64_t outCount() const { return indices.strides.shape[axis]; }
  int64_t prod(int a, int b) const {
    int64_t n = 1;
    for (int i = a; i < b; i++) n *= valueShape[i];
    return n;
  }
};

class HIPBackend {
 public:
  explicit HIPBackend(int device = 0) { check(hc_init(device, &ctx_)); }
  ~HIPBackend() { hc_shutdown(ctx_); }
  HIPBackend(const HIPBackend&) = delete;
  HIPBackend& operator=(const HIPBackend&) = delete;
  hc_ctx* context() const { return ctx_; }

  // ---- storage
  Data allocate(size_t byteCount) {
    void* p = nullptr;
    check(hc_malloc(ctx_, byteCount, &p));
    return std::make_shared<Buffer>(ctx_, p, byteCount);
  }
  Data upload(const void* host, size_t bytes) {
    Data d = allocate(bytes);
    check(hc_memcpy_h2d(ctx_, d->ptr(), host, bytes));
    return d;
  }
  void download(const Data& d, void* host, size_t bytes) { check(hc_memcpy_d2h(ctx_, host, d->ptr(), bytes)); }
  void wait() { check(hc_sync(ctx_)); }

  // ---- recording and replay (no counterpart in the reference: one call replays every op
  // issued between beginCapture and endCapture; buffers allocated in between stay reserved
  // for the graph until it is destroyed)
  void beginCapture() { check(hc_capture_begin(ctx_)); }
  hc_graph* endCapture() {
    hc_graph* g = nullptr;
    check(hc_capture_end(ctx_, &g));
    return g;
  }
  void launch(hc_graph* g) { check(hc_graph_launch(ctx_, g)); }
  // launches and copies one replay issues (after the library's rewrite of the recording)
  size_t nodeCount(hc_graph* g) {
    size_t n = 0;
    check(hc_graph_node_count(g, &n));
    return n;
  }
  void destroy(hc_graph* g) { check(hc_graph_destroy(ctx_, g)); }

  // ---- batching (no counterpart in the reference either): the calls of ordinary code are listed
  // and enqueued batch by batch, each batch rewritten like a recording; 0 = one launch per call
  // (idleAfter > 0: a list of at least that many launches is also enqueued once the device has run dry)
  void setBatching(size_t maxLaunches, size_t idleAfter = 0) { check(hc_set_batching(ctx_, maxLaunches, idleAfter)); }
  void flush() { check(hc_flush(ctx_)); }
  std::pair<uint64_t, uint64_t> batchingStats() {   // launches listed, launches enqueued in their place
    uint64_t listed = 0, enqueued = 0;
    check(hc_batching_stats(ctx_, &listed, &enqueued));
    return {listed, enqueued};
  }

  // ---- ops (Backend.swift line of each declaration in the comment)
  Data broadcast(const BroadcastData& a, DType dtype) {  // :170
    Data out = allocate(a.strides.count() * byteSize(dtype));
    hc_strides s = a.strides.c();
    check(hc_broadcast(ctx_, (int)dtype, a.data->ptr(), &s, out->ptr()));
    return out;
  }
  Data binaryOp(const BroadcastData& a, const BroadcastData& b, hc_binary op, DType dtype) {  // :178
    Data out = allocate(a.strides.count() * byteSize(dtype));
    hc_strides sa = a.strides.c(), sb = b.strides.c();
    check(hc_binary_op(ctx_, op, (int)dtype, a.data->ptr(), &sa, b.data->ptr(), &sb, out->ptr()));
    return out;
  }
  template <typename T> Data binaryOp(const Data& a, T b, hc_binary op, size_t count, DType dtype) {  // :190
    Data out = allocate(count * byteSize(dtype));
    check(hc_binary_op_scalar(ctx_, op, (int)dtype, a->ptr(), (float)b, (int64_t)b, 0, out->ptr(), count));
    return out;
  }
  template <typename T> Data binaryOp(T a, const Data& b, hc_binary op, size_t count, DType dtype) {  // :202
    Data out = allocate(count * byteSize(dtype));
    check(hc_binary_op_scalar(ctx_, op, (int)dtype, b->ptr(), (float)a, (int64_t)a, 1, out->ptr(), count));
    return out;
  }
  Data mulAdd(const BroadcastData& input, const BroadcastData& coeff, const BroadcastData& bias, DType dtype) {  // :240
    Data out = allocate(input.strides.count() * byteSize(dtype));
    hc_strides si = input.strides.c(), sc = coeff.strides.c(), sb = bias.strides.c();
    check(hc_mul_add(ctx_, (int)dtype, input.data->ptr(), &si, coeff.data->ptr(), &sc, bias.data->ptr(), &sb, out->ptr()));
    return out;
  }
  Data addMul(const BroadcastData& input, const BroadcastData& bias, const BroadcastData& coeff, DType dtype) {  // :250
    Data out = allocate(input.strides.count() * byteSize(dtype));
    hc_strides si = input.strides.c(), sc = coeff.strides.c(), sb = bias.strides.c();
    check(hc_add_mul(ctx_, (int)dtype, input.data->ptr(), &si, bias.data->ptr(), &sb, coeff.data->ptr(), &sc, out->ptr()));
    return out;
  }
  Data normalize(const Data& input, ReduceDims dims, float eps, DType dtype) {  // :265
    Data out = allocate(dims.inCount() * byteSize(dtype));
    check(hc_normalize(ctx_, (int)dtype, input->ptr(), out->ptr(), dims.outerCount, dims.reduceCount, dims.innerCount, eps));
    return out;
  }
  Data compare(const BroadcastData& a, const BroadcastData& b, hc_compare_op op, DType dtype) {  // :457
    Data out = allocate(a.strides.count());
    hc_strides sa = a.strides.c(), sb = b.strides.c();
    check(hc_compare(ctx_, op, (int)dtype, a.data->ptr(), &sa, b.data->ptr(), &sb, out->ptr()));
    return out;
  }
  Data cast(const Data& a, size_t count, DType inType, DType outType) {  // :489
    Data out = allocate(count * byteSize(outType));
    check(hc_cast(ctx_, a->ptr(), (int)inType, out->ptr(), (int)outType, count));
    return out;
  }
  template <typename T> Data pow(const Data& a, T b, T scale, const Data& scales, size_t count, DType dtype) {  // :500
    Data out = allocate(count * byteSize(dtype));
    check(hc_pow(ctx_, (int)dtype, a->ptr(), (float)b, (float)scale, (int64_t)b, (int64_t)scale,
                 scales ? scales->ptr() : nullptr, out->ptr(), count));
    return out;
  }
  Data reduce(const Data& a, hc_reduce_op op, ReduceDims dims, DType dtype) {  // :524
    const DType outType = (op == HC_ARGMAX || op == HC_ARGMIN) ? DType::int64 : dtype;
    Data out = allocate(dims.outCount() * byteSize(outType));
    check(hc_reduce(ctx_, op, (int)dtype, a->ptr(), out->ptr(), dims.outerCount, dims.reduceCount, dims.innerCount));
    return out;
  }
  Data logSoftmax(const Data& a, ReduceDims dims, DType dtype) {  // :571
    Data out = allocate(dims.inCount() * byteSize(dtype));
    check(hc_log_softmax(ctx_, (int)dtype, a->ptr(), out->ptr(), dims.outerCount, dims.reduceCount, dims.innerCount));
    return out;
  }
  Data gather(const Data& a, const ScatterGatherIndices& s, DType dtype) {  // :609
    Data out = allocate(s.indices.strides.count() * byteSize(dtype));
    // The gather of t / swap / move: indices from axisPermutation that run along the gathered axis
    // only. hc_permute moves the same bytes without reading 8 bytes of index per element.
    Buffer& idx = *s.indices.data;
    if (!idx.permutedShape.empty() || idx.byteCount() == 8) {
      int64_t n = 1;
      for (int64_t d : idx.permutedShape) n *= d;
      bool direct = !idx.permutation.empty() && s.indices.strides.shape[s.axis] == n && s.middle() == n;
      for (size_t ax = 0; direct && ax < s.indices.strides.shape.size(); ax++)
        direct = s.indices.strides.shape[ax] == 1 || s.indices.strides.strides[ax] == ((int)ax == s.axis ? 1 : 0);
      if (direct) {
        std::vector<int64_t> perm = idx.permutation, shape = idx.permutedShape;
        if (s.outer() > 1) {
          for (int64_t& p : perm) p += 1;
          perm.insert(perm.begin(), 0);
          shape.insert(shape.begin(), s.outer());
        }
        if (shape.size() <= HC_MAX_DIMS) {  // (more axes fall through to the index gather)
          check(hc_permute(ctx_, (int)dtype, a->ptr(), perm.data(), shape.data(), (int)shape.size(), s.inner(), out->ptr()));
          return out;
        }
      }
    }
    hc_strides st = s.indices.strides.c();
    check(hc_gather(ctx_, (int)dtype, a->ptr(), s.indices.data->ptr(), &st, out->ptr(), s.outer(), s.middle(),
                    s.outCount(), s.inner()));
    return out;
  }
  Data bitwiseOp(const BroadcastData& a, const BroadcastData& b, hc_bitwise_op_kind op, DType dtype) {  // :215
    Data out = allocate(a.strides.count() * byteSize(dtype));
    hc_strides sa = a.strides.c(), sb = b.strides.c();
    check(hc_bitwise_op(ctx_, op, (int)dtype, a.data->ptr(), &sa, b.data->ptr(), &sb, out->ptr()));
    return out;
  }
  Data scatter(const Data& a, const ScatterGatherIndices& s, DType dtype) {  // :621
    Data out = allocate((size_t)(s.outer() * s.middle() * s.inner()) * byteSize(dtype));
    hc_strides st = s.indices.strides.c();
    check(hc_scatter(ctx_, (int)dtype, a->ptr(), s.indices.data->ptr(), &st, out->ptr(), s.outer(), s.middle(),
                     s.outCount(), s.inner(), s.indicesAreUnique));
    return out;
  }
  Data logSoftmaxGrad(const Data& a, const Data& outGrad, ReduceDims dims, DType dtype) {  // :578
    Data out = allocate(dims.inCount() * byteSize(dtype));
    check(hc_log_softmax_grad(ctx_, (int)dtype, a->ptr(), outGrad->ptr(), out->ptr(), dims.outerCount,
                              dims.reduceCount, dims.innerCount));
    return out;
  }
  Data cumulativeSum(const Data& a, ReduceDims dims, bool exclusive, bool reverse, DType dtype) {  // :548
    return cumulative(0, a, dims, exclusive, reverse, dtype);
  }
  Data cumulativeProd(const Data& a, ReduceDims dims, bool exclusive, bool reverse, DType dtype) {  // :561
    return cumulative(1, a, dims, exclusive, reverse, dtype);
  }
  // Always stable, which `stable == false` allows (:535)
  Data argsort(const Data& a, ReduceDims dims, bool descending, bool /*stable*/, DType dtype) {
    Data out = allocate(dims.inCount() * 8);
    check(hc_argsort(ctx_, (int)dtype, a->ptr(), out->ptr(), dims.outerCount, dims.reduceCount, dims.innerCount,
                     descending));
    return out;
  }
  // min / max: a BroadcastData with a null `data` means "no bound" (Backend.swift:512-520)
  Data clamp(const BroadcastData& a, const BroadcastData& min, const BroadcastData& max, DType dtype) {
    Data out = allocate(a.strides.count() * byteSize(dtype));
    hc_strides sa = a.strides.c(), sl = min.strides.c(), sh = max.strides.c();
    check(hc_clamp(ctx_, (int)dtype, a.data->ptr(), &sa, min.data ? min.data->ptr() : nullptr,
                   min.data ? &sl : nullptr, max.data ? max.data->ptr() : nullptr, max.data ? &sh : nullptr,
                   out->ptr()));
    return out;
  }
  Data cumulative(int op, const Data& a, ReduceDims dims, bool exclusive, bool reverse, DType dtype) {
    Data out = allocate(dims.inCount() * byteSize(dtype));
    check(hc_cumulative(ctx_, op, (int)dtype, a->ptr(), out->ptr(), dims.outerCount, dims.reduceCount,
                        dims.innerCount, exclusive, reverse));
    return out;
  }
  struct AdamResult {
    Data param, moment1, moment2;
  };
  AdamResult adamW(const Data& param, const Data& grad, const Data& moment1, const Data& moment2, float beta1,
                   float beta2, float eps, float weightDecay, float lr, float step, size_t count,
                   DType dtype) {  // :818
    AdamResult r{allocate(count * byteSize(dtype)), allocate(count * byteSize(dtype)),
                 allocate(count * byteSize(dtype))};
    check(hc_adamw(ctx_, (int)dtype, param->ptr(), grad->ptr(), moment1->ptr(), moment2->ptr(), beta1, beta2, eps,
                   weightDecay, lr, step, count, r.param->ptr(), r.moment1->ptr(), r.moment2->ptr()));
    return r;
  }
  Data when(const BroadcastData& mask, const BroadcastData& a, const BroadcastData& b, DType dtype) {  // :633
    Data out = allocate(mask.strides.count() * byteSize(dtype));
    hc_strides sm = mask.strides.c(), sa = a.strides.c(), sb = b.strides.c();
    check(hc_when(ctx_, (int)dtype, mask.data->ptr(), &sm, a.data->ptr(), &sa, b.data->ptr(), &sb, out->ptr()));
    return out;
  }
  Data matmul(const Data& a, bool transA, const Data& b, bool transB, bool transOut, int64_t rows, int64_t inner,
              int64_t cols, DType dtype) {  // :650
    return batchedMatmul(1, a, transA, b, transB, transOut, rows, inner, cols, dtype);
  }
  Data batchedMatmul(int64_t matrixCount, const Data& a, bool transA, const Data& b, bool transB, bool transOut,
                     int64_t rows, int64_t inner, int64_t cols, DType dtype) {  // :661
    Data out = allocate((size_t)(matrixCount * rows * cols) * byteSize(dtype));
    check(hc_matmul(ctx_, (int)dtype, matrixCount, a->ptr(), transA, b->ptr(), transB, transOut, rows, inner, cols, out->ptr()));
    return out;
  }
  Data triangular(const Data& a, int64_t batch, int64_t rows, int64_t cols, bool upper, int64_t offset, DType dtype) {  // :674
    Data out = allocate((size_t)(batch * rows * cols) * byteSize(dtype));
    check(hc_triangular(ctx_, (int)dtype, a->ptr(), out->ptr(), batch, rows, cols, upper, offset));
    return out;
  }
  Data elemwise(const Data& a, hc_elemwise_op op, const Data& scales, size_t count, DType dtype) {  // :770
    Data out = allocate(count * byteSize(dtype));
    check(hc_elemwise(ctx_, op, (int)dtype, a->ptr(), scales ? scales->ptr() : nullptr, out->ptr(), count));
    return out;
  }
  template <typename T> Data constant(T value, size_t count, DType dtype) {  // :787
    Data out = allocate(count * byteSize(dtype));
    check(hc_fill(ctx_, (int)dtype, (float)value, (int64_t)value, out->ptr(), count));
    return out;
  }
  // The int64 index vector is written on first use of its pointer: the usual consumer is the gather
  // of t / swap / move, which runs as a direct copy from (permutation, shape) alone.
  Data axisPermutation(const std::vector<int64_t>& permutation, const std::vector<int64_t>& shape) {  // :803
    int64_t n = 1;
    for (int64_t d : shape) n *= d;
    hc_ctx* ctx = ctx_;
    Data out = std::make_shared<Buffer>(ctx_, (size_t)n * 8, [=]() -> void* {
      void* p = nullptr;
      if (hc_malloc(ctx, (size_t)n * 8, &p) != HC_OK) throw BackendError(BackendError::allocationFailed, hc_last_error_string());
      if (hc_axis_permutation(ctx, permutation.data(), shape.data(), (int)shape.size(), p) != HC_OK)
        throw BackendError(BackendError::kernelFailed, hc_last_error_string());
      return p;
    });
    out->permutation = permutation;
    out->permutedShape = shape;
    return out;
  }

  void check(int status) {
    if (status == HC_OK) return;
    const std::string msg = hc_last_error_string();
    switch (status) {
      case HC_ERR_ALLOC: throw BackendError(BackendError::allocationFailed, msg);
      case HC_ERR_LOAD:
      case HC_ERR_NO_DEVICE: throw BackendError(BackendError::failedToLoadKernels, msg);
      case HC_ERR_UNSUPPORTED: throw BackendError(BackendError::notImplemented, msg);
      default: throw BackendError(BackendError::kernelFailed, msg);
    }
  }

 private:
  hc_ctx* ctx_ = nullptr;
};

}  // namespace hc
