// The CPU leg of HCMatrixBench: the reference `CPUBackend` (Sources/Honeycrisp/BackendCPU.swift) as
// it would run on Linux, for the operations the benchmark times. One thread, like the reference,
// which funnels all CPU work through one worker (BackendCPU.swift:226,235-248); float data goes
// through whole-buffer conversions to Float and back (readBuffer / writeBuffer, :2018-2058), and the
// calls the reference makes into Accelerate go to the Linux stand-in of this package
// (swift/honeycrisp-linux/Sources/Accelerate): vDSP_mmul for the fp32 product without transposes
// (:1245-1261, forwarded to an OpenBLAS sgemm found at run time, whose thread count is reported),
// vDSP_sve for fp32 sums (:792-806), the vImage routines for half <-> float.
//
// This is the benchmark's baseline, nothing more: the HIP backend never calls it, and it is not the
// parity oracle of the test-suite (which lives elsewhere and is checked against the reference's own
// test vectors). Products can be restricted to a slab of output rows, because the literal loop takes
// minutes at 4096^3; the caller reports which rows ran.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include "../../swift/honeycrisp-linux/Sources/Accelerate/include/Accelerate.h"
#include "hip_backend.hpp"

namespace hc {

class CPUBackend {
 public:
  // readBuffer (BackendCPU.swift:2018-2043): the whole buffer as Float
  static std::vector<float> readFloats(const void* data, size_t count, DType dtype) {
    std::vector<float> out(count);
    if (dtype == DType::float32) {
      std::memcpy(out.data(), data, count * 4);
    } else {
      vImage_Buffer src{const_cast<void*>(data), 1, count, count * 2}, dst{out.data(), 1, count, count * 4};
      vImageConvert_Planar16FtoPlanarF(&src, &dst, 0);
    }
    return out;
  }
  // writeBuffer (:2045-2058)
  static void writeFloats(const float* in, size_t count, DType dtype, void* out) {
    if (dtype == DType::float32) {
      std::memcpy(out, in, count * 4);
    } else {
      vImage_Buffer src{const_cast<float*>(in), 1, count, count * 4}, dst{out, 1, count, count * 2};
      vImageConvert_PlanarFtoPlanar16F(&src, &dst, 0);
    }
  }

  // Backend.matmul on the CPU (BackendCPU.swift:1234-1313), rows [row0, row1) of the result as Float.
  // `a`, `b` are the operands already read as Float (the caller times that conversion separately).
  // fp32 without transposes and all rows: vDSP_mmul; everything else: the literal loop with a Float
  // accumulator, acc = acc + a * b in k order.
  static void matmulRows(const float* a, bool transA, const float* b, bool transB, int64_t rows, int64_t inner, int64_t cols,
                         int64_t row0, int64_t row1, bool use_vdsp, float* out) {
    if (use_vdsp && !transA && !transB) {
      vDSP_mmul(a + row0 * inner, 1, b, 1, out, 1, (vDSP_Length)(row1 - row0), (vDSP_Length)cols, (vDSP_Length)inner);
      return;
    }
    for (int64_t i = row0; i < row1; i++)
      for (int64_t j = 0; j < cols; j++) {
        float acc = 0.0f;
        for (int64_t k = 0; k < inner; k++) {
          const float x = transA ? a[k * rows + i] : a[i * inner + k];
          const float y = transB ? b[j * inner + k] : b[k * cols + j];
          acc = acc + x * y;
        }
        out[(i - row0) * cols + j] = acc;
      }
  }

  // BroadcastStrides.callAsFunction (Broadcast.swift:72-90): data index of element i of the virtual array
  static int64_t index(const BroadcastStrides& s, int64_t i) {
    int64_t result = 0;
    for (size_t d = s.shape.size(); d-- > 0;) {
      result += s.strides[d] * (i % s.shape[d]);
      i /= s.shape[d];
    }
    return result;
  }
  // binaryOp(.add) over two broadcast operands (BackendCPU.swift:267-314): vDSP only when neither side is
  // broadcast, else the element loop with one index map per operand and element
  static void add(const float* a, const BroadcastStrides& as, const float* b, const BroadcastStrides& bs, float* out) {
    const int64_t n = as.count();
    bool plain = true;
    int64_t acc = 1;
    for (size_t d = as.shape.size(); d-- > 0;) {
      plain = plain && as.strides[d] == acc && bs.strides[d] == acc;
      acc *= as.shape[d];
    }
    if (plain) {
      vDSP_vadd(a, 1, b, 1, out, 1, (vDSP_Length)n);
      return;
    }
    for (int64_t i = 0; i < n; i++) out[i] = a[index(as, i)] + b[index(bs, i)];
  }
  // ElemwiseOp.geluApprox (Elemwise.swift:109-111, 171-183)
  static float safeSigmoid(float v) { return v < -20.0f ? 0.0f : v > 20.0f ? 1.0f : 1.0f / (1.0f + expf(-v)); }
  static float safeTanh(float u) { return 2.0f * safeSigmoid(2.0f * u) - 1.0f; }
  static void geluApprox(const float* x, int64_t n, float* out) {
    for (int64_t i = 0; i < n; i++)
      out[i] = 0.5f * x[i] * (1.0f + safeTanh(0.797884561f * (x[i] + 0.044715f * powf(x[i], 3.0f))));
  }
  // reduce(.sum), fp32 (BackendCPU.swift:792-806): one vDSP_sve per output, stride innerCount
  static void sum(const float* x, ReduceDims d, float* out) {
    for (int64_t i = 0; i < d.outerCount; i++)
      for (int64_t j = 0; j < d.innerCount; j++)
        vDSP_sve(x + i * d.reduceCount * d.innerCount + j, (vDSP_Stride)d.innerCount, out + i * d.innerCount + j,
                 (vDSP_Length)d.reduceCount);
  }
  // reduce(.argmax) (BackendCPU.swift:848-877): strict compare from k = 0
  static void argmax(const float* x, ReduceDims d, int64_t* out) {
    for (int64_t i = 0; i < d.outerCount; i++)
      for (int64_t j = 0; j < d.innerCount; j++) {
        float extremum = x[j + i * d.reduceCount * d.innerCount];
        int64_t best = 0;
        for (int64_t k = 0; k < d.reduceCount; k++) {
          const float item = x[j + (k + i * d.reduceCount) * d.innerCount];
          if (item > extremum) {
            extremum = item;
            best = k;
          }
        }
        out[i * d.innerCount + j] = best;
      }
  }
  // gather (BackendCPU.swift:1108-1147), index strides by the broadcast map
  static void gather(const float* in, const int64_t* indices, const BroadcastStrides& is, int64_t outer, int64_t middle,
                     int64_t outCount, int64_t inner, float* out) {
    for (int64_t i = 0; i < outer; i++)
      for (int64_t j = 0; j < outCount; j++)
        for (int64_t k = 0; k < inner; k++) {
          const int64_t o = (i * outCount + j) * inner + k;
          out[o] = in[(i * middle + indices[index(is, o)]) * inner + k];
        }
  }
};

}  // namespace hc
