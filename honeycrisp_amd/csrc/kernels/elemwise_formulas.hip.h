// Pieces of the element-wise formulas that more than one code object needs: kernels that take over
// the work of an element-wise kernel when a recording merges it into its producer (GELU in a GEMM
// epilogue, exp after a log-softmax) must produce the bits of the separate kernel. Every file
// that includes this is built with -ffp-contract=off (the reference never fuses a * b + c).
#pragma once

// Formulas of ElemwiseOp.apply (Elemwise.swift:44-183), same expression trees.
__device__ __forceinline__ float safe_sigmoid(float x) {
  if (x < -20.0f) return 0.0f;
  if (x > 20.0f) return 1.0f;
  return 1.0f / (1.0f + expf(-x));
}
__device__ __forceinline__ float safe_tanh(float x) { return 2.0f * safe_sigmoid(2.0f * x) - 1.0f; }

// The same for results that are rounded to fp16 (11 significant bits): the hardware's exp2 and
// reciprocal (about 1 ulp of fp32 each) instead of the library's expf and an IEEE division.
// With the library routines an fp16 GELU is bound by the vector ALU (8 elements per 16-byte
// load), not by memory.
__device__ __forceinline__ float exp_hw(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ __forceinline__ float sigmoid_hw(float x) {
  // (computed first, then selected: no branch per element, so the elements of a vector overlap)
  const float inside = __builtin_amdgcn_rcpf(1.0f + exp_hw(-x));
  return x < -20.0f ? 0.0f : (x > 20.0f ? 1.0f : inside);
}
__device__ __forceinline__ float tanh_hw(float x) { return 2.0f * sigmoid_hw(2.0f * x) - 1.0f; }

// powf(f, 3.0f) of the reference formula: the cube formed in double and rounded once is the
// correctly rounded result, which is what a libm powf returns for this exponent, at a
// fraction of the cost of a general powf.
__device__ __forceinline__ float cube(float f) {
  const double d = (double)f;
  return (float)(d * d * d);
}


// ElemwiseOp.geluApprox (Elemwise.swift:109-111) on a value of tensor type T held as float; the
// caller multiplies by the scale (1 without scales) and rounds to T, as the element-wise kernel does.
template <bool HALF> __device__ __forceinline__ float gelu_approx(float f) {
  if (HALF) return 0.5f * f * (1.0f + tanh_hw(0.797884561f * (f + 0.044715f * (f * f * f))));
  return 0.5f * f * (1.0f + safe_tanh(0.797884561f * (f + 0.044715f * cube(f))));
}
