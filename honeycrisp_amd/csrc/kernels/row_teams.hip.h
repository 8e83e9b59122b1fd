// Pieces of the row kernels (reduce.hip) that other kernels reproduce bit for bit: how a team of
// lanes holds a row in registers, how it reduces a value across its lanes, and which exponential a
// kernel uses for a given element type. The fused attention kernel (attention.hip) runs the softmax
// of a row with exactly these, so that its probabilities are those of the separate row kernel.
#pragma once

#include "common.hip.h"

// every lane of an aligned group of LANES lanes (a power of two, at most a wave) gets the result
template <int LANES, typename V, typename Op> __device__ __forceinline__ V team_reduce(V v, Op op) {
#pragma unroll
  for (int o = LANES / 2; o > 0; o >>= 1) v = op(v, __shfl_xor(v, o, 64));
  return v;
}

// A row of up to LANES * VEC * CHUNKS elements held by its team in registers: lane l owns the
// 16-byte vectors l, l + LANES, ... of the row (n a multiple of VEC; rows then start 16-byte
// aligned because the buffer does). Longer rows, or ragged ones, are streamed instead.
// (NCHUNKS: vectors per lane; a kernel that knows its rows to be shorter than LANES * VEC * 4 may hold
// fewer: the order in which a lane visits its elements does not depend on it.)
template <typename T, int LANES, int NCHUNKS = 4> struct RowRegs {
  static constexpr int VEC = VecWidth<T>::value;
  static constexpr int CHUNKS = NCHUNKS;
  T v[CHUNKS][VEC];
  static __device__ __forceinline__ bool fits(uint32_t n) {
    return n % VEC == 0 && n <= (uint32_t)LANES * VEC * CHUNKS;
  }
  __device__ __forceinline__ void load(const T* row, uint32_t n, uint32_t lane) {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
      const uint32_t k = (lane + LANES * c) * VEC;
      if (k < n) load_vec<T, VEC>(row, k, 1, v[c]);
    }
  }
  template <typename F> __device__ __forceinline__ void each(uint32_t n, uint32_t lane, F f) const {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++)
      if ((lane + LANES * c) * VEC < n) {
#pragma unroll
        for (int i = 0; i < VEC; i++) f((float)v[c][i]);
      }
  }
  template <typename F> __device__ __forceinline__ void store(T* row, uint32_t n, uint32_t lane, F f) const {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
      const uint32_t k = (lane + LANES * c) * VEC;
      if (k < n) {
        T o[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) o[i] = narrow<T>(f((float)v[c][i]));
        store_vec<T, VEC>(row, k, o);
      }
    }
  }
  template <typename F>
  __device__ __forceinline__ void store2(T* row, uint32_t n, uint32_t lane, const RowRegs& other, F f) const {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
      const uint32_t k = (lane + LANES * c) * VEC;
      if (k < n) {
        T o[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) o[i] = narrow<T>(f((float)v[c][i], (float)other.v[c][i]));
        store_vec<T, VEC>(row, k, o);
      }
    }
  }
};

// exp of an fp32 value inside a kernel whose results are rounded to T: the library's expf for fp32
// tensors; for fp16 tensors (11 significant bits) the hardware's exp2, about 1 ulp of fp32, at a
// fifth of the instructions: an fp16 softmax row is bound by these, not by memory.
template <typename T> __device__ __forceinline__ float exp_in(float x) { return sizeof(T) == 2 ? exp_hw(x) : expf(x); }

