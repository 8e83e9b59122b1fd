// Pieces of the row kernels (reduce.hip) that other kernels reproduce bit for bit: how a team of
// lanes holds a row in registers, how it reduces a value across its lanes, and which exponential a
// kernel uses for a given element type. The fused attention kernel (attention.hip) runs the softmax
// of a row with exactly these, so that its probabilities are those of the separate row kernel.
#pragma once

#include "common.hip.h"
#include <type_traits>

// v of lane (l ^ O), O a power of two below 64. Inside a row of 16 lanes the exchange is a DPP move (vector ALU,
// no trip through the LDS crossbar as a ds_bpermute makes): quad permutations for 1 and 2, a rotation of the
// row for 8, and for 4 a shift of the row to either side, each written into the quads it is right for
// (bank mask 0b1010: quads 1 and 3). Across rows the general shuffle stays.
template <int CTRL, int BANKS> __device__ __forceinline__ uint32_t dpp_move(uint32_t old, uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)v, CTRL, 0xF, BANKS, false);
}
template <int O> __device__ __forceinline__ uint32_t lane_xor_bits(uint32_t v) {
  static_assert(O > 0 && O < 64 && (O & (O - 1)) == 0, "a power of two inside the wave");
  if constexpr (O == 1) return dpp_move<0xB1, 0xF>(v, v);         // quad_perm [1, 0, 3, 2]
  else if constexpr (O == 2) return dpp_move<0x4E, 0xF>(v, v);    // quad_perm [2, 3, 0, 1]
  else if constexpr (O == 4) return dpp_move<0x114, 0xA>(dpp_move<0x104, 0xF>(v, v), v);   // row_shl:4, then row_shr:4 into quads 1, 3
  else if constexpr (O == 8) return dpp_move<0x128, 0xF>(v, v);   // row_ror:8
  else return (uint32_t)__shfl_xor((int)v, O, 64);
}
template <int O, typename V> __device__ __forceinline__ V lane_xor(V v) {
  if constexpr (sizeof(V) == 4 && std::is_trivially_copyable<V>::value)
    return __builtin_bit_cast(V, lane_xor_bits<O>(__builtin_bit_cast(uint32_t, v)));
  else
    return __shfl_xor(v, O, 64);
}

// every lane of an aligned group of LANES lanes (a power of two, at most a wave) gets the result:
// v = op(v, v of lane ^ o) for o = LANES / 2, ..., 2, 1
template <int LANES, typename V, typename Op> __device__ __forceinline__ V team_reduce(V v, Op op) {
  if constexpr (LANES >= 2) {
    v = op(v, lane_xor<LANES / 2>(v));
    return team_reduce<LANES / 2>(v, op);
  } else {
    return v;
  }
}

// The same for R independent values at once (R rows a team works on side by side), step by step: the R exchanges
// of a step are issued together and their latencies overlap, where R calls of team_reduce would run one
// chain of dependent exchanges after the other. Per value the operations and their order are team_reduce's.
template <int LANES, int R, typename V, typename Op> __device__ __forceinline__ void team_reduce_each(V (&v)[R], Op op) {
  if constexpr (LANES >= 2) {
    V t[R];
#pragma unroll
    for (int j = 0; j < R; j++) t[j] = lane_xor<LANES / 2>(v[j]);
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = op(v[j], t[j]);
    team_reduce_each<LANES / 2, R>(v, op);
  }
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

