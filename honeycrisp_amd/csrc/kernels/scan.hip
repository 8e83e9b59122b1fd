// Running sums / products and argsort along the middle axis of an [outer, reduce, inner] view.
//
// cumulativeSum / cumulativeProd (BackendCPU.swift:922-998): out[k] = x[0] (op) ... (op) x[k]
// (or up to x[k-1] when exclusive), optionally from the far end. Rows (inner == 1): one wave
// per row walks it in tiles of 64 x 4 elements (in-lane scan, wave scan of the lane totals
// with shuffles, running carry); floats are combined in tree order, so they differ from the
// sequential CPU loop by rounding only; int64 is exact. Columns (inner > 1): one lane per
// column, sequential along the axis, lanes coalesced along inner.
//
// argsort (BackendCPU.swift:888-920): one block per (outer, inner) pair sorts (key, index)
// pairs with a bitonic network in LDS, up to 4096 elements. Keys are mapped to unsigned
// integers that order like the values (-0 counts as +0), inverted for descending order; the
// source index breaks ties, so the sort is stable, which the reference's `stable` flag
// asks for and its unstable variant permits.
#include "common.hip.h"

enum { SCAN_SUM = 0, SCAN_PROD = 1 };

template <int OP, typename C> __device__ __forceinline__ C scan_identity() { return OP == SCAN_SUM ? (C)0 : (C)1; }
template <int OP, typename C> __device__ __forceinline__ C scan_combine(C a, C b) {
  return OP == SCAN_SUM ? a + b : a * b;
}

template <typename T, int OP> __device__ __forceinline__ void cumulative_rows_impl(const hck_scan_args& p) {
  typedef typename Arith<T>::type C;
  constexpr int E = 4;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * (HCK_BLOCK / 64) + (threadIdx.x >> 6);
  if (row >= p.outer) return;
  const uint32_t n = p.reduce;
  const T* in = (const T*)p.in + (size_t)row * n;
  T* out = (T*)p.out + (size_t)row * n;
  C carry = scan_identity<OP, C>();
  for (uint32_t base = 0; base < n; base += 64 * E) {
    // logical positions t (in scan order) of this lane; the element sits at n-1-t when reversed
    C x[E], run = scan_identity<OP, C>();
#pragma unroll
    for (int e = 0; e < E; e++) {
      const uint32_t t = base + lane * E + e;
      x[e] = t < n ? to_arith(in[p.reverse ? n - 1 - t : t]) : scan_identity<OP, C>();
      run = scan_combine<OP, C>(run, x[e]);
    }
    // inclusive scan of the lane totals across the wave
    C incl = run;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const C up = __shfl_up(incl, d, 64);
      if (lane >= (uint32_t)d) incl = scan_combine<OP, C>(up, incl);
    }
    C before = __shfl_up(incl, 1, 64);  // everything in lanes below this one
    if (lane == 0) before = scan_identity<OP, C>();
    C acc = scan_combine<OP, C>(carry, before);
#pragma unroll
    for (int e = 0; e < E; e++) {
      const uint32_t t = base + lane * E + e;
      const C next = scan_combine<OP, C>(acc, x[e]);
      if (t < n) out[p.reverse ? n - 1 - t : t] = from_arith<T>(p.exclusive ? acc : next);
      acc = next;
    }
    carry = scan_combine<OP, C>(carry, __shfl(incl, 63, 64));
  }
}

template <typename T, int OP> __device__ __forceinline__ void cumulative_cols_impl(const hck_scan_args& p) {
  typedef typename Arith<T>::type C;
  const uint64_t t = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (t >= (uint64_t)p.outer * p.inner) return;
  const uint32_t i = (uint32_t)(t / p.inner), j = (uint32_t)(t - (uint64_t)i * p.inner);
  const size_t base = (size_t)i * p.reduce * p.inner + j;
  const T* in = (const T*)p.in + base;
  T* out = (T*)p.out + base;
  C run = scan_identity<OP, C>();
  for (uint32_t s = 0; s < p.reduce; s++) {
    const size_t k = (size_t)(p.reverse ? p.reduce - 1 - s : s) * p.inner;
    const C next = scan_combine<OP, C>(run, to_arith(in[k]));
    out[k] = from_arith<T>(p.exclusive ? run : next);
    run = next;
  }
}

#define DEF_CUMULATIVE(TN, T)                                                                                  \
  HC_KERNEL void hc_cumulative_sum_rows_##TN(hck_scan_args p) { cumulative_rows_impl<T, SCAN_SUM>(p); }        \
  HC_KERNEL void hc_cumulative_prod_rows_##TN(hck_scan_args p) { cumulative_rows_impl<T, SCAN_PROD>(p); }      \
  HC_KERNEL void hc_cumulative_sum_cols_##TN(hck_scan_args p) { cumulative_cols_impl<T, SCAN_SUM>(p); }        \
  HC_KERNEL void hc_cumulative_prod_cols_##TN(hck_scan_args p) { cumulative_cols_impl<T, SCAN_PROD>(p); }
DEF_CUMULATIVE(f32, float)
DEF_CUMULATIVE(f16, half_t)
DEF_CUMULATIVE(i64, int64_t)

// ---------------------------------------------------------------- argsort

__device__ __forceinline__ uint64_t sort_key(float x) {
  x = x + 0.0f;  // -0 -> +0: the CPU's comparison treats them as equal
  uint32_t u = __float_as_uint(x);
  u ^= (u >> 31) ? 0xffffffffu : 0x80000000u;
  return (uint64_t)u;
}
__device__ __forceinline__ uint64_t sort_key(int64_t x) { return (uint64_t)x ^ 0x8000000000000000ull; }

constexpr int ARGSORT_MAX = 4096;

template <typename T> __device__ __forceinline__ void argsort_impl(const hck_scan_args& p) {
  typedef typename Arith<T>::type C;
  __shared__ uint64_t keys[ARGSORT_MAX];
  __shared__ uint32_t idxs[ARGSORT_MAX];
  const uint32_t i = blockIdx.x / p.inner, j = blockIdx.x - i * p.inner;
  const size_t base = (size_t)i * p.reduce * p.inner + j;
  const T* in = (const T*)p.in + base;
  int64_t* out = (int64_t*)p.out + base;
  uint32_t N = 1;
  while (N < p.reduce) N <<= 1;
  // descending order = ascending order of the inverted key; padding sorts behind everything
  const uint64_t flip = p.reverse ? ((sizeof(C) == 8) ? ~0ull : 0xffffffffull) : 0ull;
  for (uint32_t t = threadIdx.x; t < N; t += HCK_BLOCK) {
    if (t < p.reduce) {
      keys[t] = sort_key((C)to_arith(in[(size_t)t * p.inner])) ^ flip;
      idxs[t] = t;
    } else {
      keys[t] = ~0ull;
      idxs[t] = 0xffffffffu;
    }
  }
  __syncthreads();
  for (uint32_t k = 2; k <= N; k <<= 1) {
    for (uint32_t s = k >> 1; s > 0; s >>= 1) {
      for (uint32_t t = threadIdx.x; t < N; t += HCK_BLOCK) {
        const uint32_t u = t ^ s;
        if (u > t) {
          const uint64_t ka = keys[t], kb = keys[u];
          const uint32_t ia = idxs[t], ib = idxs[u];
          const bool a_after_b = ka > kb || (ka == kb && ia > ib);
          const bool ascending = (t & k) == 0;
          if (a_after_b == ascending) {
            keys[t] = kb;
            keys[u] = ka;
            idxs[t] = ib;
            idxs[u] = ia;
          }
        }
      }
      __syncthreads();
    }
  }
  for (uint32_t t = threadIdx.x; t < p.reduce; t += HCK_BLOCK) out[(size_t)t * p.inner] = (int64_t)idxs[t];
}
HC_KERNEL void hc_argsort_f32(hck_scan_args p) { argsort_impl<float>(p); }
HC_KERNEL void hc_argsort_f16(hck_scan_args p) { argsort_impl<half_t>(p); }
HC_KERNEL void hc_argsort_i64(hck_scan_args p) { argsort_impl<int64_t>(p); }
