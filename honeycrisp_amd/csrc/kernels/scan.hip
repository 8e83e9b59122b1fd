// Running sums / products and argsort along the middle axis of an [outer, reduce, inner] view.
//
// cumulativeSum / cumulativeProd (BackendCPU.swift:922-998): out[k] = x[0] (op) ... (op) x[k]
// (or up to x[k-1] when exclusive), optionally from the far end. Rows (inner == 1): one wave
// per row walks it in tiles of 64 x 4 elements (in-lane scan, wave scan of the lane totals
// with shuffles, running carry); floats are combined in tree order, so they differ from the
// sequential CPU loop by rounding only; int64 is exact. Columns (inner > 1): one lane per
// column, sequential along the axis, lanes coalesced along inner. When there are too few lines
// to fill the chip, the axis is cut into segments: totals per segment, a small scan of the
// totals, then the segments are scanned starting from what precedes them.
//
// argsort (BackendCPU.swift:888-920): one block per (outer, inner) pair sorts (key, index)
// pairs with a bitonic network in LDS, up to 4096 elements; longer axes are sorted in runs of
// 4096 that are then merged pairwise (merge path through LDS, 2048 outputs per workgroup). Keys are mapped to unsigned
// integers that order like the values (-0 counts as +0), inverted for descending order; the
// source index breaks ties, so the sort is stable, which the reference's `stable` flag
// asks for and its unstable variant permits.
#include "common.hip.h"

enum { SCAN_SUM = 0, SCAN_PROD = 1 };

template <int OP, typename C> __device__ __forceinline__ C scan_identity() { return OP == SCAN_SUM ? (C)0 : (C)1; }
template <int OP, typename C> __device__ __forceinline__ C scan_combine(C a, C b) {
  return OP == SCAN_SUM ? a + b : a * b;
}

// PHASE 0: the scan itself (of whole lines, or of segments that start from their carry);
// PHASE 1: only the segments' totals, into p.carry.
template <typename T, int OP, int PHASE> __device__ __forceinline__ void cumulative_rows_impl(const hck_scan_args& p) {
  typedef typename Arith<T>::type C;
  constexpr int E = 4;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t segs = p.segs > 1 ? p.segs : 1;
  const uint32_t unit = blockIdx.x * (HCK_BLOCK / 64) + (threadIdx.x >> 6);  // (row, segment)
  if (unit >= p.outer * segs) return;
  const uint32_t row = unit / segs, seg = unit - row * segs;
  const uint32_t n = p.reduce;
  const uint32_t lo = segs > 1 ? seg * p.seg_len : 0;
  const uint32_t hi = segs > 1 ? (lo + p.seg_len < n ? lo + p.seg_len : n) : n;
  const T* in = (const T*)p.in + (size_t)row * n;
  T* out = (T*)p.out + (size_t)row * n;
  C carry = (PHASE == 0 && segs > 1) ? ((const C*)p.carry)[unit] : scan_identity<OP, C>();
  for (uint32_t base = lo; base < hi; base += 64 * E) {
    // logical positions t (in scan order) of this lane; the element sits at n-1-t when reversed
    C x[E], run = scan_identity<OP, C>();
#pragma unroll
    for (int e = 0; e < E; e++) {
      const uint32_t t = base + lane * E + e;
      x[e] = t < hi ? to_arith(in[p.reverse ? n - 1 - t : t]) : scan_identity<OP, C>();
      run = scan_combine<OP, C>(run, x[e]);
    }
    if (PHASE == 1) {
      carry = scan_combine<OP, C>(carry, run);  // per lane; combined across the wave at the end
      continue;
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
      if (t < hi) out[p.reverse ? n - 1 - t : t] = from_arith<T>(p.exclusive ? acc : next);
      acc = next;
    }
    carry = scan_combine<OP, C>(carry, __shfl(incl, 63, 64));
  }
  if (PHASE == 1) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) carry = scan_combine<OP, C>(carry, __shfl_down(carry, d, 64));
    if (lane == 0) ((C*)p.carry)[unit] = carry;
  }
}

// VEC adjacent columns per lane (VEC > 1: inner is a multiple of VEC and the buffers are
// 16-byte aligned, so every access is one 16-byte piece).
template <typename T, int OP, int PHASE, int VEC>
__device__ __forceinline__ void cumulative_cols_impl(const hck_scan_args& p) {
  typedef typename Arith<T>::type C;
  const uint32_t segs = p.segs > 1 ? p.segs : 1;
  const uint32_t innerv = p.inner / VEC;
  const uint64_t t = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;  // (i, segment, vector column)
  if (t >= (uint64_t)p.outer * segs * innerv) return;
  const uint32_t j = (uint32_t)(t % innerv) * VEC;
  const uint32_t is = (uint32_t)(t / innerv), i = is / segs, seg = is - i * segs;
  const uint32_t lo = segs > 1 ? seg * p.seg_len : 0;
  const uint32_t hi = segs > 1 ? (lo + p.seg_len < p.reduce ? lo + p.seg_len : p.reduce) : p.reduce;
  const size_t base = (size_t)i * p.reduce * p.inner + j;
  const T* in = (const T*)p.in + base;
  T* out = (T*)p.out + base;
  C* carry = (C*)p.carry + (size_t)is * p.inner + j;
  C run[VEC];
#pragma unroll
  for (int v = 0; v < VEC; v++) run[v] = (PHASE == 0 && segs > 1) ? carry[v] : scan_identity<OP, C>();
#pragma unroll 4
  for (uint32_t s = lo; s < hi; s++) {
    const size_t k = (size_t)(p.reverse ? p.reduce - 1 - s : s) * p.inner;
    T x[VEC], o[VEC];
    load_vec<T, VEC>(in + k, 0, 1, x);
#pragma unroll
    for (int v = 0; v < VEC; v++) {
      const C next = scan_combine<OP, C>(run[v], to_arith(x[v]));
      o[v] = from_arith<T>(p.exclusive ? run[v] : next);
      run[v] = next;
    }
    if (PHASE == 0) store_vec<T, VEC>(out, k, o);
  }
  if (PHASE == 1) {
#pragma unroll
    for (int v = 0; v < VEC; v++) carry[v] = run[v];
  }
}

// Segment totals -> what precedes each segment: one wave per line (i, j) scans its `segs` totals
// 64 at a time with shuffles (a lane walking them one by one would take longer than the scan
// of the data itself once a line has thousands of segments).
template <typename C, int OP> __device__ __forceinline__ void cumulative_carry_impl(const hck_scan_args& p) {
  const uint64_t line = (uint64_t)blockIdx.x * (HCK_BLOCK / 64) + (threadIdx.x >> 6);
  if (line >= (uint64_t)p.outer * p.inner) return;  // (whole waves)
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t i = (uint32_t)(line / p.inner), j = (uint32_t)(line - (uint64_t)i * p.inner);
  C* c = (C*)p.carry + (size_t)i * p.segs * p.inner + j;
  C run = scan_identity<OP, C>();
  for (uint32_t s0 = 0; s0 < p.segs; s0 += 64) {
    const uint32_t s = s0 + lane;
    const bool ok = s < p.segs;
    C incl = ok ? c[(size_t)s * p.inner] : scan_identity<OP, C>();
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const C up = __shfl_up(incl, d, 64);
      if ((int)lane >= d) incl = scan_combine<OP, C>(up, incl);
    }
    C before = __shfl_up(incl, 1, 64);
    if (lane == 0) before = scan_identity<OP, C>();
    if (ok) c[(size_t)s * p.inner] = scan_combine<OP, C>(run, before);
    run = scan_combine<OP, C>(run, __shfl(incl, 63, 64));
  }
}

#define DEF_CUMULATIVE(TN, T)                                                                                   \
  HC_KERNEL void hc_cumulative_sum_rows_##TN(hck_scan_args p) { cumulative_rows_impl<T, SCAN_SUM, 0>(p); }      \
  HC_KERNEL void hc_cumulative_prod_rows_##TN(hck_scan_args p) { cumulative_rows_impl<T, SCAN_PROD, 0>(p); }    \
  HC_KERNEL void hc_cumulative_sum_cols_##TN(hck_scan_args p) { cumulative_cols_impl<T, SCAN_SUM, 0, 1>(p); }   \
  HC_KERNEL void hc_cumulative_prod_cols_##TN(hck_scan_args p) { cumulative_cols_impl<T, SCAN_PROD, 0, 1>(p); } \
  HC_KERNEL void hc_cumulative_sum_colsv_##TN(hck_scan_args p) {                                                \
    cumulative_cols_impl<T, SCAN_SUM, 0, VecWidth<T>::value>(p);                                                \
  }                                                                                                             \
  HC_KERNEL void hc_cumulative_prod_colsv_##TN(hck_scan_args p) {                                               \
    cumulative_cols_impl<T, SCAN_PROD, 0, VecWidth<T>::value>(p);                                               \
  }                                                                                                             \
  HC_KERNEL void hc_cumulative_sum_colsv_totals_##TN(hck_scan_args p) {                                         \
    cumulative_cols_impl<T, SCAN_SUM, 1, VecWidth<T>::value>(p);                                                \
  }                                                                                                             \
  HC_KERNEL void hc_cumulative_prod_colsv_totals_##TN(hck_scan_args p) {                                        \
    cumulative_cols_impl<T, SCAN_PROD, 1, VecWidth<T>::value>(p);                                               \
  }                                                                                                             \
  HC_KERNEL void hc_cumulative_sum_rows_totals_##TN(hck_scan_args p) { cumulative_rows_impl<T, SCAN_SUM, 1>(p); }   \
  HC_KERNEL void hc_cumulative_prod_rows_totals_##TN(hck_scan_args p) { cumulative_rows_impl<T, SCAN_PROD, 1>(p); } \
  HC_KERNEL void hc_cumulative_sum_cols_totals_##TN(hck_scan_args p) { cumulative_cols_impl<T, SCAN_SUM, 1, 1>(p); }   \
  HC_KERNEL void hc_cumulative_prod_cols_totals_##TN(hck_scan_args p) { cumulative_cols_impl<T, SCAN_PROD, 1, 1>(p); }
DEF_CUMULATIVE(f32, float)
DEF_CUMULATIVE(f16, half_t)
DEF_CUMULATIVE(i64, int64_t)
HC_KERNEL void hc_cumulative_sum_carry_f32(hck_scan_args p) { cumulative_carry_impl<float, SCAN_SUM>(p); }
HC_KERNEL void hc_cumulative_prod_carry_f32(hck_scan_args p) { cumulative_carry_impl<float, SCAN_PROD>(p); }
HC_KERNEL void hc_cumulative_sum_carry_i64(hck_scan_args p) { cumulative_carry_impl<int64_t, SCAN_SUM>(p); }
HC_KERNEL void hc_cumulative_prod_carry_i64(hck_scan_args p) { cumulative_carry_impl<int64_t, SCAN_PROD>(p); }

// ---------------------------------------------------------------- argsort

__device__ __forceinline__ uint64_t sort_key(float x) {
  x = x + 0.0f;  // -0 -> +0: the CPU's comparison treats them as equal
  uint32_t u = __float_as_uint(x);
  u ^= (u >> 31) ? 0xffffffffu : 0x80000000u;
  return (uint64_t)u;
}
__device__ __forceinline__ uint64_t sort_key(int64_t x) { return (uint64_t)x ^ 0x8000000000000000ull; }

constexpr int ARGSORT_MAX = 4096;

// What the block sort orders. Keys of 32 significant bits (floats, halfs) travel with their
// index in one 64-bit word (key in the high half), so one integer comparison orders by
// (key, index); 64-bit keys keep the index in a second array. Entry i lives at slot
// i + i / 16: a lane that walks entries 16, 32, ... apart then still spreads over the banks.
constexpr uint32_t SORT_SLOTS = ARGSORT_MAX + ARGSORT_MAX / 16;
__device__ __forceinline__ uint32_t sort_slot(uint32_t i) { return i + (i >> 4); }

template <bool WIDE> struct SortBuf {
  uint64_t* keys;
  uint32_t* idxs;
  __device__ __forceinline__ void put(uint32_t i, uint64_t key, uint32_t idx) const {
    if (WIDE) {
      keys[sort_slot(i)] = key;
      idxs[sort_slot(i)] = idx;
    } else {
      keys[sort_slot(i)] = (key << 32) | idx;
    }
  }
  __device__ __forceinline__ void pad(uint32_t i) const {  // sorts behind every real entry
    keys[sort_slot(i)] = ~0ull;
    if (WIDE) idxs[sort_slot(i)] = 0xffffffffu;
  }
  __device__ __forceinline__ uint64_t key(uint32_t i) const {
    return WIDE ? keys[sort_slot(i)] : keys[sort_slot(i)] >> 32;
  }
  __device__ __forceinline__ uint32_t idx(uint32_t i) const {
    return WIDE ? idxs[sort_slot(i)] : (uint32_t)keys[sort_slot(i)];
  }
};

// Bitonic sort of N = 2^G * (workgroup size) entries in LDS with 2^G entries per lane held in
// registers: a lane picks entries that differ only in G chosen index bits, so the G
// compare-exchange stages whose strides are those bits run without touching LDS. A merge of
// runs of length k/2 (log2 k stages) therefore costs ceil(log2 k / G) round trips, and all the
// merges up to k = 2^G together cost one: 21 round trips instead of 78 stages for 4096 entries.
template <bool WIDE, int G> __device__ __forceinline__ void bitonic_sort_regs(const SortBuf<WIDE>& buf, uint32_t N) {
  constexpr int E = 1 << G;
  uint64_t kx[E];
  uint32_t ix[E];
  const uint32_t t = threadIdx.x;
  // entries idx0 | (e << L), e = 0 .. E-1
  auto load = [&](uint32_t idx0, uint32_t L) {
#pragma unroll
    for (int e = 0; e < E; e++) {
      const uint32_t slot = sort_slot(idx0 | ((uint32_t)e << L));
      kx[e] = buf.keys[slot];
      if (WIDE) ix[e] = buf.idxs[slot];
    }
  };
  auto store = [&](uint32_t idx0, uint32_t L) {
#pragma unroll
    for (int e = 0; e < E; e++) {
      const uint32_t slot = sort_slot(idx0 | ((uint32_t)e << L));
      buf.keys[slot] = kx[e];
      if (WIDE) buf.idxs[slot] = ix[e];
    }
  };
  // the g stages with strides 2^(L+g-1) .. 2^L of the merge into runs of length k
  auto stages = [&](uint32_t idx0, uint32_t L, int g, uint32_t k) {
#pragma unroll
    for (int b = G - 1; b >= 0; b--) {
      if (b < g) {
#pragma unroll
        for (int e = 0; e < E; e++) {
          if (e & (1 << b)) continue;
          const int f = e | (1 << b);
          const bool ascending = ((idx0 | ((uint32_t)e << L)) & k) == 0;
          const bool e_after_f = kx[e] > kx[f] || (WIDE && kx[e] == kx[f] && ix[e] > ix[f]);
          const bool swap = e_after_f == ascending;
          const uint64_t klo = swap ? kx[f] : kx[e], khi = swap ? kx[e] : kx[f];
          kx[e] = klo;
          kx[f] = khi;
          if (WIDE) {
            const uint32_t ilo = swap ? ix[f] : ix[e], ihi = swap ? ix[e] : ix[f];
            ix[e] = ilo;
            ix[f] = ihi;
          }
        }
      }
    }
  };
  // runs up to length E: E consecutive entries per lane
  load(t << G, 0);
#pragma unroll
  for (int m = 1; m <= G; m++) stages(t << G, 0, m, 1u << m);
  store(t << G, 0);
  __syncthreads();
  for (uint32_t m = G + 1; (1u << m) <= N; m++) {
    uint32_t left = m;  // stages left in this merge: strides 2^(left-1) .. 1
    while (left > 0) {
      const int g = left < (uint32_t)G ? (int)left : G;
      const uint32_t L = left - g;
      const uint32_t idx0 = ((t >> L) << (L + G)) | (t & ((1u << L) - 1));
      load(idx0, L);
      stages(idx0, L, g, 1u << m);
      store(idx0, L);
      __syncthreads();
      left -= g;
    }
  }
}

// The same network one stage at a time, for fewer entries than two per lane.
template <bool WIDE> __device__ __forceinline__ void bitonic_sort_small(const SortBuf<WIDE>& buf, uint32_t N) {
  const uint32_t half = N >> 1, t = threadIdx.x;
  for (uint32_t k = 2; k <= N; k <<= 1) {
    for (uint32_t s = k >> 1; s > 0; s >>= 1) {
      if (t < half) {
        const uint32_t lo = ((t & ~(s - 1)) << 1) | (t & (s - 1));
        const uint32_t pa = sort_slot(lo), pb = sort_slot(lo + s);
        const uint64_t ka = buf.keys[pa], kb = buf.keys[pb];
        const uint32_t ia = WIDE ? buf.idxs[pa] : 0, ib = WIDE ? buf.idxs[pb] : 0;
        const bool a_after_b = ka > kb || (WIDE && ka == kb && ia > ib);
        if (a_after_b == ((lo & k) == 0)) {
          buf.keys[pa] = kb;
          buf.keys[pb] = ka;
          if (WIDE) {
            buf.idxs[pa] = ib;
            buf.idxs[pb] = ia;
          }
        }
      }
      __syncthreads();
    }
  }
}

// N: a power of two, 2 <= N <= ARGSORT_MAX
template <bool WIDE> __device__ __forceinline__ void bitonic_sort_lds(const SortBuf<WIDE>& buf, uint32_t N) {
  static_assert(ARGSORT_MAX == 16 * HCK_BLOCK, "entries per lane below assume 4096 entries and 256 lanes");
  if (N == 16 * HCK_BLOCK) bitonic_sort_regs<WIDE, 4>(buf, N);
  else if (N == 8 * HCK_BLOCK) bitonic_sort_regs<WIDE, 3>(buf, N);
  else if (N == 4 * HCK_BLOCK) bitonic_sort_regs<WIDE, 2>(buf, N);
  else if (N == 2 * HCK_BLOCK) bitonic_sort_regs<WIDE, 1>(buf, N);
  else bitonic_sort_small<WIDE>(buf, N);
}

// descending order = ascending order of the inverted key
template <typename C> __device__ __forceinline__ uint64_t key_flip(uint32_t descending) {
  return descending ? ((sizeof(C) == 8) ? ~0ull : 0xffffffffull) : 0ull;
}

template <typename T> __device__ __forceinline__ void argsort_impl(const hck_scan_args& p) {
  typedef typename Arith<T>::type C;
  constexpr bool WIDE = sizeof(C) == 8;
  __shared__ uint64_t keys[SORT_SLOTS];
  __shared__ uint32_t idxs[WIDE ? SORT_SLOTS : 1];
  const SortBuf<WIDE> buf{keys, idxs};
  const uint32_t i = blockIdx.x / p.inner, j = blockIdx.x - i * p.inner;
  const size_t base = (size_t)i * p.reduce * p.inner + j;
  const T* in = (const T*)p.in + base;
  int64_t* out = (int64_t*)p.out + base;
  uint32_t N = 2;
  while (N < p.reduce) N <<= 1;
  const uint64_t flip = key_flip<C>(p.reverse);
  for (uint32_t t = threadIdx.x; t < N; t += HCK_BLOCK) {
    if (t < p.reduce) buf.put(t, sort_key((C)to_arith(in[(size_t)t * p.inner])) ^ flip, t);
    else buf.pad(t);
  }
  __syncthreads();
  bitonic_sort_lds<WIDE>(buf, N);
  for (uint32_t t = threadIdx.x; t < p.reduce; t += HCK_BLOCK) out[(size_t)t * p.inner] = (int64_t)buf.idx(t);
}

// Long axes, pass 1: block (line, chunk) sorts elements [chunk * ARGSORT_MAX, ...) of its line
// and stores the sorted (key, index) run.
template <typename T> __device__ __forceinline__ void argsort_chunks_impl(const hck_sort_args& p) {
  typedef typename Arith<T>::type C;
  constexpr bool WIDE = sizeof(C) == 8;
  __shared__ uint64_t keys[SORT_SLOTS];
  __shared__ uint32_t idxs[WIDE ? SORT_SLOTS : 1];
  const SortBuf<WIDE> buf{keys, idxs};
  const uint32_t chunks = (p.reduce + ARGSORT_MAX - 1) / ARGSORT_MAX;
  const uint32_t line = blockIdx.x / chunks, chunk = blockIdx.x - line * chunks;
  const uint32_t i = line / p.inner, j = line - i * p.inner;
  const T* in = (const T*)p.in + (size_t)i * p.reduce * p.inner + j;
  const uint32_t first = chunk * ARGSORT_MAX;
  const uint32_t count = p.reduce - first < ARGSORT_MAX ? p.reduce - first : ARGSORT_MAX;
  const uint64_t flip = key_flip<C>(p.descending);
  for (uint32_t t = threadIdx.x; t < ARGSORT_MAX; t += HCK_BLOCK) {
    if (t < count) buf.put(t, sort_key((C)to_arith(in[(size_t)(first + t) * p.inner])) ^ flip, first + t);
    else buf.pad(t);
  }
  __syncthreads();
  bitonic_sort_lds<WIDE>(buf, ARGSORT_MAX);
  const size_t dst = (size_t)line * p.reduce + first;
  for (uint32_t t = threadIdx.x; t < count; t += HCK_BLOCK) {
    p.keys_out[dst + t] = buf.key(t);
    p.idx_out[dst + t] = buf.idx(t);
  }
}

// Long axes, pass 2..: runs of length `run` are merged pairwise. A workgroup produces
// MERGE_TILE consecutive outputs of one pair of runs: two of its waves find where the merge
// path crosses the tile's first and last output (a 64-way search: every lane probes one
// candidate per round, so a run of any length needs at most a few dependent loads), the
// workgroup copies the two input windows into LDS, and every lane bisects to its own first
// output there and merges MERGE_SEG entries. (key, index) pairs are all distinct, so the
// result does not depend on how ties would be broken.
constexpr uint32_t MERGE_SEG = 8;
constexpr uint32_t MERGE_TILE = MERGE_SEG * HCK_BLOCK;

__device__ __forceinline__ bool pair_before(uint64_t ka, uint32_t ia, uint64_t kb, uint32_t ib) {
  return ka < kb || (ka == kb && ia < ib);
}

HC_KERNEL void hc_argsort_merge(hck_sort_args p) {
  __shared__ uint64_t sk[MERGE_TILE];
  __shared__ uint32_t si[MERGE_TILE];
  __shared__ uint32_t split[2];
  const uint32_t tiles = (p.reduce + MERGE_TILE - 1) / MERGE_TILE;
  const uint32_t line = blockIdx.x / tiles, tile = blockIdx.x - line * tiles;
  const size_t base = (size_t)line * p.reduce;
  const uint32_t pos = tile * MERGE_TILE;                // first output position in the line
  const uint32_t pair = pos / (2 * p.run) * (2 * p.run); // start of this pair of runs
  const uint32_t a0 = pair, a1 = min(pair + p.run, p.reduce);
  const uint32_t b0 = a1, b1 = min(pair + 2 * p.run, p.reduce);
  const uint32_t na = a1 - a0, nb = b1 - b0;
  const uint32_t d0 = pos - pair, d1 = min(d0 + MERGE_TILE, na + nb);
  const uint64_t* ka = p.keys_in + base + a0;
  const uint64_t* kb = p.keys_in + base + b0;
  const uint32_t* ia = p.idx_in + base + a0;
  const uint32_t* ib = p.idx_in + base + b0;
  const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (wave < 2) {
    // smallest x (entries taken from run A before diagonal d) with A[x] not before B[d - x - 1]
    const uint32_t d = wave == 0 ? d0 : d1;
    uint32_t lo = d > nb ? d - nb : 0, hi = d < na ? d : na;
    while (lo < hi) {
      const uint32_t step = (hi - lo + 63) / 64;
      const uint32_t x = lo + lane * step;
      const bool before = x < hi && pair_before(ka[x], ia[x], kb[d - x - 1], ib[d - x - 1]);
      const uint32_t cnt = (uint32_t)__popcll(__ballot(before));  // the candidates that hold form a prefix
      if (cnt == 0) {
        hi = lo;
      } else {
        const uint32_t next = lo + cnt * step;
        lo = lo + (cnt - 1) * step + 1;
        hi = next < hi ? next : hi;
      }
    }
    if (lane == 0) split[wave] = lo;
  }
  __syncthreads();
  const uint32_t x0 = split[0], x1 = split[1], y0 = d0 - x0, y1 = d1 - x1;
  const uint32_t ca = x1 - x0, cb = y1 - y0;  // ca + cb = d1 - d0 <= MERGE_TILE
  for (uint32_t t = threadIdx.x; t < ca + cb; t += HCK_BLOCK) {
    sk[t] = t < ca ? ka[x0 + t] : kb[y0 + t - ca];
    si[t] = t < ca ? ia[x0 + t] : ib[y0 + t - ca];
  }
  __syncthreads();
  const uint32_t d = threadIdx.x * MERGE_SEG;  // diagonal inside the tile
  if (d >= ca + cb) return;
  const uint64_t* la = sk;
  const uint64_t* lb = sk + ca;
  const uint32_t* ja = si;
  const uint32_t* jb = si + ca;
  uint32_t lo = d > cb ? d - cb : 0, hi = d < ca ? d : ca;
  while (lo < hi) {
    const uint32_t x = (lo + hi) / 2, y = d - x - 1;
    if (pair_before(la[x], ja[x], lb[y], jb[y])) lo = x + 1;
    else hi = x;
  }
  uint32_t x = lo, y = d - lo;
  const uint32_t n = min(MERGE_SEG, ca + cb - d);
  const size_t o0 = base + pair + d0 + d;
  for (uint32_t o = 0; o < n; o++) {
    bool take_a;
    if (x >= ca) take_a = false;
    else if (y >= cb) take_a = true;
    else take_a = pair_before(la[x], ja[x], lb[y], jb[y]);
    p.keys_out[o0 + o] = take_a ? la[x] : lb[y];
    p.idx_out[o0 + o] = take_a ? ja[x] : jb[y];
    if (take_a) x++;
    else y++;
  }
}

// Long axes, last pass: sorted indices to the int64 result, back in the tensor's layout.
HC_KERNEL void hc_argsort_emit(hck_sort_args p) {
  const uint64_t gid = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;
  const uint64_t total = (uint64_t)p.outer * p.inner * p.reduce;
  if (gid >= total) return;
  // gid walks the result in memory order: (i, t, j)
  const uint32_t j = (uint32_t)(gid % p.inner);
  const uint64_t r = gid / p.inner;
  const uint32_t t = (uint32_t)(r % p.reduce), i = (uint32_t)(r / p.reduce);
  const size_t line = (size_t)i * p.inner + j;
  ((int64_t*)p.out)[gid] = (int64_t)p.idx_in[line * p.reduce + t];
}

HC_KERNEL void hc_argsort_chunks_f32(hck_sort_args p) { argsort_chunks_impl<float>(p); }
HC_KERNEL void hc_argsort_chunks_f16(hck_sort_args p) { argsort_chunks_impl<half_t>(p); }
HC_KERNEL void hc_argsort_chunks_i64(hck_sort_args p) { argsort_chunks_impl<int64_t>(p); }
HC_KERNEL void hc_argsort_f32(hck_scan_args p) { argsort_impl<float>(p); }
HC_KERNEL void hc_argsort_f16(hck_scan_args p) { argsort_impl<half_t>(p); }
HC_KERNEL void hc_argsort_i64(hck_scan_args p) { argsort_impl<int64_t>(p); }
