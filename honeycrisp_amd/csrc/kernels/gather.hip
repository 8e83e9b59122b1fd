// Data-movement kernels for gfx950: int64-indexed gather, axisPermutation, triangular,
// concat. All bit-exact copies keyed by element size, not dtype.
//
// gather (BackendCPU.swift:1108-1147):
//   out[(i*out_count + j)*inner + k] = in[(i*middle + idx)*inner + k],
//   idx = indices[index_strides(flat out index)]
// Row form: when the index does not depend on k and a row is a whole number of vectors,
// one lane moves one 16-byte vector and reads the (cached) row index once; consecutive
// lanes cover consecutive vectors of a row, so both the scattered source rows and the
// dense destination are accessed in full 64-byte-or-larger segments.
#include "common.hip.h"

template <typename V> __device__ __forceinline__ void gather_rows_impl(const hck_gather_rows_args& p) {
  const uint64_t v = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;
  const uint32_t row = (uint32_t)(v / p.row_vecs);
  if (row >= p.total_rows) return;
  const uint32_t c = (uint32_t)(v - (uint64_t)row * p.row_vecs);
  uint32_t off[1];
  size_t unused;
  bcast_offsets<1, 1>(p.idx, row, off, unused);
  const int64_t idx = p.indices[off[0]];
  const uint32_t i = row / p.out_count;
  const int64_t src_row = (int64_t)i * p.middle + idx;
  ((V*)p.out)[v] = ((const V*)p.in)[src_row * (int64_t)p.row_vecs + c];
}

struct alignas(16) V16 { uint32_t x[4]; };

// Long rows (a multiple of 64 * T vectors): one wave moves 64 * T consecutive vectors of one
// row. The row index is wave-uniform, so it is fetched once per wave, and every lane has T
// independent 16-byte loads in flight.
template <int T> __device__ __forceinline__ void gather_rows_wide_impl(const hck_gather_rows_args& p) {
  const uint32_t units_per_row = p.row_vecs / (64 * T);
  const uint64_t unit = (uint64_t)blockIdx.x * (HCK_BLOCK / 64) + (threadIdx.x >> 6);
  const uint32_t row = __builtin_amdgcn_readfirstlane((uint32_t)(unit / units_per_row));
  if (row >= p.total_rows) return;
  const uint32_t chunk = __builtin_amdgcn_readfirstlane((uint32_t)(unit - (uint64_t)row * units_per_row));
  uint32_t off[1];
  size_t unused;
  bcast_offsets<1, 1>(p.idx, row, off, unused);
  const int64_t idx = p.indices[off[0]];
  const uint32_t i = row / p.out_count;
  const int64_t src_row = (int64_t)i * p.middle + idx;
  const uint32_t c = chunk * (64 * T) + (threadIdx.x & 63);
  const V16* src = (const V16*)p.in + src_row * (int64_t)p.row_vecs + c;
  V16* dst = (V16*)p.out + (uint64_t)row * p.row_vecs + c;
  V16 v[T];
#pragma unroll
  for (int t = 0; t < T; t++) v[t] = src[t * 64];
#pragma unroll
  for (int t = 0; t < T; t++) dst[t * 64] = v[t];
}
HC_KERNEL void hc_gather_rows_wide4(hck_gather_rows_args p) { gather_rows_wide_impl<4>(p); }
HC_KERNEL void hc_gather_rows_wide1(hck_gather_rows_args p) { gather_rows_wide_impl<1>(p); }

HC_KERNEL void hc_gather_rows_b16(hck_gather_rows_args p) { gather_rows_impl<V16>(p); }
HC_KERNEL void hc_gather_rows_b8(hck_gather_rows_args p) { gather_rows_impl<uint64_t>(p); }
HC_KERNEL void hc_gather_rows_b4(hck_gather_rows_args p) { gather_rows_impl<uint32_t>(p); }
HC_KERNEL void hc_gather_rows_b2(hck_gather_rows_args p) { gather_rows_impl<uint16_t>(p); }
HC_KERNEL void hc_gather_rows_b1(hck_gather_rows_args p) { gather_rows_impl<uint8_t>(p); }

// General form: one lane per output element, full index map.
template <typename V> __device__ __forceinline__ void gather_elems_impl(const hck_gather_elems_args& p) {
  const uint32_t o = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (o >= p.total) return;
  uint32_t off[1];
  size_t unused;
  bcast_offsets<1, 1>(p.idx, o, off, unused);
  const int64_t idx = p.indices[off[0]];
  const uint32_t ij = o / p.inner;
  const uint32_t k = o - ij * p.inner;
  const uint32_t i = ij / p.out_count;
  ((V*)p.out)[o] = ((const V*)p.in)[((int64_t)i * p.middle + idx) * (int64_t)p.inner + k];
}
HC_KERNEL void hc_gather_elems_b8(hck_gather_elems_args p) { gather_elems_impl<uint64_t>(p); }
HC_KERNEL void hc_gather_elems_b4(hck_gather_elems_args p) { gather_elems_impl<uint32_t>(p); }
HC_KERNEL void hc_gather_elems_b2(hck_gather_elems_args p) { gather_elems_impl<uint16_t>(p); }
HC_KERNEL void hc_gather_elems_b1(hck_gather_elems_args p) { gather_elems_impl<uint8_t>(p); }

// scatter (BackendCPU.swift:1149-1188): one lane per input element; values that share an
// index add up. The output is zeroed by the caller. Float sums are formed with hardware
// atomics, i.e. in no fixed order (the CPU adds in (i, j, k) order); half inputs accumulate
// into a float buffer that the caller rounds once afterwards, as the CPU does.
template <typename TI, typename TO> __device__ __forceinline__ void scatter_add_impl(const hck_gather_elems_args& p) {
  const uint32_t o = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (o >= p.total) return;
  uint32_t off[1];
  size_t unused;
  bcast_offsets<1, 1>(p.idx, o, off, unused);
  const int64_t idx = p.indices[off[0]];
  const uint32_t ij = o / p.inner;
  const uint32_t k = o - ij * p.inner;
  const uint32_t i = ij / p.out_count;
  TO* dst = (TO*)p.out + ((int64_t)i * p.middle + idx) * (int64_t)p.inner + k;
  const TO v = (TO)((const TI*)p.in)[o];
  __hip_atomic_fetch_add(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
HC_KERNEL void hc_scatter_add_f32(hck_gather_elems_args p) { scatter_add_impl<float, float>(p); }
HC_KERNEL void hc_scatter_add_f16(hck_gather_elems_args p) { scatter_add_impl<half_t, float>(p); }
HC_KERNEL void hc_scatter_add_i64(hck_gather_elems_args p) {
  scatter_add_impl<unsigned long long, unsigned long long>(p);
}

// scatter with indices the caller declares unique: plain stores, any element size.
template <typename V> __device__ __forceinline__ void scatter_set_impl(const hck_gather_elems_args& p) {
  const uint32_t o = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (o >= p.total) return;
  uint32_t off[1];
  size_t unused;
  bcast_offsets<1, 1>(p.idx, o, off, unused);
  const int64_t idx = p.indices[off[0]];
  const uint32_t ij = o / p.inner;
  const uint32_t k = o - ij * p.inner;
  const uint32_t i = ij / p.out_count;
  ((V*)p.out)[((int64_t)i * p.middle + idx) * (int64_t)p.inner + k] = ((const V*)p.in)[o];
}
HC_KERNEL void hc_scatter_set_b8(hck_gather_elems_args p) { scatter_set_impl<uint64_t>(p); }
HC_KERNEL void hc_scatter_set_b4(hck_gather_elems_args p) { scatter_set_impl<uint32_t>(p); }
HC_KERNEL void hc_scatter_set_b2(hck_gather_elems_args p) { scatter_set_impl<uint16_t>(p); }

// Re-pitching copy for GEMM operands whose rows are not 16-byte aligned: element-wise
// accesses (either side may be unaligned), zero beyond the valid columns. A wave owns
// 64 * G consecutive elements of one row and moves 64 consecutive elements per instruction,
// so every access is a dense 128- or 256-byte segment. grid.y = batch.
template <typename V, int G> __device__ __forceinline__ void copy2d_impl(const hck_copy2d_args& p) {
  const uint32_t groups = (p.out_cols + 64 * G - 1) / (64 * G);
  const uint64_t unit = (uint64_t)blockIdx.x * (HCK_BLOCK / 64) + (threadIdx.x >> 6);
  const uint64_t r = unit / groups;
  if (r >= p.rows) return;
  const uint32_t c0 = (uint32_t)(unit - r * groups) * (64 * G) + (threadIdx.x & 63);
  const V* src = (const V*)p.in + (uint64_t)blockIdx.y * p.in_bs + r * p.in_ld;
  V* dst = (V*)p.out + (uint64_t)blockIdx.y * p.out_bs + r * p.out_ld;
  V v[G];
#pragma unroll
  for (int e = 0; e < G; e++) v[e] = c0 + e * 64 < p.in_cols ? src[c0 + e * 64] : (V)0;
#pragma unroll
  for (int e = 0; e < G; e++)
    if (c0 + e * 64 < p.out_cols) dst[c0 + e * 64] = v[e];
}
HC_KERNEL void hc_copy2d_b2(hck_copy2d_args p) { copy2d_impl<uint16_t, 8>(p); }
HC_KERNEL void hc_copy2d_b4(hck_copy2d_args p) { copy2d_impl<uint32_t, 8>(p); }

// axisPermutation (BackendCPU.swift:1831-1849): flat source index of every element of the
// permuted view.
HC_KERNEL void hc_axis_permutation(hck_axis_perm_args p) {
  const uint32_t i = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (i >= p.total) return;
  uint32_t flat = 0;
  for (uint32_t d = 0; d < p.ndim; d++)
    flat += p.permuted_strides[d] * ((i / p.new_strides[d]) % p.new_shape[d]);
  p.out[i] = (int64_t)flat;
}

// triangular (BackendCPU.swift:1315-1348): keep the lower (upper) triangle shifted by
// `offset`, zero elsewhere. Row j keeps columns [0, j+1+offset) or [j+offset, cols).
template <typename V> __device__ __forceinline__ void triangular_impl(const hck_triangular_args& p) {
  const uint32_t o = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (o >= p.total) return;
  const uint32_t col = o % p.cols;
  const uint32_t row = (o / p.cols) % p.rows;
  bool keep;
  if (p.upper) {
    keep = (int64_t)col >= (int64_t)row + p.offset;
  } else {
    keep = (int64_t)col < (int64_t)row + 1 + p.offset;
  }
  ((V*)p.out)[o] = keep ? ((const V*)p.in)[o] : (V)0;
}
HC_KERNEL void hc_triangular_b8(hck_triangular_args p) { triangular_impl<uint64_t>(p); }
HC_KERNEL void hc_triangular_b4(hck_triangular_args p) { triangular_impl<uint32_t>(p); }
HC_KERNEL void hc_triangular_b2(hck_triangular_args p) { triangular_impl<uint16_t>(p); }
HC_KERNEL void hc_triangular_b1(hck_triangular_args p) { triangular_impl<uint8_t>(p); }

// concat (BackendCPU.swift:1768-1794), one launch per input: byte copy of an
// [outer, inner] block into a column range of the [outer, total_inner] output.
HC_KERNEL void hc_concat_bytes(hck_concat_args p) {
  const uint64_t t = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;
  const uint64_t total = (uint64_t)p.outer * p.inner;
  if (t >= total) return;
  const uint32_t o = (uint32_t)(t / p.inner);
  const uint32_t c = (uint32_t)(t - (uint64_t)o * p.inner);
  ((uint8_t*)p.out)[(uint64_t)o * p.total_inner + p.out_off + c] = ((const uint8_t*)p.in)[t];
}
