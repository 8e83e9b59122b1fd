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

// Row scatter with repeated indices (rows of whole 16-byte vectors): no atomics on the data.
// Pass 1 counts the sources of every destination row, the host scans the counts, pass 2 drops
// every source row number into its destination's slice of `list` (in whatever order the
// atomics on the cursors resolve), pass 3 gives every destination row to one workgroup, which
// sorts its slice and adds the sources in ascending order: the order of the CPU loop
// (BackendCPU.swift:1149-1188), so float sums match it bit for bit and runs repeat exactly.
HC_KERNEL void hc_scatter_rows_count(hck_scatter_rows_args p) {
  const uint32_t r = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (r >= p.total_src) return;
  uint32_t off[1];
  size_t unused;
  bcast_offsets<1, 1>(p.idx, r, off, unused);
  const uint64_t bucket = (uint64_t)(r / p.n_src) * p.n_dst + (uint64_t)p.indices[off[0]];
  __hip_atomic_fetch_add((unsigned long long*)p.counts + bucket, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

HC_KERNEL void hc_scatter_rows_fill(hck_scatter_rows_args p) {
  const uint32_t r = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (r >= p.total_src) return;
  uint32_t off[1];
  size_t unused;
  bcast_offsets<1, 1>(p.idx, r, off, unused);
  const uint64_t bucket = (uint64_t)(r / p.n_src) * p.n_dst + (uint64_t)p.indices[off[0]];
  const unsigned long long slot =
      __hip_atomic_fetch_add((unsigned long long*)p.cursor + bucket, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  p.list[p.starts[bucket] + (int64_t)slot] = r;
}

// Ascending sort of n distinct values by the whole workgroup: a bitonic network whose
// comparators all point the same way (each merge starts with a mirrored stage), so positions
// past n behave as +infinity and n need not be a power of two. Works on LDS or global memory.
__device__ __forceinline__ void sort_ascending(uint32_t* a, uint32_t n) {
  uint32_t N = 1;
  while (N < n) N <<= 1;
  auto exchange = [&](uint32_t i, uint32_t j) {
    if (j < n) {
      const uint32_t x = a[i], y = a[j];
      if (x > y) {
        a[i] = y;
        a[j] = x;
      }
    }
  };
  for (uint32_t k = 2; k <= N; k <<= 1) {
    const uint32_t h = k >> 1;
    for (uint32_t t = threadIdx.x; t < N / 2; t += HCK_BLOCK) {
      const uint32_t blk = t / h, o = t - blk * h;
      exchange(blk * k + o, blk * k + k - 1 - o);
    }
    __threadfence_block();
    __syncthreads();
    for (uint32_t s = h >> 1; s > 0; s >>= 1) {
      for (uint32_t t = threadIdx.x; t < N / 2; t += HCK_BLOCK) {
        const uint32_t i = (t / s) * 2 * s + (t % s);
        exchange(i, i + s);
      }
      __threadfence_block();
      __syncthreads();
    }
  }
}

constexpr uint32_t SCATTER_LDS_ROWS = 4096;

template <typename T> __device__ __forceinline__ void scatter_rows_sum_impl(const hck_scatter_rows_args& p) {
  typedef typename Arith<T>::type C;
  constexpr int VEC = VecWidth<T>::value;
  __shared__ uint32_t held[SCATTER_LDS_ROWS];
  const uint32_t b = blockIdx.x;  // destination row, flat over the outer axis
  const uint32_t n = (uint32_t)p.counts[b];
  uint32_t* src = p.list + p.starts[b];
  if (n > 1 && n <= SCATTER_LDS_ROWS) {
    for (uint32_t t = threadIdx.x; t < n; t += HCK_BLOCK) held[t] = src[t];
    __syncthreads();
    sort_ascending(held, n);
    src = held;
  } else if (n > SCATTER_LDS_ROWS) {
    sort_ascending(src, n);  // in place in global memory: rare (one row receiving > 4096 sources)
  }
  const T* in = (const T*)p.in;
  T* out = (T*)p.out + (size_t)b * p.row_vecs * VEC;
  for (uint32_t c = threadIdx.x; c < p.row_vecs; c += HCK_BLOCK) {
    C acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) acc[v] = (C)0;
    uint32_t t = 0;
    for (; t + 4 <= n; t += 4) {  // four loads in flight, added in order
      T x[4][VEC];
#pragma unroll
      for (int u = 0; u < 4; u++) load_vec<T, VEC>(in + ((size_t)src[t + u] * p.row_vecs + c) * VEC, 0, 1, x[u]);
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int v = 0; v < VEC; v++) acc[v] = acc[v] + to_arith(x[u][v]);
    }
    for (; t < n; t++) {
      T x[VEC];
      load_vec<T, VEC>(in + ((size_t)src[t] * p.row_vecs + c) * VEC, 0, 1, x);
#pragma unroll
      for (int v = 0; v < VEC; v++) acc[v] = acc[v] + to_arith(x[v]);
    }
    T o[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) o[v] = from_arith<T>(acc[v]);
    store_vec<T, VEC>(out, (size_t)c * VEC, o);
  }
}
HC_KERNEL void hc_scatter_rows_sum_f32(hck_scatter_rows_args p) { scatter_rows_sum_impl<float>(p); }
HC_KERNEL void hc_scatter_rows_sum_f16(hck_scatter_rows_args p) { scatter_rows_sum_impl<half_t>(p); }
HC_KERNEL void hc_scatter_rows_sum_i64(hck_scatter_rows_args p) { scatter_rows_sum_impl<int64_t>(p); }

// Re-pitching copies for GEMM operands and outputs whose rows are not 16-byte aligned. One side
// is always the library's own padded copy (base, leading dimension and batch stride multiples
// of 16 bytes), the other side is the caller's matrix, aligned to its element size only.
// A lane owns a 16-byte piece of the padded side, a wave 512 consecutive elements of one row;
// grid.y = batch. Multi-dword accesses of the caller's side need dword alignment only:
//   pad   (caller -> padded copy, zero beyond in_cols): 4-byte elements load the piece directly;
//         2-byte elements on an odd element address load the five dwords around the piece and
//         shift them by two bytes. Lanes whose window would reach past the last element of the
//         last matrix take element-wise loads instead.
//   unpad (padded result -> caller): a piece on an odd element address leaves as
//         half + three dwords + half.
typedef uint32_t CopyPiece __attribute__((ext_vector_type(4)));
typedef CopyPiece CopyPieceA4 __attribute__((aligned(4)));
template <typename V> __device__ __forceinline__ void copy2d_pad_impl(const hck_copy2d_args& p) {
  constexpr uint32_t PE = 16 / sizeof(V);            // elements per piece
  constexpr uint32_t NP = 512 / (64 * PE);           // pieces per lane
  const uint32_t groups = (p.out_cols + 511) / 512;
  const uint64_t unit = (uint64_t)blockIdx.x * (HCK_BLOCK / 64) + (threadIdx.x >> 6);
  const uint64_t r = unit / groups;
  if (r >= p.rows) return;
  const uint32_t g0 = (uint32_t)(unit - r * groups) * 512;
  // one past the last element that may be read, relative to p.in
  const uint64_t lim = (uint64_t)(gridDim.y - 1) * p.in_bs + (uint64_t)(p.rows - 1) * p.in_ld + p.in_cols;
  const uint64_t row0 = (uint64_t)blockIdx.y * p.in_bs + r * p.in_ld;
  V* dst = (V*)p.out + (uint64_t)blockIdx.y * p.out_bs + r * p.out_ld;
#pragma unroll
  for (uint32_t i = 0; i < NP; i++) {
    const uint32_t c = g0 + ((threadIdx.x & 63) + 64 * i) * PE;
    if (c >= p.out_cols) continue;
    const uint64_t e0 = row0 + c;
    const V* src = (const V*)p.in + e0;
    CopyPiece o = {0u, 0u, 0u, 0u};
    if (c < p.in_cols) {
      if (e0 + PE + 2 <= lim) {
        const uint32_t sh = sizeof(V) == 2 ? (uint32_t)((uintptr_t)src & 2) : 0u;
        const char* sa = (const char*)src - sh;
        const CopyPiece w = *reinterpret_cast<const CopyPieceA4*>(sa);
        if (sh != 0) {
          const uint32_t w4 = *reinterpret_cast<const uint32_t*>(sa + 16);
          o[0] = (w[0] >> 16) | (w[1] << 16);
          o[1] = (w[1] >> 16) | (w[2] << 16);
          o[2] = (w[2] >> 16) | (w[3] << 16);
          o[3] = (w[3] >> 16) | (w4 << 16);
        } else {
          o = w;
        }
      } else {
        V e[PE];
#pragma unroll
        for (uint32_t j = 0; j < PE; j++) e[j] = e0 + j < lim ? src[j] : (V)0;
        if constexpr (sizeof(V) == 2) {
#pragma unroll
          for (uint32_t j = 0; j < 4; j++) o[j] = (uint32_t)e[2 * j] | ((uint32_t)e[2 * j + 1] << 16);
        } else {
#pragma unroll
          for (uint32_t j = 0; j < 4; j++) o[j] = (uint32_t)e[j];
        }
      }
      if (c + PE > p.in_cols) {  // zero beyond the valid columns
        const uint32_t n = p.in_cols - c;  // 1 .. PE-1 valid elements
#pragma unroll
        for (uint32_t j = 0; j < 4; j++) {
          if constexpr (sizeof(V) == 2) {
            if (2 * j >= n) o[j] = 0u;
            else if (2 * j + 1 >= n) o[j] &= 0xffffu;
          } else {
            if (j >= n) o[j] = 0u;
          }
        }
      }
    }
    *reinterpret_cast<CopyPiece*>(dst + c) = o;
  }
}
HC_KERNEL void hc_copy2d_pad_b2(hck_copy2d_args p) { copy2d_pad_impl<uint16_t>(p); }
HC_KERNEL void hc_copy2d_pad_b4(hck_copy2d_args p) { copy2d_pad_impl<uint32_t>(p); }

template <typename V> __device__ __forceinline__ void copy2d_unpad_impl(const hck_copy2d_args& p) {
  constexpr uint32_t PE = 16 / sizeof(V);
  constexpr uint32_t NP = 512 / (64 * PE);
  const uint32_t groups = (p.out_cols + 511) / 512;
  const uint64_t unit = (uint64_t)blockIdx.x * (HCK_BLOCK / 64) + (threadIdx.x >> 6);
  const uint64_t r = unit / groups;
  if (r >= p.rows) return;
  const uint32_t g0 = (uint32_t)(unit - r * groups) * 512;
  const V* src = (const V*)p.in + (uint64_t)blockIdx.y * p.in_bs + r * p.in_ld;
  V* drow = (V*)p.out + (uint64_t)blockIdx.y * p.out_bs + r * p.out_ld;
#pragma unroll
  for (uint32_t i = 0; i < NP; i++) {
    const uint32_t c = g0 + ((threadIdx.x & 63) + 64 * i) * PE;
    if (c >= p.out_cols) continue;
    const CopyPiece v = *reinterpret_cast<const CopyPiece*>(src + c);
    V* dst = drow + c;
    const uint32_t n = p.out_cols - c < PE ? p.out_cols - c : PE;
    if (n == PE && ((uintptr_t)dst & 3) == 0) {
      *reinterpret_cast<CopyPieceA4*>(dst) = v;
    } else if (sizeof(V) == 2 && n == PE) {
      uint16_t* d16 = reinterpret_cast<uint16_t*>(dst);
      d16[0] = (uint16_t)v[0];
      uint32_t* d32 = reinterpret_cast<uint32_t*>(d16 + 1);
      d32[0] = (v[0] >> 16) | (v[1] << 16);
      d32[1] = (v[1] >> 16) | (v[2] << 16);
      d32[2] = (v[2] >> 16) | (v[3] << 16);
      d16[7] = (uint16_t)(v[3] >> 16);
    } else {
#pragma unroll
      for (uint32_t j = 0; j < PE; j++) {
        if (j < n) {
          if constexpr (sizeof(V) == 2) dst[j] = (V)(v[j / 2] >> (16 * (j & 1)));
          else dst[j] = (V)v[j];
        }
      }
    }
  }
}
HC_KERNEL void hc_copy2d_unpad_b2(hck_copy2d_args p) { copy2d_unpad_impl<uint16_t>(p); }
HC_KERNEL void hc_copy2d_unpad_b4(hck_copy2d_args p) { copy2d_unpad_impl<uint32_t>(p); }

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

// The gather that follows an axisPermutation, done directly: the same data movement as
// gather(in, axisPermutation(perm, shape)) (Index.swift:238-266, BackendCPU.swift:1108-1147),
// without writing and re-reading 8 bytes of index per element.
// Row form: a lane per VEC consecutive elements of the shared innermost axis.
template <typename V, int VEC> __device__ __forceinline__ void permute_rows_impl(const hck_permute_args& p) {
  const uint32_t v = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v >= p.total) return;
  uint32_t row = fast_div(v, p.inner_magic, p.inner_sh);
  const uint32_t col = (v - row * p.inner_vecs) * VEC;
  const size_t out_off = (size_t)row * p.inner + col;
  size_t in_off = col;
  for (int d = (int)p.ndim - 1; d >= 0; d--) {
    const uint32_t q = fast_div(row, p.magic[d], p.sh[d]);
    in_off += (size_t)(row - q * p.shape[d]) * p.in_stride[d];
    row = q;
  }
  typedef Vec<V, VEC> Pack;
  *reinterpret_cast<Pack*>((V*)p.out + out_off) = *reinterpret_cast<const Pack*>((const V*)p.in + in_off);
}
// Tile form: tiles of ta x tc elements (powers of two, ta * tc <= 4096: 64 x 64, or longer and
// narrower when one of the two axes is short) through LDS. Reads run along the source's innermost
// axis c, writes along the output's innermost axis a, both with all lanes on consecutive
// elements; one padding element per LDS row keeps the transposed accesses off the same banks.
template <typename V> __device__ __forceinline__ void permute_tile_impl(const hck_permute_args& p) {
  __shared__ V tile[4096 + 1024];
  uint32_t t = blockIdx.x;
  uint32_t q = fast_div(t, p.tiles_c_magic, p.tiles_c_sh);
  const uint32_t c0 = (t - q * p.tiles_c) << p.tc_log2;
  t = q;
  q = fast_div(t, p.tiles_a_magic, p.tiles_a_sh);
  const uint32_t a0 = (t - q * p.tiles_a) << p.ta_log2;
  uint32_t rest = q;
  size_t in_base = 0, out_base = 0;
  for (int d = (int)p.ndim - 1; d >= 0; d--) {
    const uint32_t qq = fast_div(rest, p.magic[d], p.sh[d]);
    const uint32_t r = rest - qq * p.shape[d];
    in_base += (size_t)r * p.in_stride[d];
    out_base += (size_t)r * p.out_stride[d];
    rest = qq;
  }
  const V* in = (const V*)p.in + in_base;
  V* out = (V*)p.out + out_base;
  if (p.ta_log2 == 6 && p.tc_log2 == 6) {
    // the common shape, with compile-time extents
    const uint32_t x = threadIdx.x & 63, y0 = threadIdx.x >> 6;
#pragma unroll 4
    for (uint32_t i = 0; i < 16; i++) {
      const uint32_t a = y0 + 4 * i;
      if (a0 + a < p.tile_a && c0 + x < p.tile_c) tile[a * 65 + x] = in[(size_t)(a0 + a) * p.a_stride + c0 + x];
    }
    __syncthreads();
#pragma unroll 4
    for (uint32_t i = 0; i < 16; i++) {
      const uint32_t c = y0 + 4 * i;
      if (c0 + c < p.tile_c && a0 + x < p.tile_a) out[(size_t)(c0 + c) * p.c_out_stride + a0 + x] = tile[x * 65 + c];
    }
    return;
  }
  const uint32_t n = 1u << (p.ta_log2 + p.tc_log2), pitch = (1u << p.tc_log2) + 1;
  for (uint32_t idx = threadIdx.x; idx < n; idx += HCK_BLOCK) {
    const uint32_t a = idx >> p.tc_log2, c = idx & ((1u << p.tc_log2) - 1);
    if (a0 + a < p.tile_a && c0 + c < p.tile_c) tile[a * pitch + c] = in[(size_t)(a0 + a) * p.a_stride + c0 + c];
  }
  __syncthreads();
  for (uint32_t idx = threadIdx.x; idx < n; idx += HCK_BLOCK) {
    const uint32_t c = idx >> p.ta_log2, a = idx & ((1u << p.ta_log2) - 1);
    if (a0 + a < p.tile_a && c0 + c < p.tile_c) out[(size_t)(c0 + c) * p.c_out_stride + a0 + a] = tile[a * pitch + c];
  }
}
#define DEF_PERMUTE(B, V)                                                                              \
  HC_KERNEL void hc_permute_rows_b##B##_v1(hck_permute_args p) { permute_rows_impl<V, 1>(p); }         \
  HC_KERNEL void hc_permute_rows_b##B##_vN(hck_permute_args p) { permute_rows_impl<V, 16 / B>(p); }    \
  HC_KERNEL void hc_permute_tile_b##B(hck_permute_args p) { permute_tile_impl<V>(p); }
DEF_PERMUTE(8, uint64_t)
DEF_PERMUTE(4, uint32_t)
DEF_PERMUTE(2, uint16_t)
DEF_PERMUTE(1, uint8_t)

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
// The same with N = 16 / sizeof(V) consecutive columns per lane (cols a multiple of N, buffers
// 16-byte aligned): p.total counts vectors.
template <typename V> __device__ __forceinline__ void triangular_vec_impl(const hck_triangular_args& p) {
  constexpr int N = 16 / sizeof(V);
  const uint32_t v = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v >= p.total) return;
  const uint32_t cvecs = p.cols / N;
  const uint32_t col0 = (v % cvecs) * N;
  const uint32_t row = (v / cvecs) % p.rows;
  Vec<V, N> x = reinterpret_cast<const Vec<V, N>*>(p.in)[v];
#pragma unroll
  for (int e = 0; e < N; e++) {
    const int64_t col = (int64_t)col0 + e;
    const bool keep = p.upper ? col >= (int64_t)row + p.offset : col < (int64_t)row + 1 + p.offset;
    if (!keep) x.v[e] = (V)0;
  }
  reinterpret_cast<Vec<V, N>*>(p.out)[v] = x;
}
HC_KERNEL void hc_triangular_b8_vN(hck_triangular_args p) { triangular_vec_impl<uint64_t>(p); }
HC_KERNEL void hc_triangular_b4_vN(hck_triangular_args p) { triangular_vec_impl<uint32_t>(p); }
HC_KERNEL void hc_triangular_b2_vN(hck_triangular_args p) { triangular_vec_impl<uint16_t>(p); }
HC_KERNEL void hc_triangular_b1_vN(hck_triangular_args p) { triangular_vec_impl<uint8_t>(p); }
HC_KERNEL void hc_triangular_b8(hck_triangular_args p) { triangular_impl<uint64_t>(p); }
HC_KERNEL void hc_triangular_b4(hck_triangular_args p) { triangular_impl<uint32_t>(p); }
HC_KERNEL void hc_triangular_b2(hck_triangular_args p) { triangular_impl<uint16_t>(p); }
HC_KERNEL void hc_triangular_b1(hck_triangular_args p) { triangular_impl<uint8_t>(p); }

// concat (BackendCPU.swift:1768-1794), one launch per input: copy of an [outer, inner] block
// into a column range of the [outer, total_inner] output, in units of U bytes: the host picks the
// largest U <= 16 that divides the block's row length, the output's row length, the column offset
// and both addresses. inner, total_inner and out_off count units.
template <typename U> __device__ __forceinline__ void concat_impl(const hck_concat_args& p) {
  const uint64_t t = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;
  const uint64_t total = (uint64_t)p.outer * p.inner;
  if (t >= total) return;
  const uint32_t o = (uint32_t)(t / p.inner);
  const uint32_t c = (uint32_t)(t - (uint64_t)o * p.inner);
  ((U*)p.out)[(uint64_t)o * p.total_inner + p.out_off + c] = ((const U*)p.in)[t];
}
HC_KERNEL void hc_concat_b1(hck_concat_args p) { concat_impl<uint8_t>(p); }
HC_KERNEL void hc_concat_b2(hck_concat_args p) { concat_impl<uint16_t>(p); }
HC_KERNEL void hc_concat_b4(hck_concat_args p) { concat_impl<uint32_t>(p); }
HC_KERNEL void hc_concat_b8(hck_concat_args p) { concat_impl<uint64_t>(p); }
HC_KERNEL void hc_concat_b16(hck_concat_args p) { concat_impl<V16>(p); }
