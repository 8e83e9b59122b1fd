// Device-side helpers shared by the gfx950 kernels: element traits, 16-byte vector
// access, the broadcast index map, and wave64 / block reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>

#include "../kargs.h"

typedef _Float16 half_t;

#define HC_KERNEL extern "C" __global__ __launch_bounds__(HCK_BLOCK)

// Storage type T -> arithmetic type. The CPU backend stages half through Float and
// rounds once on store (BackendCPU.swift:2018-2058), int64 stays int64.
template <typename T> struct Arith { typedef float type; };
template <> struct Arith<int64_t> { typedef int64_t type; };
template <> struct Arith<uint8_t> { typedef float type; };

template <typename T> __device__ __forceinline__ typename Arith<T>::type to_arith(T v) {
  return (typename Arith<T>::type)v;
}
template <> __device__ __forceinline__ float to_arith<uint8_t>(uint8_t v) {
  return v ? 1.0f : 0.0f;
}

// fp32 -> storage type. For half this is one v_cvt_f16_f32 (round-to-nearest-even, overflow
// to inf) of a value that is first pinned in a VGPR: without the pin the compiler folds a
// preceding multiply into v_fma_mixlo_f16 (a * b + 0), which turns a -0 product into +0.
template <typename T> __device__ __forceinline__ T narrow(float v) { return (T)v; }
template <> __device__ __forceinline__ half_t narrow<half_t>(float v) {
  asm("" : "+v"(v));
  return (half_t)v;
}

template <typename T> __device__ __forceinline__ T from_arith(typename Arith<T>::type v) {
  return (T)v;
}
template <> __device__ __forceinline__ half_t from_arith<half_t>(float v) { return narrow<half_t>(v); }
// Bool(Float) is `value != 0` (TensorElement.swift:179-181), not an integer conversion.
template <> __device__ __forceinline__ uint8_t from_arith<uint8_t>(float v) { return v == 0.0f ? 0 : 1; }

// Round an fp32 intermediate to what the tensor dtype can hold (identity for float).
template <typename T> __device__ __forceinline__ float round_through(float v) {
  return (float)narrow<T>(v);
}
template <> __device__ __forceinline__ float round_through<float>(float v) { return v; }

template <typename T, int N> struct alignas(sizeof(T) * N) Vec {
  T v[N];
};

// Elements per 16-byte access.
template <typename T> struct VecWidth { static constexpr int value = 16 / sizeof(T); };

template <typename T, int N>
__device__ __forceinline__ void load_vec(const T* base, uint32_t off, uint32_t stride, T (&dst)[N]) {
  if (N > 1 && stride == 1) {
    Vec<T, N> t = *reinterpret_cast<const Vec<T, N>*>(base + off);
#pragma unroll
    for (int i = 0; i < N; i++) dst[i] = t.v[i];
  } else {
#pragma unroll
    for (int i = 0; i < N; i++) dst[i] = base[off + i * stride];
  }
}

// N consecutive elements from an address that is aligned to the element only (in the access mode
// the runtime sets, a multi-dword load needs no alignment).
template <typename T, int N> __device__ __forceinline__ void load_vec_loose(const T* src, T (&dst)[N]) {
  struct __attribute__((packed, aligned(sizeof(T)))) Loose {
    Vec<T, N> v;
  };
  const Vec<T, N> t = reinterpret_cast<const Loose*>(src)->v;
#pragma unroll
  for (int i = 0; i < N; i++) dst[i] = t.v[i];
}

// The same with the stride known at compile time: S = 1 one 16-byte load, S = 0 one element
// repeated, S < 0 decided at run time. Kernels branch once on the (wave-uniform) strides of
// all their operands and run a body whose loads are unconditional, so they issue back to back;
// with the run-time form the compiler puts a wait for the first operand's load at the join of
// its two paths, in front of the second operand's load.
template <typename T, int N, int S>
__device__ __forceinline__ void load_vec_c(const T* base, uint32_t off, uint32_t stride, T (&dst)[N]) {
  if (S == 1) {
    Vec<T, N> t = *reinterpret_cast<const Vec<T, N>*>(base + off);
#pragma unroll
    for (int i = 0; i < N; i++) dst[i] = t.v[i];
  } else if (S == 0) {
    const T x = base[off];
#pragma unroll
    for (int i = 0; i < N; i++) dst[i] = x;
  } else {
    load_vec<T, N>(base, off, stride, dst);
  }
}
template <int S> using StrideC = std::integral_constant<int, S>;
// f(sa, sb) with the inner strides of two operands as StrideC constants: both vectors, one
// vector and one repeated element, or "run time" for anything else (and for VEC = 1, where
// every load is a single element anyway).
template <int VEC, typename F> __device__ __forceinline__ void with_strides2(const uint32_t* s, F&& f) {
  if (VEC > 1 && s[0] == 1 && s[1] == 1) f(StrideC<1>{}, StrideC<1>{});
  else if (VEC > 1 && s[0] == 1 && s[1] == 0) f(StrideC<1>{}, StrideC<0>{});
  else if (VEC > 1 && s[0] == 0 && s[1] == 1) f(StrideC<0>{}, StrideC<1>{});
  else f(StrideC<-1>{}, StrideC<-1>{});
}
// f(s) for NOPS operands that share one constant: all vectors, or "run time".
template <int VEC, int NOPS, typename F> __device__ __forceinline__ void with_strides_all(const uint32_t* s, F&& f) {
  bool ones = VEC > 1;
  for (int o = 0; o < NOPS; o++) ones = ones && s[o] == 1;
  if (ones) f(StrideC<1>{});
  else f(StrideC<-1>{});
}

template <typename T, int N>
__device__ __forceinline__ void store_vec(T* base, size_t off, const T (&src)[N]) {
  Vec<T, N> t;
#pragma unroll
  for (int i = 0; i < N; i++) t.v[i] = src[i];
  *reinterpret_cast<Vec<T, N>*>(base + off) = t;
}

// n / d with the (magic, sh) pair the host derived from d (hck_fast_div_setup): exact for every
// 32-bit n, five instructions instead of the division sequence.
__device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t magic, uint32_t sh) {
  const uint32_t t = __umulhi(magic, n);
  return (t + ((n - t) >> (sh & 0xffu))) >> (sh >> 8);
}

// Broadcast index map (Broadcast.swift:72-90) for NOPS operands at once: vector number
// v -> element offsets of the first of VEC inner elements, and the flat output offset.
template <int NOPS, int VEC>
__device__ __forceinline__ void bcast_offsets(const hck_bcast& d, uint32_t v, uint32_t (&off)[NOPS],
                                              size_t& out_off) {
  uint32_t row = fast_div(v, d.inner_magic, d.inner_sh);
  uint32_t col = (v - row * d.inner_vecs) * VEC;
  out_off = (size_t)row * d.inner + col;
#pragma unroll
  for (int o = 0; o < NOPS; o++) off[o] = col * d.inner_stride[o];
  for (int k = (int)d.n_outer - 1; k >= 0; k--) {
    uint32_t s = d.outer_shape[k];
    uint32_t q = fast_div(row, d.outer_magic[k], d.outer_sh[k]);
    uint32_t r = row - q * s;
#pragma unroll
    for (int o = 0; o < NOPS; o++) off[o] += r * d.outer_stride[o][k];
    row = q;
  }
}

// powf for the pow / normalize / AdamW kernels. Exponents 2, 0.5 and -0.5 (squares, roots and
// reciprocal roots: LayerNorm and Adam) take correctly rounded multiplies / square roots instead
// of the generic exp2(y * log2(x)) evaluation, with powf's results at zero and infinity;
// everything else is the device library's powf. All callers share this one function, so a
// fused kernel and the op-by-op composition agree bit for bit.
__device__ __forceinline__ float pow_like(float x, float b) {
  if (b == 2.0f) return x * x;
  if (b == 0.5f) {
    if (x == 0.0f) return 0.0f;
    if (x == -INFINITY) return INFINITY;
    return sqrtf(x);
  }
  if (b == -0.5f) {
    if (x == 0.0f) return INFINITY;
    if (x == -INFINITY) return 0.0f;
    return 1.0f / sqrtf(x);
  }
  return powf(x, b);
}

// ---- wave64 / block reductions ----

template <typename V, typename Op> __device__ __forceinline__ V wave_reduce(V v, Op op) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = op(v, __shfl_xor(v, o, 64));
  return v;
}

struct SumOp {
  template <typename V> __device__ __forceinline__ V operator()(V a, V b) const { return a + b; }
};
struct ProdOp {
  template <typename V> __device__ __forceinline__ V operator()(V a, V b) const { return a * b; }
};
struct MaxOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a > b ? a : b; }
};

// Reduce across the HCK_BLOCK threads of a block; every thread gets the result.
template <typename V, typename Op>
__device__ __forceinline__ V block_reduce(V v, Op op, V* lds /* >= 4 entries */) {
  v = wave_reduce(v, op);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[wave] = v;
  __syncthreads();
  V r = lds[0];
#pragma unroll
  for (int w = 1; w < HCK_BLOCK / 64; w++) r = op(r, lds[w]);
  return r;
}

// Tile (tm, tn) of a GEMM block for the direct-to-LDS kernels. Block ids equal mod 8 run on one
// XCD and share its L2: each XCD gets a compact rectangle of tiles (few distinct A and B panels)
// inside a super-block, or, without the rectangle parameters, a contiguous band. The host only
// passes powers of two for xcd_gn, xcd_sm and xcd_sn, so their divisions are shifts; one real
// division (by the number of super-blocks per row, or by tiles_n) remains.
__device__ __forceinline__ void gemm_tile_of_block(const hck_gemm_args& p, uint32_t block, uint32_t& tm, uint32_t& tn) {
  if (p.xcd_gn != 0) {
    const uint32_t lg = (uint32_t)__builtin_ctz(p.xcd_gn), lsm = (uint32_t)__builtin_ctz(p.xcd_sm),
                   lsn = (uint32_t)__builtin_ctz(p.xcd_sn);
    const uint32_t lper = 3 + lsm + lsn;             // blocks per super-block: 8 XCDs x sm x sn
    const uint32_t group = block >> lper, w = block & ((1u << lper) - 1u);
    const uint32_t x = w & 7u, t = w >> 3;
    const uint32_t sbn = p.tiles_n >> (lg + lsn);    // super-blocks per row of super-blocks
    const uint32_t sb_row = group / sbn, sb_col = group - sb_row * sbn;
    const uint32_t xm = x >> lg, xn = x & (p.xcd_gn - 1u);
    const uint32_t lm = t >> lsn, ln = t & (p.xcd_sn - 1u);
    tm = (((sb_row << (3 - lg)) + xm) << lsm) + lm;
    tn = (((sb_col << lg) + xn) << lsn) + ln;
    return;
  }
  const uint32_t total = p.tiles_m * p.tiles_n;
  uint32_t tile = block;
  if ((total & 7u) == 0) tile = (block & 7u) * (total >> 3) + (block >> 3);
  tm = tile / p.tiles_n;
  tn = tile - tm * p.tiles_n;
}

// Block (within its product) and batch slice of a workgroup of a batched launch (grid.x = blocks per product,
// grid.y = slices). Workgroups go to the eight XCDs round robin in launch order, x fastest: as launched, the blocks
// of one slice are spread over all XCDs and every XCD's L2 fetches every slice's operands. With 8 slices or more
// of at most 8 blocks each, the blocks of a slice are handed to workgroups 8 apart instead (slices in groups of 8;
// what is left over keeps the launch order), so a slice's operands are fetched by one XCD: 32 x [512, 512] x
// [512, 64] in 8 blocks per slice 7.2 -> 5.2 us. (Slices of many blocks already give every XCD a few neighbouring
// tiles; with 32 blocks per slice all on one XCD the same lines are wanted by 32 CUs at once, and 32 x
// [512, 64] x [64, 512] took 6.7 instead of 6.2 us.) Grouped products (grid.y = members over the same A, at most
// 4) are not touched.
__device__ __forceinline__ void gemm_block_and_batch(uint32_t& block, uint32_t& batch) {
  block = blockIdx.x;
  batch = blockIdx.y;
  const uint32_t nx = gridDim.x, ny = gridDim.y;
  if (ny < 8 || nx > 8) return;
  const uint32_t l = blockIdx.y * nx + blockIdx.x, grouped = ny / 8 * 8 * nx;
  if (l < grouped) {
    const uint32_t g = l / (8 * nx), r = l - g * 8 * nx;
    batch = 8 * g + (r & 7);
    block = r >> 3;
  }
}

// ---- operations merged into a GEMM's epilogue (hck_gemm_args::ep_*) ----
#include "elemwise_formulas.hip.h"

// 1 in the second build of the tiled GEMM sources (kernels *_m, whose write-out applies the operations
// a recording merged into the product), 0 in the ordinary build
#ifdef HC_GEMM_MERGED
#define HC_GEMM_IS_MERGED 1
#else
#define HC_GEMM_IS_MERGED 0
#endif

// The operations are applied to 16-byte pieces of finished outputs of type T (already rounded to
// T), in order, each in float with one rounding to T: bit for bit what the separate broadcast-add /
// element-wise kernels would have produced. A lane's pieces all lie in the same columns, so the row
// operands (a bias) are fetched once per kernel; the matrix operand (at most one of the three
// operations) is fetched for a few pieces at a time, all loads in flight before the first use.
// Entry `member` (wave-uniform, < 4) of a table in the kernel's argument struct, picked with scalar
// selects. An index computed at run time would make the compiler fetch the entry with a vector
// load; its result then sits in the same in-order counter as the direct-to-LDS loads of the main
// loop, and the first use waits for every one of those: the whole prefetch pipeline drains before
// the first MFMA (a 2048 x 512 x 2048 product took 24 us instead of 9).
template <typename P> __device__ __forceinline__ P gemm_table_entry(const P (&table)[4], uint32_t member) {
  return member == 0 ? table[0] : member == 1 ? table[1] : member == 2 ? table[2] : table[3];
}
// The operand of stage s for this workgroup's product (a member of a group has its own). The three
// are kept as three values, never as a struct or an array: an aggregate whose member is picked by
// a run-time condition ends up in memory (the compiler promoted it to LDS, and the LDS write that
// this takes waits for every direct-to-LDS load in flight).
__device__ __forceinline__ const void* gemm_epilogue_operand(const hck_gemm_args& p, int s, uint32_t member) {
  if (p.group != 0) return s == 0 ? gemm_table_entry(p.g_ep[0], member) : s == 1 ? gemm_table_entry(p.g_ep[1], member) : gemm_table_entry(p.g_ep[2], member);
  return s == 0 ? p.ep_ptr[0] : s == 1 ? p.ep_ptr[1] : p.ep_ptr[2];
}

// One 16-byte piece of C (row `row`, columns col .. col + 16 / sizeof(T) - 1) leaves a tiled GEMM
// kernel; `staged` is where the piece sits in LDS. Edge kernels skip pieces outside C. LOOSE (the
// edge kernels of the ordinary build): a row of C may start at any element (in the access mode the
// runtime sets, multi-dword stores need no alignment), and the piece that straddles N leaves
// element by element, in a loop that stays rolled (it runs for one piece per row at most and must
// not cost the write-out registers). Without LOOSE, N is a whole number of pieces.
template <typename T, typename Chunk16, bool EDGE, bool LOOSE>
__device__ __forceinline__ void gemm_store_piece(T* dst, uint32_t row, uint32_t col, uint32_t M, uint32_t N, Chunk16 v,
                                                 const char* staged) {
  static_assert(sizeof(Chunk16) == 16, "a 16-byte piece");
  if constexpr (!LOOSE) {
    if (!EDGE || (row < M && col < N)) *reinterpret_cast<Chunk16*>(dst) = v;
  } else if (row < M) {
    constexpr uint32_t PER = 16 / sizeof(T);
    if (col + PER <= N) {
      struct __attribute__((packed, aligned(sizeof(T)))) Loose {
        Chunk16 v;
      };
      reinterpret_cast<Loose*>(dst)->v = v;
    } else if (col < N) {
      const T* e = reinterpret_cast<const T*>(staged);
#pragma nounroll
      for (uint32_t x = 0; x < N - col; x++) dst[x] = e[x];
    }
  }
}

// Edge kernels, K-contiguous operand (a lane's DMA piece i of a K-slice covers k = kl .. kl +
// 16 / sizeof(T) - 1 of one row and sits at `piece`): when K is not a whole number of pieces, the
// piece that straddles K also holds what follows the row in memory (the next row's first elements
// where rows abut). The lane that fetched it clears those elements once its DMA has landed and
// before the barrier that lets anybody read the slice.
template <typename T> __device__ __forceinline__ void gemm_zero_piece_tail(char* piece, uint32_t kl, uint32_t kend) {
  constexpr uint32_t PER = 16 / sizeof(T);
  if (kl < kend && kl + PER > kend) {
    T* e = reinterpret_cast<T*>(piece);
#pragma unroll
    for (uint32_t x = 1; x < PER; x++)
      if (kl + x >= kend) e[x] = T(0);
  }
}

template <typename T, typename Chunk16>
__device__ __forceinline__ Chunk16 gemm_epilogue_row_piece(uint32_t kind, const void* ptr, uint32_t col, bool col_ok) {
  constexpr int V = 16 / sizeof(T);
  static_assert(sizeof(Chunk16) == 16, "a 16-byte piece");
  Chunk16 out = Chunk16{};
  if (!col_ok) return out;
  if (kind == HCK_EP_ADD_ROW) {
    out = *reinterpret_cast<const Chunk16*>((const T*)ptr + col);
  } else if (kind == HCK_EP_ADD_ROW_F32) {
    const float* src = (const float*)ptr + col;
    T y[V];
#pragma unroll
    for (int e = 0; e < V; e += 4) {
      const float4 w = *reinterpret_cast<const float4*>(src + e);
      y[e] = narrow<T>(w.x), y[e + 1] = narrow<T>(w.y), y[e + 2] = narrow<T>(w.z), y[e + 3] = narrow<T>(w.w);
    }
    __builtin_memcpy(&out, y, 16);
  }
  return out;
}

// the matrix operand's piece for the output piece at (row, col); one of the stages has one
template <typename T, typename Chunk16>
__device__ __forceinline__ Chunk16 gemm_epilogue_matrix_piece(const hck_gemm_args& p, const void* p0, const void* p1,
                                                              const void* p2, uint32_t row, uint32_t col) {
  // (stage picked with scalar selects, then a single load: no register is written twice)
  const bool s0 = p.ep_kind[0] == HCK_EP_ADD_MATRIX, s1 = p.ep_kind[1] == HCK_EP_ADD_MATRIX;
  const void* base = s0 ? p0 : s1 ? p1 : p2;
  const uint32_t ld = s0 ? p.ep_ld[0] : s1 ? p.ep_ld[1] : p.ep_ld[2];
  return *reinterpret_cast<const Chunk16*>((const T*)base + (size_t)row * ld + col);
}

// r0, r1, r2: the row operands of the three stages (gemm_epilogue_row_piece; passed as three values
// so that nothing can index them and they stay in registers). Straight-line code: up to three
// additions (wave-uniform branches skip the absent ones), then, in the GELU instantiation, the
// activation: the host puts GELU only at the end of a list, and never together with a matrix
// operand. (A loop over the stages with the operation picked inside cost 7 us on a 256 x 256 tile
// for a single bias addition; this form costs 1 us.)
template <typename T, typename Chunk16, bool MATRIX, bool GELU>
__device__ __forceinline__ Chunk16 gemm_epilogue_apply(const hck_gemm_args& p, Chunk16 v, Chunk16 r0, Chunk16 r1, Chunk16 r2,
                                                       Chunk16 matrix_piece) {
  constexpr int V = 16 / sizeof(T);
  T x[V];
  __builtin_memcpy(x, &v, 16);
  const uint32_t k0 = p.ep_kind[0], k1 = p.ep_kind[1], k2 = p.ep_kind[2];
  auto add = [&](uint32_t kind, Chunk16 row) {
    const Chunk16 w = MATRIX && kind == HCK_EP_ADD_MATRIX ? matrix_piece : row;
    T y[V];
    __builtin_memcpy(y, &w, 16);
#pragma unroll
    for (int e = 0; e < V; e++) x[e] = narrow<T>((float)x[e] + (float)y[e]);
  };
  auto is_add = [](uint32_t kind) { return kind == HCK_EP_ADD_ROW || kind == HCK_EP_ADD_ROW_F32 || kind == HCK_EP_ADD_MATRIX; };
  if (is_add(k0)) add(k0, r0);
  if (is_add(k1)) add(k1, r1);
  if (is_add(k2)) add(k2, r2);
  if (GELU) {
#pragma unroll
    for (int e = 0; e < V; e++) x[e] = narrow<T>(gelu_approx<sizeof(T) == 2>((float)x[e]) * 1.0f);
  }
  Chunk16 out;
  __builtin_memcpy(&out, x, 16);
  return out;
}

// Stores GROUP pieces a lane holds of one 32-row slab, with the merged operations: all loads
// first, then the arithmetic. lds_piece(it) reads piece `it` from the slab; row_of(it), col_of(it)
// say where it goes in C. COL_FIXED: all of a lane's pieces lie in the same columns and r0, r1, r2
// are the row operands for them (fetched once per kernel); otherwise they are fetched per piece.
// MATRIX: one of the operations has a matrix operand. Loads and stores share one in-order counter:
// code that loads in a loop waits, before it touches the loaded registers again, for everything
// older, stores included. The variants without a matrix operand therefore are instantiations of
// their own in which no such register exists, and their stores are never waited for.
template <typename T, typename Chunk16, bool EDGE, uint32_t GROUP, bool COL_FIXED, bool MATRIX, bool GELU, typename LdsPiece,
          typename RowOf, typename ColOf>
__device__ __forceinline__ void gemm_store_group_merged(const hck_gemm_args& p, const void* p0, const void* p1, const void* p2, Chunk16 r0,
                                                        Chunk16 r1, Chunk16 r2, T* C, uint32_t it0, LdsPiece lds_piece, RowOf row_of,
                                                        ColOf col_of) {
  Chunk16 v[GROUP], m[MATRIX ? GROUP : 1], q0[GROUP], q1[GROUP], q2[GROUP];
#pragma unroll
  for (uint32_t b = 0; b < GROUP; b++) {
    const uint32_t row = row_of(it0 + b), col = col_of(it0 + b);
    const bool inside = !EDGE || (row < p.M && col < p.N);
    v[b] = lds_piece(it0 + b);
    if (MATRIX) m[b] = inside ? gemm_epilogue_matrix_piece<T, Chunk16>(p, p0, p1, p2, row, col) : Chunk16{};
    q0[b] = COL_FIXED ? r0 : gemm_epilogue_row_piece<T, Chunk16>(p.ep_kind[0], p0, col, inside);
    q1[b] = COL_FIXED ? r1 : gemm_epilogue_row_piece<T, Chunk16>(p.ep_kind[1], p1, col, inside);
    q2[b] = COL_FIXED ? r2 : gemm_epilogue_row_piece<T, Chunk16>(p.ep_kind[2], p2, col, inside);
  }
#pragma unroll
  for (uint32_t b = 0; b < GROUP; b++) {
    const uint32_t row = row_of(it0 + b), col = col_of(it0 + b);
    if (!EDGE || (row < p.M && col < p.N))
      *reinterpret_cast<Chunk16*>(C + (size_t)row * p.c_rs + col) =
          gemm_epilogue_apply<T, Chunk16, MATRIX, GELU>(p, v[b], q0[b], q1[b], q2[b], MATRIX ? m[MATRIX ? b : 0] : Chunk16{});
  }
}

// The NIT pieces of a slab in groups of at most MAX_GROUP: a loop that is not unrolled (it reads
// LDS, not the accumulators, and copies of it for every slab would multiply the kernel's code).
template <typename T, typename Chunk16, bool EDGE, uint32_t NIT, bool COL_FIXED, uint32_t MAX_GROUP, bool MATRIX, bool GELU,
          typename LdsPiece, typename RowOf, typename ColOf>
__device__ __forceinline__ void gemm_store_slab_merged_as(const hck_gemm_args& p, const void* p0, const void* p1, const void* p2, Chunk16 r0,
                                                          Chunk16 r1, Chunk16 r2, T* C, LdsPiece lds_piece, RowOf row_of,
                                                          ColOf col_of) {
  constexpr uint32_t GROUP = (MAX_GROUP >= 4 && NIT % 4 == 0) ? 4 : (MAX_GROUP >= 3 && NIT % 3 == 0) ? 3 : (MAX_GROUP >= 2 && NIT % 2 == 0) ? 2 : 1;
  if constexpr (NIT == GROUP) {
    gemm_store_group_merged<T, Chunk16, EDGE, GROUP, COL_FIXED, MATRIX, GELU>(p, p0, p1, p2, r0, r1, r2, C, 0u, lds_piece, row_of, col_of);
  } else {
#pragma nounroll
    for (uint32_t it0 = 0; it0 < NIT; it0 += GROUP)
      gemm_store_group_merged<T, Chunk16, EDGE, GROUP, COL_FIXED, MATRIX, GELU>(p, p0, p1, p2, r0, r1, r2, C, it0, lds_piece, row_of, col_of);
  }
}
