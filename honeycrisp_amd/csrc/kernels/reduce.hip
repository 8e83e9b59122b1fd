// Axis reductions for gfx950: sum / prod / argmax / argmin over the middle axis of an
// [outer, reduce, inner] view, logSoftmax and the fused two-pass normalize.
//
// inner == 1 ("row" kernels): the reduced axis is contiguous. A wave (short rows) or a
// 256-lane block (long rows) owns one row, streams it with 16-byte loads, reduces in
// registers, then across lanes with wave64 shuffles and across waves through LDS.
// inner > 1 ("col" kernels): lanes run along the contiguous inner axis so every step of
// the reduction loop is one coalesced access; 4 waves split the reduce axis and meet
// in LDS.
//
// argmax/argmin return the first extremum exactly as the CPU's strict-compare scan from
// k = 0 does (BackendCPU.swift:848-877): ties go to the smaller index, a NaN at k > 0
// never replaces the running extremum, and a NaN at k = 0 is never replaced.
#include "common.hip.h"
#include "row_teams.hip.h"

#include <math.h>

#include <type_traits>

enum { R_SUM = 0, R_PROD = 1, R_ARGMAX = 2, R_ARGMIN = 3,
       // internal column reductions with float results (logSoftmax over a non-last axis):
       // maximum, sum of expf(x - column maximum), plain sum
       R_MAXF = 4, R_EXPSUMF = 5, R_SUMF = 6 };

template <typename C> struct ArgPair {
  C v;
  uint32_t i;
};

// Ordering key for one element of an arg-reduction: makes the parallel "better value,
// or equal value and smaller index" combine reproduce the sequential scan. For floats a
// NaN at k = 0 becomes the unbeatable extreme and a NaN elsewhere the worst value (it
// can then only tie with element 0 or later ones of larger index, never win).
template <int OP> __device__ __forceinline__ float arg_key(float x, uint32_t k) {
  if (x != x) {
    const float best = OP == R_ARGMAX ? INFINITY : -INFINITY;
    return k == 0 ? best : -best;
  }
  return x;
}
template <int OP> __device__ __forceinline__ int64_t arg_key(int64_t x, uint32_t) { return x; }

template <int OP, typename C>
__device__ __forceinline__ ArgPair<C> arg_better(ArgPair<C> a, ArgPair<C> b) {
  bool take_b = OP == R_ARGMAX ? (b.v > a.v) : (b.v < a.v);
  take_b = take_b || (b.v == a.v && b.i < a.i);
  return take_b ? b : a;
}

// Worst possible value, paired with the largest index, so that any real element wins.
template <int OP> __device__ __forceinline__ void arg_init(ArgPair<float>& p) {
  p.v = OP == R_ARGMAX ? -INFINITY : INFINITY;
  p.i = 0xffffffffu;
}
template <int OP> __device__ __forceinline__ void arg_init(ArgPair<int64_t>& p) {
  p.v = OP == R_ARGMAX ? INT64_MIN : INT64_MAX;
  p.i = 0xffffffffu;
}

template <int OP, typename C> __device__ __forceinline__ C reduce_identity() {
  if (OP == R_MAXF) return (C)-INFINITY;
  return OP == R_PROD ? (C)1 : (C)0;
}
template <int OP, typename C> __device__ __forceinline__ C reduce_combine(C a, C b) {
  if (OP == R_MAXF) return b > a ? b : a;
  return OP == R_PROD ? a * b : a + b;
}

// ---------------------------------------------------------------- rows (inner == 1)

// A row is reduced by a team of LANES lanes: 1 (rows of a few elements: a lane per row, adjacent
// lanes on adjacent rows), 8, 64 (one wave) or 256 (the whole block). SPLIT (LANES = 256): few
// long rows are cut into p.segs segments, one block each, which leave partials.
template <int LANES, int OP, typename C> __device__ __forceinline__ ArgPair<C> team_arg_reduce(ArgPair<C> p) {
#pragma unroll
  for (int o = LANES / 2; o > 0; o >>= 1) {
    ArgPair<C> q;
    q.v = __shfl_xor(p.v, o, 64);
    q.i = __shfl_xor(p.i, o, 64);
    p = arg_better<OP>(p, q);
  }
  return p;
}

// VALUE (arg-reductions, not SPLIT): the output holds the extremum itself, in the input's element
// type, instead of its index: what an arg-reduction followed by a gather of its indices from the
// same input leaves (Tensor.max / min, ReduceRepeat.swift:201-209), in one pass.
template <typename T, int OP, int LANES, bool SPLIT, bool VALUE = false>
__device__ __forceinline__ void reduce_rows_impl(const hck_reduce_args& p) {
  typedef typename Arith<T>::type C;
  constexpr int VEC = VecWidth<T>::value;
  constexpr int ROWS_PER_BLOCK = HCK_BLOCK / LANES;
  static_assert(!SPLIT || LANES == HCK_BLOCK, "segments are reduced by whole blocks");
  const uint32_t lane = threadIdx.x % LANES;
  const uint32_t seg = SPLIT ? blockIdx.x % p.segs : 0;
  const uint32_t row = SPLIT ? blockIdx.x / p.segs : blockIdx.x * ROWS_PER_BLOCK + threadIdx.x / LANES;
  const bool active = row < p.outer;
  const uint32_t n = p.reduce;
  // this team's part of the row: [k0, kend)
  const uint32_t k0 = SPLIT ? seg * p.seg_len : 0;
  const uint32_t kend = SPLIT ? (k0 + p.seg_len < n ? k0 + p.seg_len : n) : n;
  const T* in = (const T*)p.in + (size_t)(active ? row : 0) * n;
  // Rows start 16-byte aligned only when the row length is a multiple of VEC (segments are).
  const bool vec_ok = (n % VEC) == 0;
  __shared__ char lds_raw[sizeof(ArgPair<C>) * (HCK_BLOCK / 64)];

  if (OP == R_SUM || OP == R_PROD) {
    C acc = reduce_identity<OP, C>();
    if (active) {
      if (vec_ok) {
        // four independent 16-byte loads in flight per lane, combined in index order
        constexpr uint32_t STEP = LANES * VEC;
        uint32_t k = k0 + lane * VEC;
        for (; k + 3 * STEP < kend; k += 4 * STEP) {
          T a[4][VEC];
#pragma unroll
          for (int u = 0; u < 4; u++) load_vec<T, VEC>(in, k + u * STEP, 1, a[u]);
#pragma unroll
          for (int u = 0; u < 4; u++)
#pragma unroll
            for (int i = 0; i < VEC; i++) acc = reduce_combine<OP, C>(acc, to_arith(a[u][i]));
        }
        for (; k < kend; k += STEP) {
          T a[VEC];
          load_vec<T, VEC>(in, k, 1, a);
#pragma unroll
          for (int i = 0; i < VEC; i++) acc = reduce_combine<OP, C>(acc, to_arith(a[i]));
        }
      } else {
        for (uint32_t k = k0 + lane; k < kend; k += LANES) acc = reduce_combine<OP, C>(acc, to_arith(in[k]));
      }
    }
    if constexpr (LANES <= 64) {
      acc = OP == R_SUM ? team_reduce<LANES>(acc, SumOp()) : team_reduce<LANES>(acc, ProdOp());
    } else {
      acc = OP == R_SUM ? block_reduce(acc, SumOp(), (C*)lds_raw)
                        : block_reduce(acc, ProdOp(), (C*)lds_raw);
    }
    if (active && lane == 0) {
      if (SPLIT) ((C*)p.pvals)[blockIdx.x] = acc;
      else ((T*)p.out)[row] = from_arith<T>(acc);
    }
  } else {
    ArgPair<C> best;
    arg_init<OP>(best);
    if (active) {
      if (vec_ok) {
        constexpr uint32_t STEP = LANES * VEC;
        uint32_t k = k0 + lane * VEC;
        for (; k + 3 * STEP < kend; k += 4 * STEP) {
          T a[4][VEC];
#pragma unroll
          for (int u = 0; u < 4; u++) load_vec<T, VEC>(in, k + u * STEP, 1, a[u]);
#pragma unroll
          for (int u = 0; u < 4; u++)
#pragma unroll
            for (int i = 0; i < VEC; i++) {
              ArgPair<C> c;
              c.v = arg_key<OP>(to_arith(a[u][i]), k + u * STEP + i);
              c.i = k + u * STEP + i;
              best = arg_better<OP>(best, c);
            }
        }
        for (; k < kend; k += STEP) {
          T a[VEC];
          load_vec<T, VEC>(in, k, 1, a);
#pragma unroll
          for (int i = 0; i < VEC; i++) {
            ArgPair<C> c;
            c.v = arg_key<OP>(to_arith(a[i]), k + i);
            c.i = k + i;
            best = arg_better<OP>(best, c);
          }
        }
      } else {
        for (uint32_t k = k0 + lane; k < kend; k += LANES) {
          ArgPair<C> c;
          c.v = arg_key<OP>(to_arith(in[k]), k);
          c.i = k;
          best = arg_better<OP>(best, c);
        }
      }
    }
    best = team_arg_reduce<(LANES < 64 ? LANES : 64), OP>(best);
    if (LANES > 64) {
      ArgPair<C>* lds = (ArgPair<C>*)lds_raw;
      if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = best;
      __syncthreads();
      best = lds[0];
#pragma unroll
      for (int w = 1; w < HCK_BLOCK / 64; w++) best = arg_better<OP>(best, lds[w]);
    }
    if (active && lane == 0) {
      if (SPLIT) {
        ((C*)p.pvals)[blockIdx.x] = best.v;
        p.pidx[blockIdx.x] = best.i;
      } else if (VALUE) {
        ((T*)p.out)[row] = in[best.i];
      } else {
        ((int64_t*)p.out)[row] = (int64_t)best.i;
      }
    }
  }
}

// ---------------------------------------------------------------- columns (inner > 1)

// Block = up to 64 lanes along inner, VEC consecutive columns per lane (16-byte loads when the row
// pitch allows), x 4 waves along the reduce axis, meeting in LDS. When inner is narrower than a
// wave (jl < 64 lanes cover it), the wave's other lanes take further rows and meet by shuffles. The reduce axis is also
// cut into `splits` ranges handled by different blocks so that a tall, narrow input still
// fills the device; with splits > 1 the ranges leave partials (accumulator type, plus the
// index for arg-reductions) and the same kernel runs a second time with FINAL = true over
// the [outer, splits, inner] partials.
template <typename T, int OP, int VEC, bool FINAL>
__device__ __forceinline__ void reduce_cols_impl(const hck_reduce_cols_args& p) {
  typedef typename Arith<T>::type C;
  typedef typename std::conditional<FINAL, C, T>::type S;  // what this pass reads
  constexpr bool ARG = OP == R_ARGMAX || OP == R_ARGMIN;
  const uint32_t extent = FINAL ? p.splits : p.reduce;     // length of the axis this pass reduces
  const uint32_t splits = FINAL ? 1 : p.splits;
  const uint32_t chunk = FINAL ? p.splits : p.chunk;
  const uint32_t jvecs = (p.inner + VEC - 1) / VEC;
  const uint32_t jl_arg = FINAL ? p.jl_final : p.jl;
  const uint32_t jl = jl_arg ? jl_arg : 64;   // lanes along inner
  const uint32_t rl = 64 / jl;                // rows per wave and step
  const uint32_t jblocks = (jvecs + jl - 1) / jl;
  uint32_t bid = blockIdx.x;
  const uint32_t jb = bid % jblocks;
  bid /= jblocks;
  const uint32_t s = bid % splits;
  const uint32_t i = bid / splits;
  const uint32_t lane = threadIdx.x & 63, kw = threadIdx.x >> 6;
  const uint32_t jlane = lane & (jl - 1), rsub = lane / jl;
  const uint32_t j = (jb * jl + jlane) * VEC;
  const bool active = j < p.inner;
  const uint32_t k_begin = s * chunk;
  const uint32_t k_end = k_begin + chunk < extent ? k_begin + chunk : extent;
  const size_t col0 = (size_t)i * extent * p.inner + (active ? j : 0);
  const S* in = (FINAL ? (const S*)p.pvals : (const S*)p.in) + col0;
  const uint32_t* in_idx = p.pidx + col0;
  __shared__ char lds_raw[sizeof(ArgPair<C>) * HCK_BLOCK * VEC];

  C acc[VEC];
  ArgPair<C> best[VEC];
  float col_aux[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) {
    acc[e] = reduce_identity<OP, C>();
    arg_init<OP>(best[e]);
    col_aux[e] = (OP == R_EXPSUMF && !FINAL && active) ? p.aux[(size_t)i * p.inner + j + e] : 0.0f;
  }
  auto take = [&](const S (&a)[VEC], uint32_t k) {
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      if (ARG) {
        ArgPair<C> c;
        if (FINAL) {  // partials already hold the ordering key and the original index
          c.v = (C)a[e];
          c.i = in_idx[(size_t)k * p.inner + e];
        } else {
          c.v = arg_key<OP>((C)to_arith(a[e]), k);
          c.i = k;
        }
        best[e] = arg_better<OP>(best[e], c);
      } else {
        C x = (C)to_arith(a[e]);
        if (OP == R_EXPSUMF && !FINAL) x = (C)expf((float)x - col_aux[e]);
        acc[e] = reduce_combine<OP, C>(acc[e], x);
      }
    }
  };
  if (active) {
    const uint32_t step = 4 * rl;  // rows the block covers per step
    uint32_t k = k_begin + kw * rl + rsub;
    constexpr int U = 8;  // rows in flight per lane
    for (; k + step * (U - 1) < k_end; k += step * U) {
      S a[U][VEC];
#pragma unroll
      for (int u = 0; u < U; u++) load_vec<S, VEC>(in + (size_t)(k + step * u) * p.inner, 0, 1, a[u]);
#pragma unroll
      for (int u = 0; u < U; u++) take(a[u], k + step * u);
    }
    for (; k < k_end; k += step) {
      S a[VEC];
      load_vec<S, VEC>(in + (size_t)k * p.inner, 0, 1, a);
      take(a, k);
    }
  }
  // the wave's row groups meet in the lanes of group 0 (every lane takes part; idle ones hold
  // the identity / the worst pair)
  for (uint32_t o = jl; o < 64; o <<= 1) {
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      if (ARG) {
        ArgPair<C> q;
        q.v = __shfl_xor(best[e].v, o, 64);
        q.i = __shfl_xor(best[e].i, o, 64);
        best[e] = arg_better<OP>(best[e], q);
      } else {
        acc[e] = reduce_combine<OP, C>(acc[e], __shfl_xor(acc[e], o, 64));
      }
    }
  }
  const bool writer = kw == 0 && rsub == 0 && active;
  const bool last = FINAL || p.splits == 1;  // this pass writes the result itself
  if (ARG) {
    ArgPair<C>* lds = (ArgPair<C>*)lds_raw;
#pragma unroll
    for (int e = 0; e < VEC; e++) lds[threadIdx.x * VEC + e] = best[e];
    __syncthreads();
    if (writer) {
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        for (int w = 1; w < 4; w++) best[e] = arg_better<OP>(best[e], lds[(threadIdx.x + 64 * w) * VEC + e]);
        if (last) {
          ((int64_t*)p.out)[(size_t)i * p.inner + j + e] = (int64_t)best[e].i;
        } else {
          const size_t o = ((size_t)i * p.splits + s) * p.inner + j + e;
          ((C*)p.pvals)[o] = best[e].v;
          p.pidx[o] = best[e].i;
        }
      }
    }
  } else {
    C* lds = (C*)lds_raw;
#pragma unroll
    for (int e = 0; e < VEC; e++) lds[threadIdx.x * VEC + e] = acc[e];
    __syncthreads();
    if (writer) {
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        for (int w = 1; w < 4; w++) acc[e] = reduce_combine<OP, C>(acc[e], lds[(threadIdx.x + 64 * w) * VEC + e]);
        if (last && OP >= R_MAXF) ((float*)p.out)[(size_t)i * p.inner + j + e] = (float)acc[e];
        else if (last) ((T*)p.out)[(size_t)i * p.inner + j + e] = from_arith<T>(acc[e]);
        else ((C*)p.pvals)[((size_t)i * p.splits + s) * p.inner + j + e] = acc[e];
      }
    }
  }
}

#define DEF_REDUCE(NAME, OP, TN, T)                                                                   \
  HC_KERNEL void hc_reduce_rows1_##NAME##_##TN(hck_reduce_args p) { reduce_rows_impl<T, OP, 1, false>(p); } \
  HC_KERNEL void hc_reduce_rows8_##NAME##_##TN(hck_reduce_args p) { reduce_rows_impl<T, OP, 8, false>(p); } \
  HC_KERNEL void hc_reduce_rows64_##NAME##_##TN(hck_reduce_args p) { reduce_rows_impl<T, OP, 64, false>(p); } \
  HC_KERNEL void hc_reduce_rows256_##NAME##_##TN(hck_reduce_args p) { reduce_rows_impl<T, OP, 256, false>(p); } \
  HC_KERNEL void hc_reduce_rowsplit_##NAME##_##TN(hck_reduce_args p) { reduce_rows_impl<T, OP, 256, true>(p); } \
  HC_KERNEL void hc_reduce_cols_##NAME##_##TN##_v1(hck_reduce_cols_args p) {                           \
    reduce_cols_impl<T, OP, 1, false>(p);                                                              \
  }                                                                                                    \
  HC_KERNEL void hc_reduce_cols_##NAME##_##TN##_vN(hck_reduce_cols_args p) {                           \
    reduce_cols_impl<T, OP, VecWidth<T>::value, false>(p);                                             \
  }                                                                                                    \
  HC_KERNEL void hc_reduce_cols_final_##NAME##_##TN(hck_reduce_cols_args p) {                          \
    reduce_cols_impl<T, OP, 1, true>(p);                                                               \
  }
#define DEF_REDUCE_VALUE(NAME, OP, TN, T)                                                             \
  HC_KERNEL void hc_reduce_rows1_##NAME##_value_##TN(hck_reduce_args p) { reduce_rows_impl<T, OP, 1, false, true>(p); } \
  HC_KERNEL void hc_reduce_rows8_##NAME##_value_##TN(hck_reduce_args p) { reduce_rows_impl<T, OP, 8, false, true>(p); } \
  HC_KERNEL void hc_reduce_rows64_##NAME##_value_##TN(hck_reduce_args p) { reduce_rows_impl<T, OP, 64, false, true>(p); } \
  HC_KERNEL void hc_reduce_rows256_##NAME##_value_##TN(hck_reduce_args p) { reduce_rows_impl<T, OP, 256, false, true>(p); }
#define DEF_REDUCE_T(TN, T)                                                                          \
  DEF_REDUCE(sum, R_SUM, TN, T)                                                                      \
  DEF_REDUCE(prod, R_PROD, TN, T)                                                                    \
  DEF_REDUCE(argmax, R_ARGMAX, TN, T)                                                                \
  DEF_REDUCE(argmin, R_ARGMIN, TN, T)                                                                \
  DEF_REDUCE_VALUE(argmax, R_ARGMAX, TN, T)                                                          \
  DEF_REDUCE_VALUE(argmin, R_ARGMIN, TN, T)
DEF_REDUCE_T(f32, float)
DEF_REDUCE_T(f16, half_t)
DEF_REDUCE_T(i64, int64_t)
// bool tensors reduce as Float 0 / 1 (readBuffer(Float.self), BackendCPU.swift:2018-2030): what
// Tensor.all / some issue (argmin / argmax + gather, ReduceRepeat.swift:103-162); a sum or product
// written back as bool is "any" / "all".
DEF_REDUCE_T(b8, uint8_t)

// ---------------------------------------------------------------- row teams

// A row is worked on by a team of LANES lanes: 1 or 8 (short rows, many per wave), one wave
// (4 rows per block) or the whole block.
template <int LANES> struct Team {
  static __device__ __forceinline__ uint32_t lane() { return threadIdx.x % LANES; }
  static __device__ __forceinline__ uint32_t row() {
    return blockIdx.x * (HCK_BLOCK / LANES) + threadIdx.x / LANES;
  }
  // every lane of the team gets the result; `lds` holds >= 4 floats (block teams only)
  template <typename Op> static __device__ __forceinline__ float reduce(float v, Op op, float* lds) {
    if constexpr (LANES <= 64) return team_reduce<LANES>(v, op);
    else return block_reduce(v, op, lds);
  }
};

// Streaming pass over a row that does not fit the registers: f(x, k) for every element, with
// 16-byte loads when the row length allows them.
template <typename T, int LANES, typename F>
__device__ __forceinline__ void stream_row(const T* row, uint32_t n, uint32_t lane, F f) {
  constexpr int VEC = VecWidth<T>::value;
  if (n % VEC == 0) {
    for (uint32_t k = lane * VEC; k < n; k += LANES * VEC) {
      T a[VEC];
      load_vec<T, VEC>(row, k, 1, a);
#pragma unroll
      for (int i = 0; i < VEC; i++) f((float)a[i], k + i);
    }
  } else {
    for (uint32_t k = lane; k < n; k += LANES) f((float)row[k], k);
  }
}
// ... and one that also writes: out[k] = f(x, k).
template <typename T, int LANES, typename F>
__device__ __forceinline__ void stream_row_out(const T* row, T* out, uint32_t n, uint32_t lane, F f) {
  constexpr int VEC = VecWidth<T>::value;
  if (n % VEC == 0) {
    for (uint32_t k = lane * VEC; k < n; k += LANES * VEC) {
      T a[VEC], o[VEC];
      load_vec<T, VEC>(row, k, 1, a);
#pragma unroll
      for (int i = 0; i < VEC; i++) o[i] = narrow<T>(f((float)a[i], k + i));
      store_vec<T, VEC>(out, k, o);
    }
  } else {
    for (uint32_t k = lane; k < n; k += LANES) out[k] = narrow<T>(f((float)row[k], k));
  }
}

// ---------------------------------------------------------------- logSoftmax

// logSoftmax (BackendCPU.swift:1000-1038): max, sum of expf(x - max), x - (logf(sum) + max),
// all in Float. Rows (inner == 1): a wave or a block per row; the row stays in registers when
// it fits, else passes 2 and 3 re-read it (L2).
// NaNs are skipped by the strict compare here and on the CPU alike; any NaN in the row then
// turns the exp-sum, and with it the whole row, into NaN on both.
template <typename T, int LANES> __device__ __forceinline__ void log_softmax_rows_impl(const hck_reduce_args& p) {
  __shared__ float lds[HCK_BLOCK / 64];
  const uint32_t lane = Team<LANES>::lane(), row = Team<LANES>::row();
  if (row >= p.outer) return;  // (never taken by a block team: one row per block)
  const uint32_t n = p.reduce;
  const T* in = (const T*)p.in + (size_t)row * n;
  T* out = (T*)p.out + (size_t)row * n;
  if (RowRegs<T, LANES>::fits(n)) {
    RowRegs<T, LANES> r;
    r.load(in, n, lane);
    float m = -INFINITY;
    r.each(n, lane, [&](float x) { if (x > m) m = x; });
    m = Team<LANES>::reduce(m, MaxOp(), lds);
    float s = 0.0f;
    r.each(n, lane, [&](float x) { s += exp_in<T>(x - m); });
    s = Team<LANES>::reduce(s, SumOp(), lds);
    const float log_sum = logf(s) + m;
    r.store(out, n, lane, [&](float x) { return x - log_sum; });
    return;
  }
  float m = -INFINITY;
  stream_row<T, LANES>(in, n, lane, [&](float x, uint32_t) { if (x > m) m = x; });
  m = Team<LANES>::reduce(m, MaxOp(), lds);
  float s = 0.0f;
  stream_row<T, LANES>(in, n, lane, [&](float x, uint32_t) { s += exp_in<T>(x - m); });
  s = Team<LANES>::reduce(s, SumOp(), lds);
  const float log_sum = logf(s) + m;
  stream_row_out<T, LANES>(in, out, n, lane, [&](float x, uint32_t) { return x - log_sum; });
}

// Columns (inner > 1): per-column maximum and exp-sum come from the split column reductions
// above (R_MAXF, R_EXPSUMF), then one element-wise pass applies them.
template <typename T, int VEC, bool GRAD> __device__ __forceinline__ void softmax_cols_apply_impl(const hck_softmax_cols_args& p) {
  const uint32_t jvecs = (p.inner + VEC - 1) / VEC;
  const uint64_t t = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;
  const uint64_t rows = (uint64_t)p.outer * p.reduce;
  const uint64_t r = t / jvecs;
  if (r >= rows) return;
  const uint32_t j = (uint32_t)(t - r * jvecs) * VEC;
  const uint32_t i = (uint32_t)(r / p.reduce);
  const size_t off = (size_t)r * p.inner + j, col = (size_t)i * p.inner + j;
  T x[VEC], g[VEC], o[VEC];
  load_vec<T, VEC>((const T*)p.in + off, 0, 1, x);
  if (GRAD) load_vec<T, VEC>((const T*)p.grad + off, 0, 1, g);
#pragma unroll
  for (int e = 0; e < VEC; e++) {
    if (j + e < p.inner) {
      const float log_sum = p.col_expsum[col + e];  // (already logf(exp-sum) + maximum, see below)
      if (GRAD) o[e] = narrow<T>((float)g[e] - p.col_gradsum[col + e] * expf((float)x[e] - log_sum));
      else o[e] = narrow<T>((float)x[e] - log_sum);
    }
  }
  store_vec<T, VEC>((T*)p.out, off, o);
}
// exp-sum -> logf(exp-sum) + maximum, once per column and in place (the apply pass would
// otherwise evaluate logf once per element).
HC_KERNEL void hc_log_softmax_cols_logsum(hck_softmax_cols_args p) {
  const uint64_t t = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (t >= (uint64_t)p.outer * p.inner) return;
  float* s = const_cast<float*>(p.col_expsum);
  s[t] = logf(s[t]) + p.col_max[t];
}
#define DEF_SOFTMAX_COLS(TN, T)                                                                        \
  HC_KERNEL void hc_reduce_cols_maxf_##TN##_v1(hck_reduce_cols_args p) { reduce_cols_impl<T, R_MAXF, 1, false>(p); } \
  HC_KERNEL void hc_reduce_cols_maxf_##TN##_vN(hck_reduce_cols_args p) {                               \
    reduce_cols_impl<T, R_MAXF, VecWidth<T>::value, false>(p);                                         \
  }                                                                                                    \
  HC_KERNEL void hc_reduce_cols_final_maxf_##TN(hck_reduce_cols_args p) { reduce_cols_impl<T, R_MAXF, 1, true>(p); } \
  HC_KERNEL void hc_reduce_cols_expsumf_##TN##_v1(hck_reduce_cols_args p) {                            \
    reduce_cols_impl<T, R_EXPSUMF, 1, false>(p);                                                       \
  }                                                                                                    \
  HC_KERNEL void hc_reduce_cols_expsumf_##TN##_vN(hck_reduce_cols_args p) {                            \
    reduce_cols_impl<T, R_EXPSUMF, VecWidth<T>::value, false>(p);                                      \
  }                                                                                                    \
  HC_KERNEL void hc_reduce_cols_final_expsumf_##TN(hck_reduce_cols_args p) {                           \
    reduce_cols_impl<T, R_EXPSUMF, 1, true>(p);                                                        \
  }                                                                                                    \
  HC_KERNEL void hc_reduce_cols_sumf_##TN##_v1(hck_reduce_cols_args p) { reduce_cols_impl<T, R_SUMF, 1, false>(p); } \
  HC_KERNEL void hc_reduce_cols_sumf_##TN##_vN(hck_reduce_cols_args p) {                               \
    reduce_cols_impl<T, R_SUMF, VecWidth<T>::value, false>(p);                                         \
  }                                                                                                    \
  HC_KERNEL void hc_reduce_cols_final_sumf_##TN(hck_reduce_cols_args p) { reduce_cols_impl<T, R_SUMF, 1, true>(p); } \
  HC_KERNEL void hc_log_softmax_cols_apply_##TN##_v1(hck_softmax_cols_args p) {                        \
    softmax_cols_apply_impl<T, 1, false>(p);                                                           \
  }                                                                                                    \
  HC_KERNEL void hc_log_softmax_cols_apply_##TN##_vN(hck_softmax_cols_args p) {                        \
    softmax_cols_apply_impl<T, VecWidth<T>::value, false>(p);                                          \
  }                                                                                                    \
  HC_KERNEL void hc_log_softmax_grad_cols_apply_##TN##_v1(hck_softmax_cols_args p) {                   \
    softmax_cols_apply_impl<T, 1, true>(p);                                                            \
  }                                                                                                    \
  HC_KERNEL void hc_log_softmax_grad_cols_apply_##TN##_vN(hck_softmax_cols_args p) {                   \
    softmax_cols_apply_impl<T, VecWidth<T>::value, true>(p);                                           \
  }
DEF_SOFTMAX_COLS(f32, float)
DEF_SOFTMAX_COLS(f16, half_t)

HC_KERNEL void hc_log_softmax_rows_f32(hck_reduce_args p) { log_softmax_rows_impl<float, 64>(p); }
HC_KERNEL void hc_log_softmax_rows1_f32(hck_reduce_args p) { log_softmax_rows_impl<float, 1>(p); }
HC_KERNEL void hc_log_softmax_rows8_f32(hck_reduce_args p) { log_softmax_rows_impl<float, 8>(p); }
HC_KERNEL void hc_log_softmax_rows_f16(hck_reduce_args p) { log_softmax_rows_impl<half_t, 64>(p); }
HC_KERNEL void hc_log_softmax_rows1_f16(hck_reduce_args p) { log_softmax_rows_impl<half_t, 1>(p); }
HC_KERNEL void hc_log_softmax_rows8_f16(hck_reduce_args p) { log_softmax_rows_impl<half_t, 8>(p); }
HC_KERNEL void hc_log_softmax_rows256_f32(hck_reduce_args p) { log_softmax_rows_impl<float, 256>(p); }
HC_KERNEL void hc_log_softmax_rows256_f16(hck_reduce_args p) { log_softmax_rows_impl<half_t, 256>(p); }

// The chain [x * scale] [+ mask] -> logSoftmax [-> exp] (an attention softmax as a Honeycrisp
// model writes it) in one pass over rows that fit the team's registers: the arithmetic of the
// separate kernels, with every intermediate rounded to T where they would have stored it.
template <typename T, int LANES> __device__ __forceinline__ void softmax_chain_rows_impl(const hck_softmax_chain_args& p) {
  __shared__ float lds[HCK_BLOCK / 64];
  const uint32_t lane = Team<LANES>::lane(), row = Team<LANES>::row();
  if (row >= p.outer) return;
  const uint32_t n = p.reduce;
  constexpr int VEC = RowRegs<T, LANES>::VEC, CHUNKS = RowRegs<T, LANES>::CHUNKS;
  RowRegs<T, LANES> r;
  r.load((const T*)p.in + (size_t)row * n, n, lane);
  if (p.flags & HCK_SM_SCALE) {
    const float s = p.scale;
#pragma unroll
    for (int c = 0; c < CHUNKS; c++)
#pragma unroll
      for (int i = 0; i < VEC; i++) r.v[c][i] = narrow<T>((float)r.v[c][i] * s);
  }
  if (p.flags & HCK_SM_MASK) {
    RowRegs<T, LANES> m;
    m.load((const T*)p.mask + (size_t)(row % p.mask_rows) * n, n, lane);
#pragma unroll
    for (int c = 0; c < CHUNKS; c++)
      if ((lane + LANES * c) * VEC < n) {
#pragma unroll
        for (int i = 0; i < VEC; i++) r.v[c][i] = narrow<T>((float)r.v[c][i] + (float)m.v[c][i]);
      }
  }
  float mx = -INFINITY;
  r.each(n, lane, [&](float x) { if (x > mx) mx = x; });
  mx = Team<LANES>::reduce(mx, MaxOp(), lds);
  float s = 0.0f;
  r.each(n, lane, [&](float x) { s += exp_in<T>(x - mx); });
  s = Team<LANES>::reduce(s, SumOp(), lds);
  const float log_sum = logf(s) + mx;
  const bool then_exp = (p.flags & HCK_SM_EXP) != 0;
  r.store((T*)p.out + (size_t)row * n, n, lane, [&](float x) {
    const float ls = x - log_sum;
    if (!then_exp) return ls;
    // ElemwiseOp.exp on the stored log-probability (fp16: the hardware exponential, as the element-wise kernel)
    const float stored = (float)narrow<T>(ls);
    return (sizeof(T) == 2 ? exp_hw(stored) : expf(stored)) * 1.0f;
  });
}
HC_KERNEL void hc_softmax_chain_rows_f32(hck_softmax_chain_args p) { softmax_chain_rows_impl<float, 64>(p); }
HC_KERNEL void hc_softmax_chain_rows8_f32(hck_softmax_chain_args p) { softmax_chain_rows_impl<float, 8>(p); }
HC_KERNEL void hc_softmax_chain_rows_f16(hck_softmax_chain_args p) { softmax_chain_rows_impl<half_t, 64>(p); }
HC_KERNEL void hc_softmax_chain_rows8_f16(hck_softmax_chain_args p) { softmax_chain_rows_impl<half_t, 8>(p); }

// logSoftmaxGrad (BackendCPU.swift:1040-1085): g - sum(g) * expf(x - (logf(sum exp(x - max)) + max)).
template <typename T, int LANES>
__device__ __forceinline__ void log_softmax_grad_rows_impl(const hck_reduce_args& p) {
  __shared__ float lds[HCK_BLOCK / 64];
  const uint32_t lane = Team<LANES>::lane(), row = Team<LANES>::row();
  if (row >= p.outer) return;
  const uint32_t n = p.reduce;
  const T* in = (const T*)p.in + (size_t)row * n;
  const T* grad = (const T*)p.in2 + (size_t)row * n;
  T* out = (T*)p.out + (size_t)row * n;
  if (RowRegs<T, LANES>::fits(n)) {
    RowRegs<T, LANES> r, g;
    r.load(in, n, lane);
    g.load(grad, n, lane);
    float m = -INFINITY, gs = 0.0f;
    r.each(n, lane, [&](float x) { if (x > m) m = x; });
    g.each(n, lane, [&](float x) { gs += x; });
    m = Team<LANES>::reduce(m, MaxOp(), lds);
    gs = Team<LANES>::reduce(gs, SumOp(), lds);
    float s = 0.0f;
    r.each(n, lane, [&](float x) { s += expf(x - m); });
    s = Team<LANES>::reduce(s, SumOp(), lds);
    const float log_sum = logf(s) + m;
    g.store2(out, n, lane, r, [&](float gv, float x) { return gv - gs * expf(x - log_sum); });
    return;
  }
  float m = -INFINITY, gs = 0.0f;
  stream_row<T, LANES>(in, n, lane, [&](float x, uint32_t) { if (x > m) m = x; });
  stream_row<T, LANES>(grad, n, lane, [&](float x, uint32_t) { gs += x; });
  m = Team<LANES>::reduce(m, MaxOp(), lds);
  gs = Team<LANES>::reduce(gs, SumOp(), lds);
  float s = 0.0f;
  stream_row<T, LANES>(in, n, lane, [&](float x, uint32_t) { s += expf(x - m); });
  s = Team<LANES>::reduce(s, SumOp(), lds);
  const float log_sum = logf(s) + m;
  stream_row_out<T, LANES>(grad, out, n, lane,
                           [&](float gv, uint32_t k) { return gv - gs * expf((float)in[k] - log_sum); });
}

HC_KERNEL void hc_log_softmax_grad_rows_f32(hck_reduce_args p) { log_softmax_grad_rows_impl<float, 64>(p); }
HC_KERNEL void hc_log_softmax_grad_rows1_f32(hck_reduce_args p) { log_softmax_grad_rows_impl<float, 1>(p); }
HC_KERNEL void hc_log_softmax_grad_rows8_f32(hck_reduce_args p) { log_softmax_grad_rows_impl<float, 8>(p); }
HC_KERNEL void hc_log_softmax_grad_rows_f16(hck_reduce_args p) { log_softmax_grad_rows_impl<half_t, 64>(p); }
HC_KERNEL void hc_log_softmax_grad_rows1_f16(hck_reduce_args p) { log_softmax_grad_rows_impl<half_t, 1>(p); }
HC_KERNEL void hc_log_softmax_grad_rows8_f16(hck_reduce_args p) { log_softmax_grad_rows_impl<half_t, 8>(p); }
HC_KERNEL void hc_log_softmax_grad_rows256_f32(hck_reduce_args p) { log_softmax_grad_rows_impl<float, 256>(p); }
HC_KERNEL void hc_log_softmax_grad_rows256_f16(hck_reduce_args p) { log_softmax_grad_rows_impl<half_t, 256>(p); }

// ---------------------------------------------------------------- normalize

// normalize for inner == 1, fused: the base-class composition (Backend.swift:265-327)
//   mean = sum(x) * (1/n); c = x - mean; var = sum(c^2) * (1/n);
//   out = c * (var + eps)^-0.5
// with every intermediate rounded to the tensor dtype where the composed backend calls
// would have stored it. c^2 is x*x for fp32 (pow special case) and powf(x, 2) for fp16
// (generic path), as on the CPU.
template <typename T, int LANES> __device__ __forceinline__ void normalize_rows_impl(const hck_reduce_args& p) {
  __shared__ float lds[HCK_BLOCK / 64];
  const uint32_t lane = Team<LANES>::lane(), row = Team<LANES>::row();
  if (row >= p.outer) return;
  const uint32_t n = p.reduce;
  const T* in = (const T*)p.in + (size_t)row * n;
  T* out = (T*)p.out + (size_t)row * n;
  const float inv_n = 1.0f / (float)n;
  auto square = [](float c) { return round_through<T>(sizeof(T) == 4 ? c * c : 1.0f * 1.0f * pow_like(c, 2.0f)); };
  if (RowRegs<T, LANES>::fits(n)) {
    RowRegs<T, LANES> r;
    r.load(in, n, lane);
    float s = 0.0f;
    r.each(n, lane, [&](float x) { s += x; });
    s = round_through<T>(Team<LANES>::reduce(s, SumOp(), lds));
    const float mean = round_through<T>(s * inv_n);
    float sq = 0.0f;
    r.each(n, lane, [&](float x) { sq += square(round_through<T>(x - mean)); });
    sq = round_through<T>(Team<LANES>::reduce(sq, SumOp(), lds));
    const float var = round_through<T>(sq * inv_n);
    const float shifted = round_through<T>(var + p.eps);
    const float normer = round_through<T>(1.0f * 1.0f * pow_like(shifted, -0.5f));
    r.store(out, n, lane, [&](float x) { return round_through<T>(x - mean) * normer; });
    return;
  }
  float s = 0.0f;
  stream_row<T, LANES>(in, n, lane, [&](float x, uint32_t) { s += x; });
  s = round_through<T>(Team<LANES>::reduce(s, SumOp(), lds));
  const float mean = round_through<T>(s * inv_n);
  float sq = 0.0f;
  stream_row<T, LANES>(in, n, lane, [&](float x, uint32_t) { sq += square(round_through<T>(x - mean)); });
  sq = round_through<T>(Team<LANES>::reduce(sq, SumOp(), lds));
  const float var = round_through<T>(sq * inv_n);
  const float shifted = round_through<T>(var + p.eps);
  const float normer = round_through<T>(1.0f * 1.0f * pow_like(shifted, -0.5f));
  stream_row_out<T, LANES>(in, out, n, lane, [&](float x, uint32_t) { return round_through<T>(x - mean) * normer; });
}
HC_KERNEL void hc_normalize_rows_f32(hck_reduce_args p) { normalize_rows_impl<float, 64>(p); }
HC_KERNEL void hc_normalize_rows1_f32(hck_reduce_args p) { normalize_rows_impl<float, 1>(p); }
HC_KERNEL void hc_normalize_rows8_f32(hck_reduce_args p) { normalize_rows_impl<float, 8>(p); }
HC_KERNEL void hc_normalize_rows_f16(hck_reduce_args p) { normalize_rows_impl<half_t, 64>(p); }
HC_KERNEL void hc_normalize_rows1_f16(hck_reduce_args p) { normalize_rows_impl<half_t, 1>(p); }
HC_KERNEL void hc_normalize_rows8_f16(hck_reduce_args p) { normalize_rows_impl<half_t, 8>(p); }
HC_KERNEL void hc_normalize_rows256_f32(hck_reduce_args p) { normalize_rows_impl<float, 256>(p); }
HC_KERNEL void hc_normalize_rows256_f16(hck_reduce_args p) { normalize_rows_impl<half_t, 256>(p); }

// The chain [cast to fp32] -> normalize (fp32, a wave per row) [-> x * (gain [+ c]) + bias] [-> cast]
// (a LayerNorm as Trainable.swift:787-829 issues it) in one pass. Elements are spread over the
// lanes as the fp32 normalize kernel spreads them (lane l: the 4-element groups l, l + 64, ...) and
// summed in its order, so the row statistics have the same bits; the affine part is mulAdd's
// x * c + b and the scalar kernel's gain + c.
template <typename TI, typename TO> __device__ __forceinline__ void layernorm_rows_impl(const hck_layernorm_args& p) {
  constexpr int VEC = 4, CHUNKS = 4, LANES = 64;
  const uint32_t lane = Team<LANES>::lane(), row = Team<LANES>::row();
  if (row >= p.outer) return;
  const uint32_t n = p.reduce;
  const TI* in = (const TI*)p.in + (size_t)row * n;
  TO* out = (TO*)p.out + (size_t)row * n;
  float v[CHUNKS][VEC];
#pragma unroll
  for (int c = 0; c < CHUNKS; c++) {
    const uint32_t k = (lane + LANES * c) * VEC;
    if (k < n) {
      TI a[VEC];
      load_vec<TI, VEC>(in, k, 1, a);
#pragma unroll
      for (int i = 0; i < VEC; i++) v[c][i] = (float)a[i];
    }
  }
  auto each = [&](auto f) {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++)
      if ((lane + LANES * c) * VEC < n) {
#pragma unroll
        for (int i = 0; i < VEC; i++) f(v[c][i]);
      }
  };
  // the row operands of the affine part: fetched now, used after the two reductions
  const bool affine = (p.flags & HCK_LN_AFFINE) != 0, gain_add = (p.flags & HCK_LN_GAIN_ADD) != 0;
  float g[CHUNKS][VEC], b[CHUNKS][VEC];
  if (affine) {
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
      const uint32_t k = (lane + LANES * c) * VEC;
      if (k < n) {
        load_vec<float, VEC>((const float*)p.gain, k, 1, g[c]);
        load_vec<float, VEC>((const float*)p.bias, k, 1, b[c]);
      }
    }
  }
  const float inv_n = 1.0f / (float)n;
  float s = 0.0f;
  each([&](float x) { s += x; });
  s = Team<LANES>::reduce(s, SumOp(), nullptr);
  const float mean = s * inv_n;
  float sq = 0.0f;
  each([&](float x) {
    const float d = x - mean;
    sq += d * d;
  });
  sq = Team<LANES>::reduce(sq, SumOp(), nullptr);
  const float var = sq * inv_n;
  const float shifted = var + p.eps;
  const float normer = 1.0f * 1.0f * pow_like(shifted, -0.5f);
#pragma unroll
  for (int c = 0; c < CHUNKS; c++) {
    const uint32_t k = (lane + LANES * c) * VEC;
    if (k < n) {
      TO o[VEC];
#pragma unroll
      for (int i = 0; i < VEC; i++) {
        float y = (v[c][i] - mean) * normer;
        if (affine) {
          const float coeff = gain_add ? g[c][i] + p.gain_add : g[c][i];
          y = y * coeff + b[c][i];
        }
        o[i] = narrow<TO>(y);
      }
      store_vec<TO, VEC>(out, k, o);
    }
  }
}
HC_KERNEL void hc_layernorm_rows_f32_f32(hck_layernorm_args p) { layernorm_rows_impl<float, float>(p); }
HC_KERNEL void hc_layernorm_rows_f16_f32(hck_layernorm_args p) { layernorm_rows_impl<half_t, float>(p); }
HC_KERNEL void hc_layernorm_rows_f32_f16(hck_layernorm_args p) { layernorm_rows_impl<float, half_t>(p); }
HC_KERNEL void hc_layernorm_rows_f16_f16(hck_layernorm_args p) { layernorm_rows_impl<half_t, half_t>(p); }
