// Bandwidth-bound element-wise kernels for gfx950: broadcasting binary ops, compare,
// tensor-scalar ops, mulAdd/addMul, when, broadcast copy, unary maps, pow, cast, fill.
//
// All of them are pure streaming kernels: one 16-byte vector per lane per access,
// consecutive lanes on consecutive vectors (fully coalesced 1 KiB per wave), index
// arithmetic once per vector rather than once per element. Arithmetic follows the CPU
// backend: float dtypes compute in fp32 and round once on store, int64 stays int64.
// Built with -ffp-contract=off so a*b+c is two roundings, as in the reference.
#include "common.hip.h"

// ---------------------------------------------------------------- scalar semantics

// Python-style modulus (TensorElement.swift:124-132).
__device__ __forceinline__ float mod_pos_f(float l, float r) {
  return l < 0 ? fmodf(r - fmodf(r - l, r), r) : fmodf(l, r);
}
__device__ __forceinline__ float modulus(float l, float r) {
  return r < 0 ? -mod_pos_f(-l, -r) : mod_pos_f(l, r);
}
// (TensorElement.swift:214-222)
__device__ __forceinline__ int64_t mod_pos_i(int64_t l, int64_t r) {
  return l < 0 ? (r - ((r - l) % r)) % r : l % r;
}
__device__ __forceinline__ int64_t modulus(int64_t l, int64_t r) {
  return r < 0 ? -mod_pos_i(-l, -r) : mod_pos_i(l, r);
}

enum { OP_ADD = 0, OP_MUL = 1, OP_SUB = 2, OP_DIV = 3, OP_MOD = 4 };

// NumericBinaryOp.apply (BinaryOps.swift:9-22).
template <int OP, typename C> __device__ __forceinline__ C binop(C a, C b) {
  if (OP == OP_ADD) return a + b;
  if (OP == OP_MUL) return a * b;
  if (OP == OP_SUB) return a - b;
  if (OP == OP_DIV) return a / b;
  return modulus(a, b);
}

enum { CMP_EQ = 0, CMP_NE, CMP_LT, CMP_LE, CMP_GT, CMP_GE };

// ComparisonOp.apply (Comparison.swift:12-27).
template <int OP, typename C> __device__ __forceinline__ bool cmpop(C a, C b) {
  if (OP == CMP_EQ) return a == b;
  if (OP == CMP_NE) return a != b;
  if (OP == CMP_LT) return a < b;
  if (OP == CMP_LE) return a <= b;
  if (OP == CMP_GT) return a > b;
  return a >= b;
}

// ---------------------------------------------------------------- broadcasting binary

// binaryOp(BroadcastData, BroadcastData) (BackendCPU.swift:267-314).
template <typename T, int OP, int VEC> __device__ __forceinline__ void binary_impl(const hck_binary_args& p) {
  typedef typename Arith<T>::type C;
  uint32_t v = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v >= p.d.total_vecs) return;
  uint32_t off[2];
  size_t o;
  bcast_offsets<2, VEC>(p.d, v, off, o);
  with_strides2<VEC>(p.d.inner_stride, [&](auto sa, auto sb) {
    T a[VEC], b[VEC], r[VEC];
    load_vec_c<T, VEC, decltype(sa)::value>((const T*)p.a, off[0], p.d.inner_stride[0], a);
    load_vec_c<T, VEC, decltype(sb)::value>((const T*)p.b, off[1], p.d.inner_stride[1], b);
    __builtin_amdgcn_sched_barrier(0);  // every load is issued before the first use of one
#pragma unroll
    for (int i = 0; i < VEC; i++) r[i] = from_arith<T>(binop<OP, C>(to_arith(a[i]), to_arith(b[i])));
    store_vec<T, VEC>((T*)p.out, o, r);
  });
}

// compare(BroadcastData, BroadcastData) (BackendCPU.swift:541-571): bool output.
template <typename T, int OP, int VEC> __device__ __forceinline__ void compare_impl(const hck_binary_args& p) {
  uint32_t v = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v >= p.d.total_vecs) return;
  uint32_t off[2];
  size_t o;
  bcast_offsets<2, VEC>(p.d, v, off, o);
  with_strides2<VEC>(p.d.inner_stride, [&](auto sa, auto sb) {
    T a[VEC], b[VEC];
    uint8_t r[VEC];
    load_vec_c<T, VEC, decltype(sa)::value>((const T*)p.a, off[0], p.d.inner_stride[0], a);
    load_vec_c<T, VEC, decltype(sb)::value>((const T*)p.b, off[1], p.d.inner_stride[1], b);
    __builtin_amdgcn_sched_barrier(0);  // every load is issued before the first use of one
#pragma unroll
    for (int i = 0; i < VEC; i++) r[i] = cmpop<OP>(to_arith(a[i]), to_arith(b[i])) ? 1 : 0;
    store_vec<uint8_t, VEC>((uint8_t*)p.out, o, r);
  });
}

// broadcast (BackendCPU.swift:255-265): raw element copy, keyed by element size.
template <typename T, int VEC> __device__ __forceinline__ void bcast_copy_impl(const hck_binary_args& p) {
  uint32_t v = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v >= p.d.total_vecs) return;
  uint32_t off[1];
  size_t o;
  bcast_offsets<1, VEC>(p.d, v, off, o);
  T a[VEC];
  load_vec<T, VEC>((const T*)p.a, off[0], p.d.inner_stride[0], a);
  store_vec<T, VEC>((T*)p.out, o, a);
}

// mulAdd / addMul (BackendCPU.swift:445-539): x*c + b and (x + b)*c.
template <typename T, int MULADD, int VEC> __device__ __forceinline__ void fused3_impl(const hck_ternary_args& p) {
  typedef typename Arith<T>::type C;
  uint32_t v = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v >= p.d.total_vecs) return;
  uint32_t off[3];
  size_t o;
  bcast_offsets<3, VEC>(p.d, v, off, o);
  with_strides_all<VEC, 3>(p.d.inner_stride, [&](auto sc) {
    constexpr int S = decltype(sc)::value;
    T x[VEC], c[VEC], b[VEC], r[VEC];
    load_vec_c<T, VEC, S>((const T*)p.x, off[0], p.d.inner_stride[0], x);
    load_vec_c<T, VEC, S>((const T*)p.y, off[1], p.d.inner_stride[1], c);
    load_vec_c<T, VEC, S>((const T*)p.z, off[2], p.d.inner_stride[2], b);
    __builtin_amdgcn_sched_barrier(0);  // every load is issued before the first use of one
#pragma unroll
    for (int i = 0; i < VEC; i++) {
      C xv = to_arith(x[i]), cv = to_arith(c[i]), bv = to_arith(b[i]);
      r[i] = from_arith<T>(MULADD ? xv * cv + bv : (xv + bv) * cv);
    }
    store_vec<T, VEC>((T*)p.out, o, r);
  });
}

// when (BackendCPU.swift:1190-1220): x = bool mask, y/z = branches; raw element copy.
template <typename T, int VEC> __device__ __forceinline__ void when_impl(const hck_ternary_args& p) {
  uint32_t v = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v >= p.d.total_vecs) return;
  uint32_t off[3];
  size_t o;
  bcast_offsets<3, VEC>(p.d, v, off, o);
  with_strides_all<VEC, 3>(p.d.inner_stride, [&](auto sc) {
    constexpr int S = decltype(sc)::value;
    uint8_t m[VEC];
    T a[VEC], b[VEC], r[VEC];
    load_vec_c<uint8_t, VEC, S>((const uint8_t*)p.x, off[0], p.d.inner_stride[0], m);
    load_vec_c<T, VEC, S>((const T*)p.y, off[1], p.d.inner_stride[1], a);
    load_vec_c<T, VEC, S>((const T*)p.z, off[2], p.d.inner_stride[2], b);
    __builtin_amdgcn_sched_barrier(0);  // every load is issued before the first use of one
#pragma unroll
    for (int i = 0; i < VEC; i++) r[i] = m[i] != 0 ? a[i] : b[i];
    store_vec<T, VEC>((T*)p.out, o, r);
  });
}

// bitwiseOp (BackendCPU.swift:407-443): or / and / xor on the raw bits, any dtype, keyed by
// element size; the scalar form repeats an element-sized bit pattern.
enum { BIT_OR = 0, BIT_AND = 1, BIT_XOR = 2 };
template <int OP, typename U> __device__ __forceinline__ U bitop(U a, U b) {
  return OP == BIT_OR ? (U)(a | b) : OP == BIT_AND ? (U)(a & b) : (U)(a ^ b);
}
template <typename U, int OP, int VEC> __device__ __forceinline__ void bitwise_impl(const hck_binary_args& p) {
  uint32_t v = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v >= p.d.total_vecs) return;
  uint32_t off[2];
  size_t o;
  bcast_offsets<2, VEC>(p.d, v, off, o);
  with_strides2<VEC>(p.d.inner_stride, [&](auto sa, auto sb) {
    U a[VEC], b[VEC], r[VEC];
    load_vec_c<U, VEC, decltype(sa)::value>((const U*)p.a, off[0], p.d.inner_stride[0], a);
    load_vec_c<U, VEC, decltype(sb)::value>((const U*)p.b, off[1], p.d.inner_stride[1], b);
    __builtin_amdgcn_sched_barrier(0);  // every load is issued before the first use of one
#pragma unroll
    for (int i = 0; i < VEC; i++) r[i] = bitop<OP>(a[i], b[i]);
    store_vec<U, VEC>((U*)p.out, o, r);
  });
}
#define DEF_BITWISE(BN, U, V)                                                                         \
  HC_KERNEL void hc_bitwise_or_##BN##_v##V(hck_binary_args p) { bitwise_impl<U, BIT_OR, V>(p); }      \
  HC_KERNEL void hc_bitwise_and_##BN##_v##V(hck_binary_args p) { bitwise_impl<U, BIT_AND, V>(p); }    \
  HC_KERNEL void hc_bitwise_xor_##BN##_v##V(hck_binary_args p) { bitwise_impl<U, BIT_XOR, V>(p); }
DEF_BITWISE(b1, uint8_t, 1)
DEF_BITWISE(b1, uint8_t, 16)
DEF_BITWISE(b2, uint16_t, 1)
DEF_BITWISE(b2, uint16_t, 8)
DEF_BITWISE(b4, uint32_t, 1)
DEF_BITWISE(b4, uint32_t, 4)
DEF_BITWISE(b8, uint64_t, 1)
DEF_BITWISE(b8, uint64_t, 2)

// clamp (BackendCPU.swift:704-782): Swift.min(hi, Swift.max(lo, x)) on Float / Int64, where
// max(a, b) = b >= a ? b : a and min(a, b) = b < a ? b : a. MODE 0 both bounds, 1 lower
// only, 2 upper only (the unused operand aliases x).
template <typename T, int MODE, int VEC> __device__ __forceinline__ void clamp_impl(const hck_ternary_args& p) {
  typedef typename Arith<T>::type C;
  uint32_t v = blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v >= p.d.total_vecs) return;
  uint32_t off[3];
  size_t o;
  bcast_offsets<3, VEC>(p.d, v, off, o);
  T x[VEC], lo[VEC], hi[VEC], r[VEC];
  load_vec<T, VEC>((const T*)p.x, off[0], p.d.inner_stride[0], x);
  load_vec<T, VEC>((const T*)p.y, off[1], p.d.inner_stride[1], lo);
  load_vec<T, VEC>((const T*)p.z, off[2], p.d.inner_stride[2], hi);
#pragma unroll
  for (int i = 0; i < VEC; i++) {
    C val = to_arith(x[i]);
    if (MODE != 2) {
      const C l = to_arith(lo[i]);
      val = val >= l ? val : l;
    }
    if (MODE != 1) {
      const C h = to_arith(hi[i]);
      val = val < h ? val : h;
    }
    r[i] = from_arith<T>(val);
  }
  store_vec<T, VEC>((T*)p.out, o, r);
}

#define DEF_BINARY_OPS(TN, T, V)                                                                      \
  HC_KERNEL void hc_binary_add_##TN##_v##V(hck_binary_args p) { binary_impl<T, OP_ADD, V>(p); }      \
  HC_KERNEL void hc_binary_mul_##TN##_v##V(hck_binary_args p) { binary_impl<T, OP_MUL, V>(p); }      \
  HC_KERNEL void hc_binary_sub_##TN##_v##V(hck_binary_args p) { binary_impl<T, OP_SUB, V>(p); }      \
  HC_KERNEL void hc_binary_div_##TN##_v##V(hck_binary_args p) { binary_impl<T, OP_DIV, V>(p); }      \
  HC_KERNEL void hc_binary_mod_##TN##_v##V(hck_binary_args p) { binary_impl<T, OP_MOD, V>(p); }      \
  HC_KERNEL void hc_compare_eq_##TN##_v##V(hck_binary_args p) { compare_impl<T, CMP_EQ, V>(p); }     \
  HC_KERNEL void hc_compare_ne_##TN##_v##V(hck_binary_args p) { compare_impl<T, CMP_NE, V>(p); }     \
  HC_KERNEL void hc_compare_lt_##TN##_v##V(hck_binary_args p) { compare_impl<T, CMP_LT, V>(p); }     \
  HC_KERNEL void hc_compare_le_##TN##_v##V(hck_binary_args p) { compare_impl<T, CMP_LE, V>(p); }     \
  HC_KERNEL void hc_compare_gt_##TN##_v##V(hck_binary_args p) { compare_impl<T, CMP_GT, V>(p); }     \
  HC_KERNEL void hc_compare_ge_##TN##_v##V(hck_binary_args p) { compare_impl<T, CMP_GE, V>(p); }     \
  HC_KERNEL void hc_mul_add_##TN##_v##V(hck_ternary_args p) { fused3_impl<T, 1, V>(p); }             \
  HC_KERNEL void hc_add_mul_##TN##_v##V(hck_ternary_args p) { fused3_impl<T, 0, V>(p); }             \
  HC_KERNEL void hc_clamp_both_##TN##_v##V(hck_ternary_args p) { clamp_impl<T, 0, V>(p); }           \
  HC_KERNEL void hc_clamp_min_##TN##_v##V(hck_ternary_args p) { clamp_impl<T, 1, V>(p); }            \
  HC_KERNEL void hc_clamp_max_##TN##_v##V(hck_ternary_args p) { clamp_impl<T, 2, V>(p); }

DEF_BINARY_OPS(f32, float, 1)
DEF_BINARY_OPS(f32, float, 4)
DEF_BINARY_OPS(f16, half_t, 1)
DEF_BINARY_OPS(f16, half_t, 8)
DEF_BINARY_OPS(i64, int64_t, 1)
DEF_BINARY_OPS(i64, int64_t, 2)

// compare on bool inputs goes through Float in the reference (BackendCPU.swift:566-570).
#define DEF_COMPARE_BOOL(V)                                                                          \
  HC_KERNEL void hc_compare_eq_b8_v##V(hck_binary_args p) { compare_impl<uint8_t, CMP_EQ, V>(p); }   \
  HC_KERNEL void hc_compare_ne_b8_v##V(hck_binary_args p) { compare_impl<uint8_t, CMP_NE, V>(p); }   \
  HC_KERNEL void hc_compare_lt_b8_v##V(hck_binary_args p) { compare_impl<uint8_t, CMP_LT, V>(p); }   \
  HC_KERNEL void hc_compare_le_b8_v##V(hck_binary_args p) { compare_impl<uint8_t, CMP_LE, V>(p); }   \
  HC_KERNEL void hc_compare_gt_b8_v##V(hck_binary_args p) { compare_impl<uint8_t, CMP_GT, V>(p); }   \
  HC_KERNEL void hc_compare_ge_b8_v##V(hck_binary_args p) { compare_impl<uint8_t, CMP_GE, V>(p); }
DEF_COMPARE_BOOL(1)
DEF_COMPARE_BOOL(16)

// Element-size keyed copies (b1/b2/b4/b8 = bytes per element).
#define DEF_COPY(BN, T, V)                                                                           \
  HC_KERNEL void hc_broadcast_##BN##_v##V(hck_binary_args p) { bcast_copy_impl<T, V>(p); }           \
  HC_KERNEL void hc_when_##BN##_v##V(hck_ternary_args p) { when_impl<T, V>(p); }
DEF_COPY(b1, uint8_t, 1)
DEF_COPY(b1, uint8_t, 16)
DEF_COPY(b2, uint16_t, 1)
DEF_COPY(b2, uint16_t, 8)
DEF_COPY(b4, uint32_t, 1)
DEF_COPY(b4, uint32_t, 4)
DEF_COPY(b8, uint64_t, 1)
DEF_COPY(b8, uint64_t, 2)

// ---------------------------------------------------------------- contiguous maps

// Apply f to `count` contiguous elements: 16-byte vectors, the ragged tail by scalar
// accesses from the first lanes of block 0.
template <typename TI, typename TO, typename F>
__device__ __forceinline__ void map_contiguous(const TI* in, TO* out, uint64_t count, F f) {
  constexpr int VEC = VecWidth<TI>::value < VecWidth<TO>::value ? VecWidth<TI>::value : VecWidth<TO>::value;
  const uint64_t nvec = count / VEC;
  const uint64_t v = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v < nvec) {
    TI a[VEC];
    TO r[VEC];
    load_vec<TI, VEC>(in + v * VEC, 0, 1, a);
#pragma unroll
    for (int i = 0; i < VEC; i++) r[i] = f(a[i], v * VEC + i);
    store_vec<TO, VEC>(out, v * VEC, r);
  }
  if (v < count - nvec * VEC) {
    const uint64_t i = nvec * VEC + v;
    out[i] = f(in[i], i);
  }
}

// binaryOp(Tensor.Data, T) / (T, Tensor.Data) (BackendCPU.swift:316-405). The host maps
// the fp32 forms onto these: x / s -> MUL with 1/s, x - s -> ADD with -s; s - x uses
// RSUB = x * -1 + s (vDSP_vsmsa); s / x uses RDIV.
enum { SOP_ADD = 0, SOP_MUL, SOP_SUB, SOP_DIV, SOP_MOD, SOP_RSUB_F32, SOP_RSUB, SOP_RDIV, SOP_RMOD };

template <typename T, int SOP> __device__ __forceinline__ void scalar_impl(const hck_scalar_args& p) {
  typedef typename Arith<T>::type C;
  const C s = sizeof(C) == 8 ? (C)p.si : (C)p.sf;
  map_contiguous((const T*)p.in, (T*)p.out, p.count, [s](T xv, uint64_t) {
    C x = to_arith(xv);
    C r;
    if (SOP == SOP_ADD) r = x + s;
    else if (SOP == SOP_MUL) r = x * s;
    else if (SOP == SOP_SUB) r = x - s;
    else if (SOP == SOP_DIV) r = x / s;
    else if (SOP == SOP_MOD) r = modulus(x, s);
    else if (SOP == SOP_RSUB_F32) r = x * (C)-1 + s;
    else if (SOP == SOP_RSUB) r = s - x;
    else if (SOP == SOP_RDIV) r = s / x;
    else r = modulus(s, x);
    return from_arith<T>(r);
  });
}

#define DEF_SCALAR(TN, T)                                                                            \
  HC_KERNEL void hc_scalar_add_##TN(hck_scalar_args p) { scalar_impl<T, SOP_ADD>(p); }               \
  HC_KERNEL void hc_scalar_mul_##TN(hck_scalar_args p) { scalar_impl<T, SOP_MUL>(p); }               \
  HC_KERNEL void hc_scalar_sub_##TN(hck_scalar_args p) { scalar_impl<T, SOP_SUB>(p); }               \
  HC_KERNEL void hc_scalar_div_##TN(hck_scalar_args p) { scalar_impl<T, SOP_DIV>(p); }               \
  HC_KERNEL void hc_scalar_mod_##TN(hck_scalar_args p) { scalar_impl<T, SOP_MOD>(p); }               \
  HC_KERNEL void hc_scalar_rsubf_##TN(hck_scalar_args p) { scalar_impl<T, SOP_RSUB_F32>(p); }        \
  HC_KERNEL void hc_scalar_rsub_##TN(hck_scalar_args p) { scalar_impl<T, SOP_RSUB>(p); }             \
  HC_KERNEL void hc_scalar_rdiv_##TN(hck_scalar_args p) { scalar_impl<T, SOP_RDIV>(p); }             \
  HC_KERNEL void hc_scalar_rmod_##TN(hck_scalar_args p) { scalar_impl<T, SOP_RMOD>(p); }
DEF_SCALAR(f32, float)
DEF_SCALAR(f16, half_t)
DEF_SCALAR(i64, int64_t)

// compare(Tensor.Data, T) / (T, Tensor.Data) (BackendCPU.swift:573-624).
template <typename T, int OP, int FIRST> __device__ __forceinline__ void cmp_scalar_impl(const hck_scalar_args& p) {
  typedef typename Arith<T>::type C;
  const C s = sizeof(C) == 8 ? (C)p.si : (C)p.sf;
  map_contiguous((const T*)p.in, (uint8_t*)p.out, p.count, [s](T xv, uint64_t) {
    C x = to_arith(xv);
    return (uint8_t)((FIRST ? cmpop<OP>(s, x) : cmpop<OP>(x, s)) ? 1 : 0);
  });
}
#define DEF_CMP_SCALAR1(TN, T, ON, OP)                                                               \
  HC_KERNEL void hc_cmps_##ON##_##TN(hck_scalar_args p) { cmp_scalar_impl<T, OP, 0>(p); }            \
  HC_KERNEL void hc_cmps_r##ON##_##TN(hck_scalar_args p) { cmp_scalar_impl<T, OP, 1>(p); }
#define DEF_CMP_SCALAR(TN, T)                                                                        \
  DEF_CMP_SCALAR1(TN, T, eq, CMP_EQ)                                                                 \
  DEF_CMP_SCALAR1(TN, T, ne, CMP_NE)                                                                 \
  DEF_CMP_SCALAR1(TN, T, lt, CMP_LT)                                                                 \
  DEF_CMP_SCALAR1(TN, T, le, CMP_LE)                                                                 \
  DEF_CMP_SCALAR1(TN, T, gt, CMP_GT)                                                                 \
  DEF_CMP_SCALAR1(TN, T, ge, CMP_GE)
DEF_CMP_SCALAR(f32, float)
DEF_CMP_SCALAR(f16, half_t)
DEF_CMP_SCALAR(i64, int64_t)
DEF_CMP_SCALAR(b8, uint8_t)

// ---------------------------------------------------------------- unary (elemwise)

#include "elemwise_formulas.hip.h"

__device__ __forceinline__ float fast_erf(float a) {
  float r, s, t, u;
  t = fabsf(a);
  s = a * a;
  if (t > 0.927734375f) {
    r = -1.72853470e-5f * t + 3.83197126e-4f;
    u = -3.88396438e-3f * t + 2.42546219e-2f;
    r = r * s + u;
    r = r * t + -1.06777877e-1f;
    r = r * t + -6.34846687e-1f;
    r = r * t + -1.28717512e-1f;
    r = r * t + -t;
    r = 1.0f - expf(r);
    r = copysignf(r, a);
  } else {
    r = -5.96761703e-4f;
    r = r * s + 4.99119423e-3f;
    r = r * s + -2.67681349e-2f;
    r = r * s + 1.12819925e-1f;
    r = r * s + -3.76125336e-1f;
    r = r * s + 1.28379166e-1f;
    r = r * a + a;
  }
  return r;
}
__device__ __forceinline__ float simple_erf_grad(float f) {
  return fabsf(f) > 20.0f ? 0.0f : 1.1283791670955126f * expf(-f * f);
}

enum {
  E_SIN = 0, E_COS, E_MINUS_SIN, E_TAN, E_TAN_GRAD, E_ATAN, E_ATAN_GRAD, E_ACOS, E_ACOS_GRAD,
  E_ASIN, E_ASIN_GRAD, E_EXP, E_LOG, E_RECIP, E_SIGMOID, E_SIGMOID_GRAD, E_RELU, E_RELU_GRAD,
  E_ABS, E_ABS_GRAD, E_GELU_APPROX, E_GELU_APPROX_GRAD, E_GELU_EXACT, E_GELU_EXACT_GRAD, E_ERF,
  E_ERF_GRAD, E_FLOOR, E_CEIL, E_ROUND
};

// HALF: the caller rounds the result to fp16.
template <int OP, bool HALF> __device__ __forceinline__ float elemwise_apply(float f) {
  if (HALF) {
    if (OP == E_EXP) return exp_hw(f);
    if (OP == E_SIGMOID) return sigmoid_hw(f);
    if (OP == E_GELU_APPROX) return gelu_approx<true>(f);
  }
  switch (OP) {
    case E_SIN: return sinf(f);
    case E_COS: return cosf(f);
    case E_MINUS_SIN: return -sinf(f);
    case E_TAN: return tanf(f);
    case E_TAN_GRAD: return 1.0f / powf(cosf(f), 2.0f);
    case E_ATAN: return atanf(f);
    case E_ATAN_GRAD: return 1.0f / (1.0f + powf(f, 2.0f));
    case E_ACOS: return acosf(f);
    case E_ACOS_GRAD: return -1.0f / sqrtf(1.0f - powf(f, 2.0f));
    case E_ASIN: return asinf(f);
    case E_ASIN_GRAD: return 1.0f / sqrtf(1.0f - powf(f, 2.0f));
    case E_EXP: return expf(f);
    case E_LOG: return logf(f);
    case E_RECIP: return 1.0f / f;
    case E_SIGMOID: return safe_sigmoid(f);
    case E_SIGMOID_GRAD: return safe_sigmoid(f) * safe_sigmoid(-f);
    case E_RELU: return f < 0.0f ? 0.0f : f;
    case E_RELU_GRAD: return f < 0.0f ? 0.0f : 1.0f;
    case E_ABS: return f < 0.0f ? -f : f;
    case E_ABS_GRAD: return f < 0.0f ? -1.0f : 1.0f;
    case E_GELU_APPROX: return gelu_approx<false>(f);
    case E_GELU_APPROX_GRAD: {
      float tanh_term = tanhf(0.035677408145115f * powf(f, 3.0f) + 0.797884561f * f);
      return 0.5f * f * (1.0f - powf(tanh_term, 2.0f)) *
                 (0.107032224435345f * powf(f, 2.0f) + 0.797884561f) +
             0.5f * tanh_term + 0.5f;
    }
    case E_GELU_EXACT: return f * 0.5f * (1.0f + fast_erf(f * 0.7071067811865475f));
    case E_GELU_EXACT_GRAD: {
      const float c = 0.7071067811865475f;
      float term1 = 0.5f * (1.0f + fast_erf(f * c));
      float term2 = 0.5f * f * c * simple_erf_grad(f * c);
      return term1 + term2;
    }
    case E_ERF: return fast_erf(f);
    case E_ERF_GRAD: return simple_erf_grad(f);
    case E_FLOOR: return floorf(f);
    case E_CEIL: return ceilf(f);
    default: return roundf(f);
  }
}

// elemwise (BackendCPU.swift:1748-1766): out = f(x) * (scales?[i] ?? 1).
template <typename T, int OP> __device__ __forceinline__ void elemwise_impl(const hck_map_args& p) {
  const T* scales = (const T*)p.scales;
  if (scales) {
    map_contiguous((const T*)p.in, (T*)p.out, p.count, [scales](T xv, uint64_t i) {
      return narrow<T>(elemwise_apply<OP, sizeof(T) == 2>((float)xv) * (float)scales[i]);
    });
  } else {
    map_contiguous((const T*)p.in, (T*)p.out, p.count,
                   [](T xv, uint64_t) { return narrow<T>(elemwise_apply<OP, sizeof(T) == 2>((float)xv) * 1.0f); });
  }
}

#define DEF_ELEMWISE(NAME, OP)                                                                       \
  HC_KERNEL void hc_elemwise_##NAME##_f32(hck_map_args p) { elemwise_impl<float, OP>(p); }           \
  HC_KERNEL void hc_elemwise_##NAME##_f16(hck_map_args p) { elemwise_impl<half_t, OP>(p); }
DEF_ELEMWISE(sin, E_SIN)
DEF_ELEMWISE(cos, E_COS)
DEF_ELEMWISE(minus_sin, E_MINUS_SIN)
DEF_ELEMWISE(tan, E_TAN)
DEF_ELEMWISE(tan_grad, E_TAN_GRAD)
DEF_ELEMWISE(atan, E_ATAN)
DEF_ELEMWISE(atan_grad, E_ATAN_GRAD)
DEF_ELEMWISE(acos, E_ACOS)
DEF_ELEMWISE(acos_grad, E_ACOS_GRAD)
DEF_ELEMWISE(asin, E_ASIN)
DEF_ELEMWISE(asin_grad, E_ASIN_GRAD)
DEF_ELEMWISE(exp, E_EXP)
DEF_ELEMWISE(log, E_LOG)
DEF_ELEMWISE(recip, E_RECIP)
DEF_ELEMWISE(sigmoid, E_SIGMOID)
DEF_ELEMWISE(sigmoid_grad, E_SIGMOID_GRAD)
DEF_ELEMWISE(relu, E_RELU)
DEF_ELEMWISE(relu_grad, E_RELU_GRAD)
DEF_ELEMWISE(abs, E_ABS)
DEF_ELEMWISE(abs_grad, E_ABS_GRAD)
DEF_ELEMWISE(gelu_approx, E_GELU_APPROX)
DEF_ELEMWISE(gelu_approx_grad, E_GELU_APPROX_GRAD)
DEF_ELEMWISE(gelu_exact, E_GELU_EXACT)
DEF_ELEMWISE(gelu_exact_grad, E_GELU_EXACT_GRAD)
DEF_ELEMWISE(erf, E_ERF)
DEF_ELEMWISE(erf_grad, E_ERF_GRAD)
DEF_ELEMWISE(floor, E_FLOOR)
DEF_ELEMWISE(ceil, E_CEIL)
DEF_ELEMWISE(round, E_ROUND)

// ---------------------------------------------------------------- pow

// pow (BackendCPU.swift:648-702). MODE 0: scale * s * powf(x, b) (generic Float path);
// fp32 special cases: MODE 1 b == 2 (x*x, then *scale if scale != 1), MODE 2 b == -1
// (scale / x), MODE 3 b == 1 (x * scale); each followed by * scales[i] when given.
template <typename T, int MODE> __device__ __forceinline__ void pow_impl(const hck_map_args& p) {
  const T* scales = (const T*)p.scales;
  const float b = p.p0, scale = p.p1;
  map_contiguous((const T*)p.in, (T*)p.out, p.count, [=](T xv, uint64_t i) {
    float x = (float)xv;
    float r;
    if (MODE == 0) {
      r = scale * (scales ? (float)scales[i] : 1.0f) * pow_like(x, b);
    } else {
      if (MODE == 1) {
        r = x * x;
        if (scale != 1.0f) r = r * scale;
      } else if (MODE == 2) {
        r = scale / x;
      } else {
        r = x * scale;
      }
      if (scales) r = r * (float)scales[i];
    }
    return narrow<T>(r);
  });
}
HC_KERNEL void hc_pow_generic_f32(hck_map_args p) { pow_impl<float, 0>(p); }
HC_KERNEL void hc_pow_generic_f16(hck_map_args p) { pow_impl<half_t, 0>(p); }
HC_KERNEL void hc_pow_square_f32(hck_map_args p) { pow_impl<float, 1>(p); }
HC_KERNEL void hc_pow_recip_f32(hck_map_args p) { pow_impl<float, 2>(p); }
HC_KERNEL void hc_pow_linear_f32(hck_map_args p) { pow_impl<float, 3>(p); }

// Int64.pow (TensorElement.swift:205-207): Int64(pow(Double(x), Double(Float(b)))). The
// exponent is integral here, so the power is formed by squaring in double: exact, hence
// equal to a correctly rounded pow(), whenever |x^b| < 2^53.
HC_KERNEL void hc_pow_generic_i64(hck_map_args p) {
  const int64_t* scales = (const int64_t*)p.scales;
  const double b = (double)(float)p.i0;
  const int64_t scale = p.i1;
  map_contiguous((const int64_t*)p.in, (int64_t*)p.out, p.count, [=](int64_t x, uint64_t i) {
    double base = (double)x, acc = 1.0;
    double e = b < 0 ? -b : b;
    while (e >= 1.0) {
      const double half_e = floor(e * 0.5);
      if (e - 2.0 * half_e != 0.0) acc *= base;
      base *= base;
      e = half_e;
    }
    if (b < 0) acc = 1.0 / acc;
    int64_t pw = (int64_t)acc;
    return scale * (scales ? scales[i] : (int64_t)1) * pw;
  });
}

// ---------------------------------------------------------------- adamW

// One AdamW step (Backend.swift:818-892), the base class's op-by-op composition in one pass:
// every intermediate is rounded to the tensor dtype where the composition would have stored
// a tensor, squares and roots take the same paths as the pow kernels above (fp32: x*x then
// *scale unless scale == 1; fp16 and every root: scale * 1 * powf), and the file is built
// without FMA contraction, so the results equal the composed ones bit for bit.
template <typename T>
__device__ __forceinline__ void adamw_one(const hck_adamw_args& p, float param, float g, float m, float v,
                                          T& out_param, T& out_m, T& out_v) {
  const float m_scaled = round_through<T>(p.beta1 * m);
  const float g_scaled = round_through<T>(p.one_minus_beta1 * g);
  const float new_m = round_through<T>(m_scaled + g_scaled);
  float g_sq;
  if (sizeof(T) == 4) {
    g_sq = g * g;
    if (p.one_minus_beta2 != 1.0f) g_sq = g_sq * p.one_minus_beta2;
  } else {
    g_sq = round_through<T>(p.one_minus_beta2 * 1.0f * pow_like(g, p.exp_square));
  }
  const float v_scaled = round_through<T>(p.beta2 * v);
  const float new_v = round_through<T>(v_scaled + g_sq);
  const float m_hat = round_through<T>(new_m * p.bias1);
  const float v_hat = round_through<T>(new_v * p.bias2);
  const float root = round_through<T>(1.0f * 1.0f * pow_like(v_hat, p.exp_root));
  const float denom = round_through<T>(root + p.eps);
  const float ratio = round_through<T>(m_hat / denom);
  const float step_dir = round_through<T>(ratio * p.lr);
  const float decayed = round_through<T>(param * p.decay);
  out_param = narrow<T>(decayed - step_dir);
  out_m = narrow<T>(new_m);
  out_v = narrow<T>(new_v);
}

// 16-byte vectors, grid-stride; the ragged tail (< VEC elements) is done by the first lanes.
template <typename T> __device__ __forceinline__ void adamw_impl(const hck_adamw_args& p) {
  constexpr int VEC = VecWidth<T>::value;
  const uint64_t nvec = p.count / VEC;
  const uint64_t stride = (uint64_t)gridDim.x * HCK_BLOCK;
  const uint64_t t = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;
  for (uint64_t i = t; i < nvec; i += stride) {
    T pa[VEC], g[VEC], m[VEC], v[VEC], op[VEC], om[VEC], ov[VEC];
    load_vec<T, VEC>((const T*)p.param + i * VEC, 0, 1, pa);
    load_vec<T, VEC>((const T*)p.grad + i * VEC, 0, 1, g);
    load_vec<T, VEC>((const T*)p.m1 + i * VEC, 0, 1, m);
    load_vec<T, VEC>((const T*)p.m2 + i * VEC, 0, 1, v);
#pragma unroll
    for (int e = 0; e < VEC; e++)
      adamw_one<T>(p, (float)pa[e], (float)g[e], (float)m[e], (float)v[e], op[e], om[e], ov[e]);
    store_vec<T, VEC>((T*)p.out_param, i * VEC, op);
    store_vec<T, VEC>((T*)p.out_m1, i * VEC, om);
    store_vec<T, VEC>((T*)p.out_m2, i * VEC, ov);
  }
  const uint64_t i = nvec * VEC + t;
  if (i < p.count)
    adamw_one<T>(p, (float)((const T*)p.param)[i], (float)((const T*)p.grad)[i], (float)((const T*)p.m1)[i],
                 (float)((const T*)p.m2)[i], ((T*)p.out_param)[i], ((T*)p.out_m1)[i], ((T*)p.out_m2)[i]);
}
HC_KERNEL void hc_adamw_f32(hck_adamw_args p) { adamw_impl<float>(p); }
HC_KERNEL void hc_adamw_f16(hck_adamw_args p) { adamw_impl<half_t>(p); }

// ---------------------------------------------------------------- cast / fill

// cast (BackendCPU.swift:626-646 + TensorElement.swift:225-323): int64 sources convert
// directly; every other source is staged through Float.
template <typename TO> __device__ __forceinline__ TO cast_from_float(float v) { return narrow<TO>(v); }
template <> __device__ __forceinline__ uint8_t cast_from_float<uint8_t>(float v) { return v == 0 ? 0 : 1; }
template <typename TO> __device__ __forceinline__ TO cast_from_i64(int64_t v) { return (TO)v; }
template <> __device__ __forceinline__ uint8_t cast_from_i64<uint8_t>(int64_t v) { return v == 0 ? 0 : 1; }
template <> __device__ __forceinline__ half_t cast_from_i64<half_t>(int64_t v) { return narrow<half_t>((float)v); }

#define DEF_CAST_F(IN, TI, ON, TO)                                                                   \
  HC_KERNEL void hc_cast_##IN##_##ON(hck_map_args p) {                                               \
    map_contiguous((const TI*)p.in, (TO*)p.out, p.count,                                             \
                   [](TI x, uint64_t) { return cast_from_float<TO>(to_arith<TI>(x)); });             \
  }
#define DEF_CAST_I(ON, TO)                                                                           \
  HC_KERNEL void hc_cast_i64_##ON(hck_map_args p) {                                                  \
    map_contiguous((const int64_t*)p.in, (TO*)p.out, p.count,                                        \
                   [](int64_t x, uint64_t) { return cast_from_i64<TO>(x); });                        \
  }
DEF_CAST_F(f32, float, f16, half_t)
DEF_CAST_F(f32, float, i64, int64_t)
DEF_CAST_F(f32, float, b8, uint8_t)
DEF_CAST_F(f16, half_t, f32, float)
DEF_CAST_F(f16, half_t, i64, int64_t)
DEF_CAST_F(f16, half_t, b8, uint8_t)
DEF_CAST_F(b8, uint8_t, f32, float)
DEF_CAST_F(b8, uint8_t, f16, half_t)
DEF_CAST_F(b8, uint8_t, i64, int64_t)
DEF_CAST_I(f32, float)
DEF_CAST_I(f16, half_t)
DEF_CAST_I(b8, uint8_t)

// constant (BackendCPU.swift:1796-1815): the host converts the value to the element's
// bit pattern (i0); the kernel only replicates it.
template <typename T> __device__ __forceinline__ void fill_impl(const hck_map_args& p) {
  constexpr int VEC = VecWidth<T>::value;
  const T val = (T)p.i0;
  T* out = (T*)p.out;
  const uint64_t nvec = p.count / VEC;
  const uint64_t v = (uint64_t)blockIdx.x * HCK_BLOCK + threadIdx.x;
  if (v < nvec) {
    T r[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) r[i] = val;
    store_vec<T, VEC>(out, v * VEC, r);
  }
  if (v < p.count - nvec * VEC) out[nvec * VEC + v] = val;
}
HC_KERNEL void hc_fill_b1(hck_map_args p) { fill_impl<uint8_t>(p); }
HC_KERNEL void hc_fill_b2(hck_map_args p) { fill_impl<uint16_t>(p); }
HC_KERNEL void hc_fill_b4(hck_map_args p) { fill_impl<uint32_t>(p); }
HC_KERNEL void hc_fill_b8(hck_map_args p) { fill_impl<uint64_t>(p); }
