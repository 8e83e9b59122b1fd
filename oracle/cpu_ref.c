/*
 * TEST INFRASTRUCTURE ONLY - see cpu_ref.h. CPU restatement of the reference
 * CPUBackend arithmetic (Sources/Honeycrisp/BackendCPU.swift and friends).
 *
 * Build with -O2 -ffp-contract=off -fno-fast-math: Swift never fuses a*b+c
 * and evaluates Float expressions in binary32.
 *
 * Where the reference calls Accelerate (vDSP_vadd, vDSP_sve, vDSP_mmul ...)
 * the textbook routine is used; summation order inside vDSP_sve / vDSP_mmul
 * is unspecified, so fp32 sum and fp32 NN matmul are tolerance-only.
 */
#include "cpu_ref.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 0;

void ref_set_threads(int n) { g_threads = n; }

static int nthreads(void) {
#ifdef _OPENMP
  return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---- binary16 <-> binary32 (TensorElement.swift:262-277, 325-338: vImage planar
 * conversions = IEEE round-to-nearest-even, overflow to inf, subnormals kept) ---- */

uint16_t ref_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) { /* inf / nan */
    if (absx > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((absx >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx >= 0x477ff000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx < 0x38800000u) { /* subnormal half or zero: < 2^-14 */
    if (absx < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 (2^-25 itself ties to even 0) */
    int exp = (int)(absx >> 23);
    uint32_t mant = (absx & 0x7fffffu) | 0x800000u;
    int shift = 126 - exp; /* value = mant * 2^(exp-150); half subnormal unit 2^-24 */
    /* result = mant >> shift with RNE, shift in [14, 24] */
    uint32_t res = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (res & 1u))) res++;
    return (uint16_t)(sign | res);
  }
  {
    uint32_t exp = (absx >> 23) - 112u;
    uint32_t mant = absx & 0x7fffffu;
    uint32_t res = (exp << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (res & 1u))) res++;
    return (uint16_t)(sign | res);
  }
}

float ref_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t mant = h & 0x3ffu;
  uint32_t x;
  if (exp == 0) {
    if (mant == 0) {
      x = sign;
    } else {
      int e = -1;
      do {
        mant <<= 1;
        e++;
      } while (!(mant & 0x400u));
      x = sign | ((uint32_t)(112 - e) << 23) | ((mant & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    x = sign | 0x7f800000u | (mant << 13);
  } else {
    x = sign | ((exp + 112u) << 23) | (mant << 13);
  }
  float f;
  memcpy(&f, &x, 4);
  return f;
}

void ref_f32_to_f16_n(const float* in, uint16_t* out, size_t n) {
#pragma omp parallel for num_threads(nthreads()) if (n > 65536)
  for (size_t i = 0; i < n; i++) out[i] = ref_f32_to_f16(in[i]);
}

void ref_f16_to_f32_n(const uint16_t* in, float* out, size_t n) {
#pragma omp parallel for num_threads(nthreads()) if (n > 65536)
  for (size_t i = 0; i < n; i++) out[i] = ref_f16_to_f32(in[i]);
}

static size_t dtype_size(int dtype) {
  switch (dtype) {
    case REF_I64: return 8;
    case REF_BOOL: return 1;
    case REF_F16: return 2;
    default: return 4;
  }
}

/* readBuffer(Float.self, ...) (BackendCPU.swift:2018-2030): fp32 is used in place,
 * anything else is converted wholesale (pointerToArray, TensorElement.swift:279-323). */
static const float* load_f(int dtype, const void* p, size_t n, float** owned) {
  *owned = NULL;
  if (dtype == REF_F32) return (const float*)p;
  float* buf = (float*)malloc((n ? n : 1) * sizeof(float));
  *owned = buf;
  if (dtype == REF_F16) {
    ref_f16_to_f32_n((const uint16_t*)p, buf, n);
  } else if (dtype == REF_BOOL) {
    const uint8_t* b = (const uint8_t*)p;
    for (size_t i = 0; i < n; i++) buf[i] = b[i] ? 1.0f : 0.0f;
  } else {
    const int64_t* v = (const int64_t*)p;
    for (size_t i = 0; i < n; i++) buf[i] = (float)v[i];
  }
  return buf;
}

/* writeBuffer(Float.self, ...) (BackendCPU.swift:2045-2058): compute into a Float
 * array, then arrayToPointer (TensorElement.swift:225-260). */
static float* out_f(int dtype, void* p, size_t n, float** owned) {
  *owned = NULL;
  if (dtype == REF_F32) return (float*)p;
  *owned = (float*)malloc((n ? n : 1) * sizeof(float));
  return *owned;
}

static void store_f(int dtype, void* p, size_t n, float* owned) {
  if (!owned) return;
  if (dtype == REF_F16) {
    ref_f32_to_f16_n(owned, (uint16_t*)p, n);
  } else if (dtype == REF_BOOL) {
    uint8_t* b = (uint8_t*)p;
    for (size_t i = 0; i < n; i++) b[i] = owned[i] == 0 ? 0 : 1;
  } else if (dtype == REF_I64) {
    int64_t* v = (int64_t*)p;
    for (size_t i = 0; i < n; i++) v[i] = (int64_t)owned[i];
  }
  free(owned);
}

/* ---- BroadcastStrides (Broadcast.swift:15-30, 72-90) ---- */

static int64_t shape_product(const ref_strides* s) {
  int64_t n = 1;
  for (uint32_t d = 0; d < s->ndim; d++) n *= s->shape[d];
  return n;
}

static int64_t data_count(const ref_strides* s) {
  int64_t n = 1;
  for (uint32_t d = 0; d < s->ndim; d++)
    if (s->strides[d] != 0) n *= s->shape[d];
  return n;
}

static int is_noop(const ref_strides* s) {
  for (uint32_t d = 0; d < s->ndim; d++)
    if (!(s->strides[d] != 0 || s->shape[d] == 1)) return 0;
  return 1;
}

int64_t ref_strides_index(const ref_strides* s, int64_t i) {
  if (is_noop(s)) return i;
  int64_t cur = i, result = 0;
  for (int d = (int)s->ndim - 1; d >= 0; d--) {
    result += s->strides[d] * (cur % s->shape[d]);
    cur /= s->shape[d];
  }
  return result;
}

/* ---- scalar semantics (TensorElement.swift:95-133, 196-223; BinaryOps.swift:9-22) ---- */

static float modulus_f(float lhs, float rhs) {
  if (rhs < 0) return -modulus_f(-lhs, -rhs);
  if (lhs < 0) return fmodf(rhs - fmodf(rhs - lhs, rhs), rhs);
  return fmodf(lhs, rhs);
}

static int64_t modulus_i(int64_t lhs, int64_t rhs) {
  if (rhs < 0) return -modulus_i(-lhs, -rhs);
  if (lhs < 0) return (rhs - ((rhs - lhs) % rhs)) % rhs;
  return lhs % rhs;
}

static inline float binop_f(int op, float a, float b) {
  switch (op) {
    case REF_ADD: return a + b;
    case REF_MUL: return a * b;
    case REF_SUB: return a - b;
    case REF_DIV: return a / b;
    default: return modulus_f(a, b);
  }
}

static inline int64_t binop_i(int op, int64_t a, int64_t b) {
  switch (op) {
    case REF_ADD: return (int64_t)((uint64_t)a + (uint64_t)b);
    case REF_MUL: return (int64_t)((uint64_t)a * (uint64_t)b);
    case REF_SUB: return (int64_t)((uint64_t)a - (uint64_t)b);
    case REF_DIV: return a / b;
    default: return modulus_i(a, b);
  }
}

/* ---- broadcast (BackendCPU.swift:255-265) ---- */

void ref_broadcast(int dtype, const void* a, const ref_strides* as, void* out) {
  int64_t n = shape_product(as);
  size_t el = dtype_size(dtype);
  for (int64_t i = 0; i < n; i++)
    memcpy((char*)out + el * i, (const char*)a + el * ref_strides_index(as, i), el);
}

/* ---- binaryOp tensor x tensor (BackendCPU.swift:267-314) ---- */

void ref_binary_op(int op, int dtype, const void* a, const ref_strides* as, const void* b,
                   const ref_strides* bs, void* out) {
  int64_t n = shape_product(as);
  if (dtype == REF_I64) {
    const int64_t* x = (const int64_t*)a;
    const int64_t* y = (const int64_t*)b;
    int64_t* z = (int64_t*)out;
    for (int64_t i = 0; i < n; i++)
      z[i] = binop_i(op, x[ref_strides_index(as, i)], y[ref_strides_index(bs, i)]);
    return;
  }
  /* fp32 with both operands un-broadcast takes vDSP_vadd/vmul/vdiv/vsub (:276-293):
   * the same IEEE element-wise operations as the generic loop below. */
  float *ao, *bo, *zo;
  const float* x = load_f(dtype, a, (size_t)data_count(as), &ao);
  const float* y = load_f(dtype, b, (size_t)data_count(bs), &bo);
  float* z = out_f(dtype, out, (size_t)n, &zo);
#pragma omp parallel for num_threads(nthreads()) if (n > 65536)
  for (int64_t i = 0; i < n; i++)
    z[i] = binop_f(op, x[ref_strides_index(as, i)], y[ref_strides_index(bs, i)]);
  store_f(dtype, out, (size_t)n, zo);
  free(ao);
  free(bo);
}

/* ---- binaryOp tensor x scalar / scalar x tensor (BackendCPU.swift:316-405) ---- */

void ref_binary_op_scalar(int op, int dtype, const void* a, float sf, int64_t si,
                          int scalar_first, void* out, size_t count) {
  if (dtype == REF_I64) {
    const int64_t* x = (const int64_t*)a;
    int64_t* z = (int64_t*)out;
    for (size_t i = 0; i < count; i++)
      z[i] = scalar_first ? binop_i(op, si, x[i]) : binop_i(op, x[i], si);
    return;
  }
  if (dtype == REF_F32 && op != REF_MOD) {
    const float* x = (const float*)a;
    float* z = (float*)out;
    if (!scalar_first) {
      /* :325-342: div multiplies by the reciprocal, sub adds the negation */
      float s = op == REF_DIV ? 1.0f / sf : (op == REF_SUB ? -sf : sf);
      if (op == REF_ADD || op == REF_SUB) {
        for (size_t i = 0; i < count; i++) z[i] = x[i] + s; /* vDSP_vsadd */
      } else {
        for (size_t i = 0; i < count; i++) z[i] = x[i] * s; /* vDSP_vsmul */
      }
    } else {
      /* :366-389 */
      switch (op) {
        case REF_ADD:
          for (size_t i = 0; i < count; i++) z[i] = x[i] + sf;
          break;
        case REF_MUL:
          for (size_t i = 0; i < count; i++) z[i] = x[i] * sf;
          break;
        case REF_DIV:
          for (size_t i = 0; i < count; i++) z[i] = sf / x[i]; /* vDSP_svdiv */
          break;
        default:
          for (size_t i = 0; i < count; i++) z[i] = x[i] * -1.0f + sf; /* vDSP_vsmsa */
          break;
      }
    }
    return;
  }
  float *ao, *zo;
  const float* x = load_f(dtype, a, count, &ao);
  float* z = out_f(dtype, out, count, &zo);
  for (size_t i = 0; i < count; i++)
    z[i] = scalar_first ? binop_f(op, sf, x[i]) : binop_f(op, x[i], sf);
  store_f(dtype, out, count, zo);
  free(ao);
}

/* ---- mulAdd / addMul (BackendCPU.swift:445-539) ---- */

static void fused3(int is_mul_add, int dtype, const void* in, const ref_strides* is,
                   const void* coeff, const ref_strides* cs, const void* bias,
                   const ref_strides* bs, void* out) {
  int64_t n = shape_product(is);
  if (dtype == REF_I64) {
    const int64_t* x = (const int64_t*)in;
    const int64_t* c = (const int64_t*)coeff;
    const int64_t* b = (const int64_t*)bias;
    int64_t* z = (int64_t*)out;
    for (int64_t i = 0; i < n; i++) {
      int64_t xv = x[ref_strides_index(is, i)], cv = c[ref_strides_index(cs, i)],
              bv = b[ref_strides_index(bs, i)];
      z[i] = is_mul_add ? binop_i(REF_ADD, binop_i(REF_MUL, xv, cv), bv)
                        : binop_i(REF_MUL, binop_i(REF_ADD, xv, bv), cv);
    }
    return;
  }
  /* the all-simple fp32 case uses vDSP_vma / vDSP_vam: D = A*B + C and D = (A+B)*C */
  float *xo, *co, *bo, *zo;
  const float* x = load_f(dtype, in, (size_t)data_count(is), &xo);
  const float* c = load_f(dtype, coeff, (size_t)data_count(cs), &co);
  const float* b = load_f(dtype, bias, (size_t)data_count(bs), &bo);
  float* z = out_f(dtype, out, (size_t)n, &zo);
  for (int64_t i = 0; i < n; i++) {
    float xv = x[ref_strides_index(is, i)], cv = c[ref_strides_index(cs, i)],
          bv = b[ref_strides_index(bs, i)];
    z[i] = is_mul_add ? xv * cv + bv : (xv + bv) * cv;
  }
  store_f(dtype, out, (size_t)n, zo);
  free(xo);
  free(co);
  free(bo);
}

void ref_mul_add(int dtype, const void* in, const ref_strides* is, const void* coeff,
                 const ref_strides* cs, const void* bias, const ref_strides* bs, void* out) {
  fused3(1, dtype, in, is, coeff, cs, bias, bs, out);
}

void ref_add_mul(int dtype, const void* in, const ref_strides* is, const void* bias,
                 const ref_strides* bs, const void* coeff, const ref_strides* cs, void* out) {
  fused3(0, dtype, in, is, coeff, cs, bias, bs, out);
}

/* ---- compare (BackendCPU.swift:541-624, Comparison.swift:12-27) ---- */

static inline int cmp_f(int op, float a, float b) {
  switch (op) {
    case REF_EQ: return a == b;
    case REF_NE: return a != b;
    case REF_LT: return a < b;
    case REF_LE: return a <= b;
    case REF_GT: return a > b;
    default: return a >= b;
  }
}

static inline int cmp_i(int op, int64_t a, int64_t b) {
  switch (op) {
    case REF_EQ: return a == b;
    case REF_NE: return a != b;
    case REF_LT: return a < b;
    case REF_LE: return a <= b;
    case REF_GT: return a > b;
    default: return a >= b;
  }
}

void ref_compare(int op, int dtype, const void* a, const ref_strides* as, const void* b,
                 const ref_strides* bs, uint8_t* out) {
  int64_t n = shape_product(as);
  if (dtype == REF_I64) {
    const int64_t* x = (const int64_t*)a;
    const int64_t* y = (const int64_t*)b;
    for (int64_t i = 0; i < n; i++)
      out[i] = (uint8_t)cmp_i(op, x[ref_strides_index(as, i)], y[ref_strides_index(bs, i)]);
    return;
  }
  float *ao, *bo;
  const float* x = load_f(dtype, a, (size_t)data_count(as), &ao);
  const float* y = load_f(dtype, b, (size_t)data_count(bs), &bo);
  for (int64_t i = 0; i < n; i++)
    out[i] = (uint8_t)cmp_f(op, x[ref_strides_index(as, i)], y[ref_strides_index(bs, i)]);
  free(ao);
  free(bo);
}

void ref_compare_scalar(int op, int dtype, const void* a, float sf, int64_t si, int scalar_first,
                        uint8_t* out, size_t count) {
  if (dtype == REF_I64) {
    const int64_t* x = (const int64_t*)a;
    for (size_t i = 0; i < count; i++)
      out[i] = (uint8_t)(scalar_first ? cmp_i(op, si, x[i]) : cmp_i(op, x[i], si));
    return;
  }
  float* ao;
  const float* x = load_f(dtype, a, count, &ao);
  for (size_t i = 0; i < count; i++)
    out[i] = (uint8_t)(scalar_first ? cmp_f(op, sf, x[i]) : cmp_f(op, x[i], sf));
  free(ao);
}

/* ---- cast (BackendCPU.swift:626-646 + TensorElement.swift:225-323) ---- */

void ref_cast(const void* in, int in_type, void* out, int out_type, size_t count) {
  if (in_type == REF_I64) {
    /* staged through [Int64]; Int64.isFloatLossy => B(x.toInt64()) */
    const int64_t* x = (const int64_t*)in;
    switch (out_type) {
      case REF_I64: memcpy(out, in, count * 8); break;
      case REF_BOOL:
        for (size_t i = 0; i < count; i++) ((uint8_t*)out)[i] = x[i] == 0 ? 0 : 1;
        break;
      case REF_F32:
        for (size_t i = 0; i < count; i++) ((float*)out)[i] = (float)x[i];
        break;
      default:
        for (size_t i = 0; i < count; i++) ((uint16_t*)out)[i] = ref_f32_to_f16((float)x[i]);
        break;
    }
    return;
  }
  /* staged through [Float] */
  float* ao;
  const float* x = load_f(in_type, in, count, &ao);
  switch (out_type) {
    case REF_I64:
      for (size_t i = 0; i < count; i++) ((int64_t*)out)[i] = (int64_t)x[i];
      break;
    case REF_BOOL:
      for (size_t i = 0; i < count; i++) ((uint8_t*)out)[i] = x[i] == 0 ? 0 : 1;
      break;
    case REF_F32:
      if (out != (void*)x) memcpy(out, x, count * 4);
      break;
    default: ref_f32_to_f16_n(x, (uint16_t*)out, count); break;
  }
  free(ao);
}

/* ---- pow (BackendCPU.swift:648-702) ---- */

void ref_pow(int dtype, const void* in, float bf, float scalef, int64_t bi, int64_t scalei,
             const void* scales, void* out, size_t count) {
  if (dtype == REF_I64) {
    /* Int64.pow: Int64(Foundation.pow(Double(self), Double(exponent.toFloat()))) */
    const int64_t* x = (const int64_t*)in;
    const int64_t* s = (const int64_t*)scales;
    int64_t* z = (int64_t*)out;
    for (size_t i = 0; i < count; i++) {
      int64_t p = (int64_t)pow((double)x[i], (double)(float)bi);
      z[i] = binop_i(REF_MUL, binop_i(REF_MUL, scalei, s ? s[i] : 1), p);
    }
    return;
  }
  if (dtype == REF_F32 && (bf == 2.0f || bf == -1.0f || bf == 1.0f)) {
    const float* x = (const float*)in;
    const float* s = (const float*)scales;
    float* z = (float*)out;
    if (bf == 2.0f) {
      for (size_t i = 0; i < count; i++) z[i] = x[i] * x[i];
      if (scalef != 1.0f)
        for (size_t i = 0; i < count; i++) z[i] = z[i] * scalef;
    } else if (bf == -1.0f) {
      for (size_t i = 0; i < count; i++) z[i] = scalef / x[i];
    } else {
      for (size_t i = 0; i < count; i++) z[i] = x[i] * scalef;
    }
    if (s)
      for (size_t i = 0; i < count; i++) z[i] = z[i] * s[i];
    return;
  }
  float *ao, *so = NULL, *zo;
  const float* x = load_f(dtype, in, count, &ao);
  const float* s = scales ? load_f(dtype, scales, count, &so) : NULL;
  float* z = out_f(dtype, out, count, &zo);
  for (size_t i = 0; i < count; i++) z[i] = scalef * (s ? s[i] : 1.0f) * powf(x[i], bf);
  store_f(dtype, out, count, zo);
  free(ao);
  free(so);
}

/* ---- elemwise (BackendCPU.swift:1748-1766, formulas Elemwise.swift:44-183) ---- */

static float safe_sigmoid(float x) {
  if (x < -20.0f) return 0.0f;
  if (x > 20.0f) return 1.0f;
  return 1.0f / (1.0f + expf(-x));
}

static float safe_tanh(float x) { return 2.0f * safe_sigmoid(2.0f * x) - 1.0f; }

static float nofma(float x, float y, float z) { return x * y + z; }

static float fast_erf(float a) {
  float r, s, t, u;
  t = fabsf(a);
  s = a * a;
  if (t > 0.927734375f) {
    r = nofma(-1.72853470e-5f, t, 3.83197126e-4f);
    u = nofma(-3.88396438e-3f, t, 2.42546219e-2f);
    r = nofma(r, s, u);
    r = nofma(r, t, -1.06777877e-1f);
    r = nofma(r, t, -6.34846687e-1f);
    r = nofma(r, t, -1.28717512e-1f);
    r = nofma(r, t, -t);
    r = 1.0f - expf(r);
    r = copysignf(r, a);
  } else {
    r = -5.96761703e-4f;
    r = nofma(r, s, 4.99119423e-3f);
    r = nofma(r, s, -2.67681349e-2f);
    r = nofma(r, s, 1.12819925e-1f);
    r = nofma(r, s, -3.76125336e-1f);
    r = nofma(r, s, 1.28379166e-1f);
    r = nofma(r, a, a);
  }
  return r;
}

static float simple_erf_grad(float f) {
  return fabsf(f) > 20.0f ? 0.0f : 1.1283791670955126f * expf(-f * f);
}

static float elemwise_apply(int op, float f) {
  switch (op) {
    case REF_SIN: return sinf(f);
    case REF_COS: return cosf(f);
    case REF_MINUS_SIN: return -sinf(f);
    case REF_TAN: return tanf(f);
    case REF_TAN_GRAD: return 1.0f / powf(cosf(f), 2.0f);
    case REF_ATAN: return atanf(f);
    case REF_ATAN_GRAD: return 1.0f / (1.0f + powf(f, 2.0f));
    case REF_ACOS: return acosf(f);
    case REF_ACOS_GRAD: return -1.0f / sqrtf(1.0f - powf(f, 2.0f));
    case REF_ASIN: return asinf(f);
    case REF_ASIN_GRAD: return 1.0f / sqrtf(1.0f - powf(f, 2.0f));
    case REF_EXP: return expf(f);
    case REF_LOG: return logf(f);
    case REF_RECIP: return 1.0f / f;
    case REF_SIGMOID: return safe_sigmoid(f);
    case REF_SIGMOID_GRAD: return safe_sigmoid(f) * safe_sigmoid(-f);
    case REF_RELU: return f < 0.0f ? 0.0f : f;
    case REF_RELU_GRAD: return f < 0.0f ? 0.0f : 1.0f;
    case REF_ABS: return f < 0.0f ? -f : f;
    case REF_ABS_GRAD: return f < 0.0f ? -1.0f : 1.0f;
    case REF_GELU_APPROX:
      return 0.5f * f * (1.0f + safe_tanh(0.797884561f * (f + 0.044715f * powf(f, 3.0f))));
    case REF_GELU_APPROX_GRAD: {
      float tanh_term = tanhf(0.035677408145115f * powf(f, 3.0f) + 0.797884561f * f);
      return 0.5f * f * (1.0f - powf(tanh_term, 2.0f)) *
                 (0.107032224435345f * powf(f, 2.0f) + 0.797884561f) +
             0.5f * tanh_term + 0.5f;
    }
    case REF_GELU_EXACT: return f * 0.5f * (1.0f + fast_erf(f * 0.7071067811865475f));
    case REF_GELU_EXACT_GRAD: {
      const float c = 0.7071067811865475f;
      float term1 = 0.5f * (1.0f + fast_erf(f * c));
      float term2 = 0.5f * f * c * simple_erf_grad(f * c);
      return term1 + term2;
    }
    case REF_ERF: return fast_erf(f);
    case REF_ERF_GRAD: return simple_erf_grad(f);
    case REF_FLOOR: return floorf(f);
    case REF_CEIL: return ceilf(f);
    default: return roundf(f); /* Float.rounded() = to nearest, ties away from zero */
  }
}

void ref_elemwise(int op, int dtype, const void* in, const void* scales, void* out, size_t count) {
  float *ao, *so = NULL, *zo;
  const float* x = load_f(dtype, in, count, &ao);
  const float* s = scales ? load_f(dtype, scales, count, &so) : NULL;
  float* z = out_f(dtype, out, count, &zo);
#pragma omp parallel for num_threads(nthreads()) if (count > 65536)
  for (size_t i = 0; i < count; i++) z[i] = elemwise_apply(op, x[i]) * (s ? s[i] : 1.0f);
  store_f(dtype, out, count, zo);
  free(ao);
  free(so);
}

/* ---- reduce (BackendCPU.swift:784-886) ---- */

void ref_reduce(int op, int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
                int64_t inner) {
  size_t in_count = (size_t)(outer * reduce * inner), out_count = (size_t)(outer * inner);
  if (dtype == REF_I64) {
    const int64_t* arr = (const int64_t*)in;
    int64_t* o = (int64_t*)out;
    for (int64_t i = 0; i < outer; i++)
      for (int64_t j = 0; j < inner; j++) {
        const int64_t* base = arr + j + i * reduce * inner;
        int64_t r;
        if (op == REF_SUM) {
          r = 0;
          for (int64_t k = 0; k < reduce; k++) r = binop_i(REF_ADD, r, base[k * inner]);
        } else if (op == REF_PROD) {
          r = 1;
          for (int64_t k = 0; k < reduce; k++) r = binop_i(REF_MUL, r, base[k * inner]);
        } else {
          int64_t ext = base[0];
          r = 0;
          for (int64_t k = 0; k < reduce; k++) {
            int64_t item = base[k * inner];
            if (op == REF_ARGMIN ? item < ext : item > ext) {
              ext = item;
              r = k;
            }
          }
        }
        o[i * inner + j] = r;
      }
    return;
  }
  float* ao;
  const float* arr = load_f(dtype, in, in_count, &ao);
  if (op == REF_ARGMAX || op == REF_ARGMIN) {
    int64_t* o = (int64_t*)out;
#pragma omp parallel for num_threads(nthreads()) if (in_count > 65536)
    for (int64_t i = 0; i < outer; i++)
      for (int64_t j = 0; j < inner; j++) {
        const float* base = arr + j + i * reduce * inner;
        float ext = base[0];
        int64_t idx = 0;
        for (int64_t k = 0; k < reduce; k++) {
          float item = base[k * inner];
          if (op == REF_ARGMIN ? item < ext : item > ext) {
            ext = item;
            idx = k;
          }
        }
        o[i * inner + j] = idx;
      }
  } else {
    /* fp32 sum goes through vDSP_sve (:792-806, order unspecified); the sequential
     * order of the generic loop (:810-828) is used for every float dtype here. */
    float* zo;
    float* z = out_f(dtype, out, out_count, &zo);
#pragma omp parallel for num_threads(nthreads()) if (in_count > 65536)
    for (int64_t i = 0; i < outer; i++)
      for (int64_t j = 0; j < inner; j++) {
        const float* base = arr + j + i * reduce * inner;
        float r = op == REF_SUM ? 0.0f : 1.0f;
        if (op == REF_SUM)
          for (int64_t k = 0; k < reduce; k++) r = r + base[k * inner];
        else
          for (int64_t k = 0; k < reduce; k++) r = r * base[k * inner];
        z[i * inner + j] = r;
      }
    store_f(dtype, out, out_count, zo);
  }
  free(ao);
}

/* ---- logSoftmax (BackendCPU.swift:1000-1038) ---- */

void ref_log_softmax(int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
                     int64_t inner) {
  size_t total = (size_t)(outer * reduce * inner);
  float *ao, *zo;
  const float* arr = load_f(dtype, in, total, &ao);
  float* z = out_f(dtype, out, total, &zo);
#pragma omp parallel for num_threads(nthreads()) if (total > 65536)
  for (int64_t i = 0; i < outer; i++) {
    int64_t off = i * inner * reduce;
    for (int64_t j = 0; j < inner; j++) {
      float max = 0;
      for (int64_t k = 0; k < reduce; k++) {
        float item = arr[j + k * inner + off];
        if (k == 0 || item > max) max = item;
      }
      float exp_sum = 0;
      for (int64_t k = 0; k < reduce; k++) exp_sum += expf(arr[j + k * inner + off] - max);
      float log_sum = logf(exp_sum) + max;
      for (int64_t k = 0; k < reduce; k++) {
        int64_t idx = j + k * inner + off;
        z[idx] = arr[idx] - log_sum;
      }
    }
  }
  store_f(dtype, out, total, zo);
  free(ao);
}

/* ---- gather (BackendCPU.swift:1108-1147): pure data movement, any dtype ---- */

void ref_gather(int dtype, const void* in, const int64_t* idx, const ref_strides* idx_strides,
                void* out, int64_t outer, int64_t middle, int64_t out_count, int64_t inner) {
  size_t el = dtype_size(dtype);
#pragma omp parallel for num_threads(nthreads()) if (outer * out_count * inner > 65536)
  for (int64_t ij = 0; ij < outer * out_count; ij++) {
    int64_t i = ij / out_count;
    for (int64_t k = 0; k < inner; k++) {
      int64_t out_idx = ij * inner + k;
      int64_t in_idx = idx[ref_strides_index(idx_strides, out_idx)];
      memcpy((char*)out + el * out_idx,
             (const char*)in + el * ((i * middle + in_idx) * inner + k), el);
    }
  }
}

/* ---- cumulativeSum / cumulativeProd (BackendCPU.swift:922-998) ---- */

void ref_cumulative(int op, int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
                    int64_t inner, int exclusive, int reverse) {
  size_t total = (size_t)(outer * reduce * inner);
  if (dtype == REF_I64) {
    const int64_t* x = (const int64_t*)in;
    int64_t* z = (int64_t*)out;
    for (int64_t i = 0; i < outer; i++)
      for (int64_t j = 0; j < inner; j++) {
        int64_t run = op == 0 ? 0 : 1;
        for (int64_t t = 0; t < reduce; t++) {
          int64_t k = reverse ? reduce - 1 - t : t;
          int64_t idx = j + (k + i * reduce) * inner;
          int64_t next = op == 0 ? run + x[idx] : run * x[idx];
          z[idx] = exclusive ? run : next;
          run = next;
        }
      }
    return;
  }
  float *xo, *zo;
  const float* x = load_f(dtype, in, total, &xo);
  float* z = out_f(dtype, out, total, &zo);
  for (int64_t i = 0; i < outer; i++)
    for (int64_t j = 0; j < inner; j++) {
      float run = op == 0 ? 0.0f : 1.0f;
      for (int64_t t = 0; t < reduce; t++) {
        int64_t k = reverse ? reduce - 1 - t : t;
        int64_t idx = j + (k + i * reduce) * inner;
        float next = op == 0 ? run + x[idx] : run * x[idx];
        z[idx] = exclusive ? run : next;
        run = next;
      }
    }
  store_f(dtype, out, total, zo);
  free(xo);
}

/* ---- argsort (BackendCPU.swift:888-920), stable: insertion into a merge sort ---- */

static void argsort_merge(const double* key, int64_t* idx, int64_t* tmp, int64_t n, int descending) {
  for (int64_t width = 1; width < n; width *= 2) {
    for (int64_t lo = 0; lo < n; lo += 2 * width) {
      int64_t mid = lo + width < n ? lo + width : n, hi = lo + 2 * width < n ? lo + 2 * width : n;
      int64_t a = lo, b = mid, o = lo;
      while (a < mid && b < hi) {
        /* take from the right run only if it is strictly ahead: equal keys keep their order */
        int right = descending ? key[idx[b]] > key[idx[a]] : key[idx[b]] < key[idx[a]];
        tmp[o++] = right ? idx[b++] : idx[a++];
      }
      while (a < mid) tmp[o++] = idx[a++];
      while (b < hi) tmp[o++] = idx[b++];
    }
    memcpy(idx, tmp, (size_t)n * sizeof(int64_t));
  }
}

void ref_argsort(int dtype, const void* in, int64_t* out, int64_t outer, int64_t reduce, int64_t inner,
                 int descending) {
  size_t total = (size_t)(outer * reduce * inner);
  float* xo = NULL;
  const float* xf = dtype == REF_I64 ? NULL : load_f(dtype, in, total, &xo);
  double* key = (double*)malloc((size_t)(reduce ? reduce : 1) * sizeof(double));
  int64_t* idx = (int64_t*)malloc((size_t)(reduce ? reduce : 1) * sizeof(int64_t));
  int64_t* tmp = (int64_t*)malloc((size_t)(reduce ? reduce : 1) * sizeof(int64_t));
  for (int64_t i = 0; i < outer; i++)
    for (int64_t j = 0; j < inner; j++) {
      for (int64_t k = 0; k < reduce; k++) {
        int64_t src = j + (k + i * reduce) * inner;
        /* int64 keys of the tests fit a double exactly (|x| < 2^53) */
        key[k] = dtype == REF_I64 ? (double)((const int64_t*)in)[src] : (double)xf[src];
        idx[k] = k;
      }
      argsort_merge(key, idx, tmp, reduce, descending);
      for (int64_t k = 0; k < reduce; k++) out[j + (k + i * reduce) * inner] = idx[k];
    }
  free(key);
  free(idx);
  free(tmp);
  free(xo);
}

/* ---- bitwiseOp (BackendCPU.swift:407-425): byte by byte, as the reference does ---- */

void ref_bitwise_op(int op, int dtype, const void* a, const ref_strides* as, const void* b,
                    const ref_strides* bs, void* out) {
  int64_t count = shape_product(as);
  int64_t el = (int64_t)dtype_size(dtype);
  const uint8_t *x = (const uint8_t*)a, *y = (const uint8_t*)b;
  uint8_t* z = (uint8_t*)out;
  for (int64_t i = 0; i < count * el; i++) {
    uint8_t p = x[ref_strides_index(as, i / el) * el + i % el];
    uint8_t q = y[ref_strides_index(bs, i / el) * el + i % el];
    z[i] = op == 0 ? (uint8_t)(p | q) : op == 1 ? (uint8_t)(p & q) : (uint8_t)(p ^ q);
  }
}

/* ---- scatter (BackendCPU.swift:1149-1188): sequential accumulation in Float / Int64 ---- */

void ref_scatter(int dtype, const void* in, const int64_t* idx, const ref_strides* idx_strides,
                 void* out, int64_t outer, int64_t middle, int64_t out_count, int64_t inner) {
  size_t n_in = (size_t)(outer * out_count * inner), n_out = (size_t)(outer * middle * inner);
  if (dtype == REF_I64) {
    const int64_t* x = (const int64_t*)in;
    int64_t* z = (int64_t*)out;
    for (size_t t = 0; t < n_out; t++) z[t] = 0;
    for (int64_t i = 0; i < outer; i++)
      for (int64_t j = 0; j < out_count; j++)
        for (int64_t k = 0; k < inner; k++) {
          int64_t in_idx = (i * out_count + j) * inner + k;
          int64_t j_out = idx[ref_strides_index(idx_strides, in_idx)];
          int64_t out_idx = (i * middle + j_out) * inner + k;
          z[out_idx] = z[out_idx] + x[in_idx];
        }
    return;
  }
  float *xo, *zo;
  const float* x = load_f(dtype, in, n_in, &xo);
  float* z = out_f(dtype, out, n_out, &zo);
  for (size_t t = 0; t < n_out; t++) z[t] = 0.0f;
  for (int64_t i = 0; i < outer; i++)
    for (int64_t j = 0; j < out_count; j++)
      for (int64_t k = 0; k < inner; k++) {
        int64_t in_idx = (i * out_count + j) * inner + k;
        int64_t j_out = idx[ref_strides_index(idx_strides, in_idx)];
        int64_t out_idx = (i * middle + j_out) * inner + k;
        z[out_idx] = z[out_idx] + x[in_idx];
      }
  store_f(dtype, out, n_out, zo);
  free(xo);
}

/* ---- logSoftmaxGrad (BackendCPU.swift:1040-1085) ---- */

void ref_log_softmax_grad(int dtype, const void* in, const void* out_grad, void* out, int64_t outer,
                          int64_t reduce, int64_t inner) {
  size_t total = (size_t)(outer * reduce * inner);
  float *ao, *go, *zo;
  const float* arr = load_f(dtype, in, total, &ao);
  const float* grad = load_f(dtype, out_grad, total, &go);
  float* z = out_f(dtype, out, total, &zo);
#pragma omp parallel for num_threads(nthreads()) if (total > 65536)
  for (int64_t i = 0; i < outer; i++) {
    int64_t off = i * inner * reduce;
    for (int64_t j = 0; j < inner; j++) {
      float max = 0, grad_sum = 0;
      for (int64_t k = 0; k < reduce; k++) {
        int64_t idx = j + k * inner + off;
        float item = arr[idx];
        grad_sum += grad[idx];
        if (k == 0 || item > max) max = item;
      }
      float exp_sum = 0;
      for (int64_t k = 0; k < reduce; k++) exp_sum += expf(arr[j + k * inner + off] - max);
      float log_sum = logf(exp_sum) + max;
      for (int64_t k = 0; k < reduce; k++) {
        int64_t idx = j + k * inner + off;
        z[idx] = grad[idx] - grad_sum * expf(arr[idx] - log_sum);
      }
    }
  }
  store_f(dtype, out, total, zo);
  free(ao);
  free(go);
}

/* ---- clamp (BackendCPU.swift:704-782): Swift.min / Swift.max on Float or Int64 ----
 * Swift.max(x, y) returns y unless x > y ... precisely: max(x, y) = y >= x ? y : x and
 * min(x, y) = y < x ? y : x (stdlib Algorithm.swift), which fixes what a NaN does. */

static float swift_maxf(float x, float y) { return y >= x ? y : x; }
static float swift_minf(float x, float y) { return y < x ? y : x; }
static int64_t swift_maxi(int64_t x, int64_t y) { return y >= x ? y : x; }
static int64_t swift_mini(int64_t x, int64_t y) { return y < x ? y : x; }

void ref_clamp(int dtype, const void* a, const ref_strides* as, const void* lo, const ref_strides* ls,
               const void* hi, const ref_strides* hs, void* out) {
  int64_t n = shape_product(as);
  if (dtype == REF_I64) {
    const int64_t *x = (const int64_t*)a, *l = (const int64_t*)lo, *h = (const int64_t*)hi;
    int64_t* z = (int64_t*)out;
    for (int64_t i = 0; i < n; i++) {
      int64_t v = x[ref_strides_index(as, i)];
      if (l) v = swift_maxi(l[ref_strides_index(ls, i)], v);
      if (h) v = swift_mini(h[ref_strides_index(hs, i)], v);
      z[i] = v;
    }
    return;
  }
  float *xo, *lo_o = NULL, *hi_o = NULL, *zo;
  const float* x = load_f(dtype, a, (size_t)data_count(as), &xo);
  const float* l = lo ? load_f(dtype, lo, (size_t)data_count(ls), &lo_o) : NULL;
  const float* h = hi ? load_f(dtype, hi, (size_t)data_count(hs), &hi_o) : NULL;
  float* z = out_f(dtype, out, (size_t)n, &zo);
  for (int64_t i = 0; i < n; i++) {
    float v = x[ref_strides_index(as, i)];
    if (l) v = swift_maxf(l[ref_strides_index(ls, i)], v);
    if (h) v = swift_minf(h[ref_strides_index(hs, i)], v);
    z[i] = v;
  }
  store_f(dtype, out, (size_t)n, zo);
  free(xo);
  free(lo_o);
  free(hi_o);
}

/* ---- when (BackendCPU.swift:1190-1220) ---- */

void ref_when(int dtype, const uint8_t* mask, const ref_strides* ms, const void* a,
              const ref_strides* as, const void* b, const ref_strides* bs, void* out) {
  int64_t n = shape_product(ms);
  size_t el = dtype_size(dtype);
  for (int64_t i = 0; i < n; i++) {
    if (mask[ref_strides_index(ms, i)] != 0)
      memcpy((char*)out + el * i, (const char*)a + el * ref_strides_index(as, i), el);
    else
      memcpy((char*)out + el * i, (const char*)b + el * ref_strides_index(bs, i), el);
  }
}

/* ---- matmul / batchedMatmul (BackendCPU.swift:1222-1313) ----
 *
 * The reference runs i, j, k loops with acc = acc + a*b in Float (or Int64) and
 * one store per output. ref_matmul computes every output with that same k
 * order but iterates i, k, j over a [K, N] copy of B so that the inner loop is
 * contiguous: each acc[j] still sees k = 0, 1, 2 ... in turn, so results are
 * bit-identical to the reference loop (ref_matmul_rows below is the literal
 * loop; tests check the two agree bit for bit). fp32 without transposes goes
 * through vDSP_mmul in the reference (order unspecified). */

__attribute__((target_clones("avx2", "default"))) static void matmul_rows_ikj(
    const float* a, int trans_a, const float* bkn, int64_t rows, int64_t inner, int64_t cols,
    int64_t i0, int64_t i1, float* c, int trans_out) {
  float* acc = (float*)malloc((size_t)(cols ? cols : 1) * sizeof(float));
  for (int64_t i = i0; i < i1; i++) {
    for (int64_t j = 0; j < cols; j++) acc[j] = 0.0f;
    for (int64_t k = 0; k < inner; k++) {
      float av = trans_a ? a[i + k * rows] : a[i * inner + k];
      const float* brow = bkn + k * cols;
      for (int64_t j = 0; j < cols; j++) acc[j] = acc[j] + av * brow[j];
    }
    if (trans_out)
      for (int64_t j = 0; j < cols; j++) c[i + j * rows] = acc[j];
    else
      memcpy(c + i * cols, acc, (size_t)cols * sizeof(float));
  }
  free(acc);
}

void ref_matmul(int dtype, int64_t batch, const void* a, int trans_a, const void* b, int trans_b,
                int trans_out, int64_t rows, int64_t inner, int64_t cols, void* out) {
  size_t a_count = (size_t)(rows * inner), b_count = (size_t)(inner * cols),
         c_count = (size_t)(rows * cols);
  if (dtype == REF_I64) {
    const int64_t* x = (const int64_t*)a;
    const int64_t* y = (const int64_t*)b;
    int64_t* z = (int64_t*)out;
    for (int64_t m = 0; m < batch; m++)
      for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < cols; j++) {
          int64_t acc = 0;
          for (int64_t k = 0; k < inner; k++) {
            int64_t av = trans_a ? x[m * a_count + i + k * rows] : x[m * a_count + i * inner + k];
            int64_t bv = trans_b ? y[m * b_count + k + j * inner] : y[m * b_count + k * cols + j];
            acc = binop_i(REF_ADD, acc, binop_i(REF_MUL, av, bv));
          }
          if (trans_out)
            z[m * c_count + i + j * rows] = acc;
          else
            z[m * c_count + i * cols + j] = acc;
        }
    return;
  }
  float *ao, *bo, *zo;
  const float* x = load_f(dtype, a, (size_t)batch * a_count, &ao);
  const float* y = load_f(dtype, b, (size_t)batch * b_count, &bo);
  float* z = out_f(dtype, out, (size_t)batch * c_count, &zo);
  float* bt = trans_b ? (float*)malloc((b_count ? b_count : 1) * sizeof(float)) : NULL;
  for (int64_t m = 0; m < batch; m++) {
    const float* bm = y + m * b_count;
    if (trans_b) {
      /* stored [cols, inner]; element (k, j) at j * inner + k */
#pragma omp parallel for num_threads(nthreads()) if (b_count > 65536)
      for (int64_t k = 0; k < inner; k++)
        for (int64_t j = 0; j < cols; j++) bt[k * cols + j] = bm[j * inner + k];
      bm = bt;
    }
    int nt = nthreads();
    if (c_count * (size_t)inner < (1u << 20)) nt = 1;
#pragma omp parallel for num_threads(nt) schedule(dynamic, 1)
    for (int64_t i0 = 0; i0 < rows; i0 += 16) {
      int64_t i1 = i0 + 16 < rows ? i0 + 16 : rows;
      matmul_rows_ikj(x + m * a_count, trans_a, bm, rows, inner, cols, i0, i1, z + m * c_count,
                      trans_out);
    }
  }
  free(bt);
  store_f(dtype, out, (size_t)batch * c_count, zo);
  free(ao);
  free(bo);
}

/* The literal reference loop (:1260-1304) on rows [row0, row1) of one matrix, one
 * thread, including the whole-buffer fp16 -> Float staging of readBuffer (:2018-2030).
 * This is what the CPU baseline times; out_f32 receives the Float accumulators
 * ((row1-row0) x cols, row-major) before any rounding to the output dtype. */
void ref_matmul_rows(int dtype, const void* a, int trans_a, const void* b, int trans_b,
                     int64_t rows, int64_t inner, int64_t cols, int64_t row0, int64_t row1,
                     float* out_f32) {
  float *ao, *bo;
  int saved = g_threads;
  g_threads = 1;
  const float* arr_a = load_f(dtype, a, (size_t)(rows * inner), &ao);
  const float* arr_b = load_f(dtype, b, (size_t)(inner * cols), &bo);
  g_threads = saved;
  for (int64_t i = row0; i < row1; i++)
    for (int64_t j = 0; j < cols; j++) {
      float acc = 0.0f;
      for (int64_t k = 0; k < inner; k++) {
        float av = trans_a ? arr_a[i + k * rows] : arr_a[i * inner + k];
        float bv = trans_b ? arr_b[k + j * inner] : arr_b[k * cols + j];
        acc = acc + av * bv;
      }
      out_f32[(i - row0) * cols + j] = acc;
    }
  free(ao);
  free(bo);
}

/* ---- triangular (BackendCPU.swift:1315-1348) ---- */

void ref_triangular(int dtype, const void* in, void* out, int64_t batch, int64_t rows,
                    int64_t cols, int upper, int64_t offset) {
  size_t el = dtype_size(dtype);
  memset(out, 0, el * (size_t)(rows * cols * batch));
  for (int64_t i = 0; i < batch; i++)
    for (int64_t j = 0; j < rows; j++) {
      const char* row_in = (const char*)in + (i * rows + j) * cols * (int64_t)el;
      char* row_out = (char*)out + (i * rows + j) * cols * (int64_t)el;
      if (upper) {
        int64_t n = cols - j - offset;
        if (n > cols) n = cols;
        if (n > 0) {
          int64_t skip = cols - n;
          memcpy(row_out + skip * (int64_t)el, row_in + skip * (int64_t)el, (size_t)n * el);
        }
      } else {
        int64_t n = (j + 1) + offset;
        if (n > cols) n = cols;
        if (n > 0) memcpy(row_out, row_in, (size_t)n * el);
      }
    }
}

/* ---- constant (BackendCPU.swift:1796-1815) ---- */

void ref_fill(int dtype, float vf, int64_t vi, void* out, size_t count) {
  switch (dtype) {
    case REF_I64:
      for (size_t i = 0; i < count; i++) ((int64_t*)out)[i] = vi;
      break;
    case REF_BOOL:
      for (size_t i = 0; i < count; i++) ((uint8_t*)out)[i] = vf == 0 ? 0 : 1;
      break;
    case REF_F16: {
      uint16_t h = ref_f32_to_f16(vf);
      for (size_t i = 0; i < count; i++) ((uint16_t*)out)[i] = h;
      break;
    }
    default:
      for (size_t i = 0; i < count; i++) ((float*)out)[i] = vf;
      break;
  }
}

/* ---- axisPermutation (BackendCPU.swift:1831-1849) ---- */

void ref_axis_permutation(const int64_t* perm, const int64_t* shape, int ndim, int64_t* out) {
  int64_t old_strides[REF_MAX_DIMS], permuted[REF_MAX_DIMS], new_shape[REF_MAX_DIMS],
      new_strides[REF_MAX_DIMS];
  int64_t total = 1;
  for (int d = ndim - 1; d >= 0; d--) {
    old_strides[d] = total;
    total *= shape[d];
  }
  for (int d = 0; d < ndim; d++) {
    permuted[d] = old_strides[perm[d]];
    new_shape[d] = shape[perm[d]];
  }
  int64_t acc = 1;
  for (int d = ndim - 1; d >= 0; d--) {
    new_strides[d] = acc;
    acc *= new_shape[d];
  }
  for (int64_t i = 0; i < total; i++) {
    int64_t flat = 0;
    for (int d = 0; d < ndim; d++) flat += permuted[d] * ((i / new_strides[d]) % new_shape[d]);
    out[i] = flat;
  }
}

/* ---- normalize: the base-class composition (Backend.swift:265-327), op by op, so
 * that every intermediate is rounded to the tensor dtype exactly as the composed
 * backend calls round it ---- */

void ref_normalize(int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
                   int64_t inner, float eps) {
  size_t el = dtype_size(dtype);
  size_t full = (size_t)(outer * reduce * inner), red = (size_t)(outer * inner);
  ref_strides fs = {3, 0, {outer, reduce, inner}, {reduce * inner, inner, 1}};
  ref_strides rs = {3, 0, {outer, reduce, inner}, {inner, 0, 1}};
  void* t_red = malloc((red ? red : 1) * el);
  void* mean = malloc((red ? red : 1) * el);
  void* centered = malloc((full ? full : 1) * el);
  void* sq = malloc((full ? full : 1) * el);
  void* var = malloc((red ? red : 1) * el);
  void* norm = malloc((red ? red : 1) * el);
  float inv_n = 1.0f / (float)reduce;
  ref_reduce(REF_SUM, dtype, in, t_red, outer, reduce, inner);
  ref_binary_op_scalar(REF_MUL, dtype, t_red, inv_n, 0, 0, mean, red);
  ref_binary_op(REF_SUB, dtype, in, &fs, mean, &rs, centered);
  ref_pow(dtype, centered, 2.0f, 1.0f, 2, 1, NULL, sq, full);
  ref_reduce(REF_SUM, dtype, sq, t_red, outer, reduce, inner);
  ref_binary_op_scalar(REF_MUL, dtype, t_red, inv_n, 0, 0, var, red);
  ref_binary_op_scalar(REF_ADD, dtype, var, eps, 0, 0, t_red, red);
  ref_pow(dtype, t_red, -0.5f, 1.0f, 0, 1, NULL, norm, red);
  ref_binary_op(REF_MUL, dtype, centered, &fs, norm, &rs, out);
  free(t_red);
  free(mean);
  free(centered);
  free(sq);
  free(var);
  free(norm);
}

/* ---- concat (BackendCPU.swift:1768-1794) ---- */

void ref_concat(int dtype, const void* const* inputs, const int64_t* inner_counts, int n_inputs,
                int64_t outer, void* out) {
  size_t el = dtype_size(dtype);
  size_t off = 0;
  for (int64_t i = 0; i < outer; i++)
    for (int t = 0; t < n_inputs; t++) {
      size_t chunk = (size_t)inner_counts[t] * el;
      memcpy((char*)out + off, (const char*)inputs[t] + (size_t)i * chunk, chunk);
      off += chunk;
    }
}
