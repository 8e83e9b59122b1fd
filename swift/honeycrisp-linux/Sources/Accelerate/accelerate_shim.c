/* Implementation of the Accelerate stand-in declared in include/Accelerate.h.
 * Build: cc -O2 -fPIC -ffp-contract=off -fno-fast-math accelerate_shim.c -ldl -lm
 * (SwiftPM: a C target; -ffp-contract=off through cSettings unsafeFlags). */
#include "include/Accelerate.h"

#include <dlfcn.h>
#include <math.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ---- element-wise vDSP (BackendCPU.swift:284-512, 666-680) ----
 * The loops run forwards, element by element, so an output that aliases an input at the same
 * stride (vDSP_vmul(z,1,scales,1,z,1,n), :680) reads each element before it is overwritten. */

void vDSP_vadd(const float* a, vDSP_Stride ia, const float* b, vDSP_Stride ib, float* c, vDSP_Stride ic, vDSP_Length n) {
  for (vDSP_Length i = 0; i < n; i++) c[(long)i * ic] = a[(long)i * ia] + b[(long)i * ib];
}

void vDSP_vmul(const float* a, vDSP_Stride ia, const float* b, vDSP_Stride ib, float* c, vDSP_Stride ic, vDSP_Length n) {
  for (vDSP_Length i = 0; i < n; i++) c[(long)i * ic] = a[(long)i * ia] * b[(long)i * ib];
}

/* C = A - B with B passed FIRST (Apple's operand order; vDSP_vsub(y,1,x,1,z,...) is z = x - y). */
void vDSP_vsub(const float* b, vDSP_Stride ib, const float* a, vDSP_Stride ia, float* c, vDSP_Stride ic, vDSP_Length n) {
  for (vDSP_Length i = 0; i < n; i++) c[(long)i * ic] = a[(long)i * ia] - b[(long)i * ib];
}

/* C = A / B with B passed FIRST (vDSP_vdiv(y,1,x,1,z,...) is z = x / y). */
void vDSP_vdiv(const float* b, vDSP_Stride ib, const float* a, vDSP_Stride ia, float* c, vDSP_Stride ic, vDSP_Length n) {
  for (vDSP_Length i = 0; i < n; i++) c[(long)i * ic] = a[(long)i * ia] / b[(long)i * ib];
}

void vDSP_vsadd(const float* a, vDSP_Stride ia, const float* s, float* c, vDSP_Stride ic, vDSP_Length n) {
  const float v = *s;
  for (vDSP_Length i = 0; i < n; i++) c[(long)i * ic] = a[(long)i * ia] + v;
}

void vDSP_vsmul(const float* a, vDSP_Stride ia, const float* s, float* c, vDSP_Stride ic, vDSP_Length n) {
  const float v = *s;
  for (vDSP_Length i = 0; i < n; i++) c[(long)i * ic] = a[(long)i * ia] * v;
}

void vDSP_svdiv(const float* s, const float* a, vDSP_Stride ia, float* c, vDSP_Stride ic, vDSP_Length n) {
  const float v = *s;
  for (vDSP_Length i = 0; i < n; i++) c[(long)i * ic] = v / a[(long)i * ia];
}

void vDSP_vsmsa(const float* a, vDSP_Stride ia, const float* m, const float* add, float* c, vDSP_Stride ic,
                vDSP_Length n) {
  const float mv = *m, av = *add;
  for (vDSP_Length i = 0; i < n; i++) {
    const float prod = a[(long)i * ia] * mv;
    c[(long)i * ic] = prod + av;
  }
}

void vDSP_vma(const float* a, vDSP_Stride ia, const float* b, vDSP_Stride ib, const float* c, vDSP_Stride ic,
              float* d, vDSP_Stride id, vDSP_Length n) {
  for (vDSP_Length i = 0; i < n; i++) {
    const float prod = a[(long)i * ia] * b[(long)i * ib];
    d[(long)i * id] = prod + c[(long)i * ic];
  }
}

void vDSP_vam(const float* a, vDSP_Stride ia, const float* b, vDSP_Stride ib, const float* c, vDSP_Stride ic,
              float* d, vDSP_Stride id, vDSP_Length n) {
  for (vDSP_Length i = 0; i < n; i++) {
    const float sum = a[(long)i * ia] + b[(long)i * ib];
    d[(long)i * id] = sum * c[(long)i * ic];
  }
}

void vDSP_sve(const float* a, vDSP_Stride ia, float* out, vDSP_Length n) {
  float sum = 0.0f;
  for (vDSP_Length i = 0; i < n; i++) sum += a[(long)i * ia];
  *out = sum;
}

void vDSP_mtrans(const float* a, vDSP_Stride ia, float* c, vDSP_Stride ic, vDSP_Length m, vDSP_Length n) {
  /* C is m x n, A is n x m */
  for (vDSP_Length i = 0; i < m; i++)
    for (vDSP_Length j = 0; j < n; j++) c[(long)(i * n + j) * ic] = a[(long)(j * m + i) * ia];
}

/* ---- BLAS / LAPACK found at run time ---- */

enum { CblasRowMajor = 101, CblasNoTrans = 111 };
typedef void (*sgemm32_fn)(int, int, int, int, int, int, float, const float*, int, const float*, int, float, float*, int);
typedef void (*sgemm64_fn)(int, int, int, int64_t, int64_t, int64_t, float, const float*, int64_t, const float*,
                           int64_t, float, float*, int64_t);

static pthread_once_t g_once = PTHREAD_ONCE_INIT;
static void* g_lib = NULL;
static sgemm32_fn g_sgemm32 = NULL;
static sgemm64_fn g_sgemm64 = NULL;
static int g_lapack_ilp64 = 0;
static void *g_sgeqrf = NULL, *g_sorgqr = NULL, *g_sgesvd = NULL;
static int (*g_get_threads)(void) = NULL;
static char g_backend[512] = "built-in";

static void* first_symbol(void* lib, const char* const* names, const char** which) {
  for (int i = 0; names[i]; i++) {
    void* p = dlsym(lib, names[i]);
    if (p) {
      if (which) *which = names[i];
      return p;
    }
  }
  return NULL;
}

static void bind_library(void) {
  static const char* const candidates[] = {"libopenblas.so.0", "libopenblas.so", "libopenblas64_.so.0",
                                           "libblas.so.3",     "libcblas.so.3",  NULL};
  const char* forced = getenv("HC_ACCELERATE_BLAS");
  if (forced && strcmp(forced, "builtin") == 0) return;
  const char* path = NULL;
  if (forced && *forced) {
    g_lib = dlopen(forced, RTLD_NOW | RTLD_LOCAL);
    path = forced;
    if (!g_lib) fprintf(stderr, "Accelerate shim: cannot load HC_ACCELERATE_BLAS=%s (%s); using the built-in sgemm\n", forced, dlerror());
  } else {
    for (int i = 0; candidates[i] && !g_lib; i++) {
      g_lib = dlopen(candidates[i], RTLD_NOW | RTLD_LOCAL);
      path = candidates[i];
    }
  }
  if (!g_lib) return;
  /* plain names (LP64), the scipy / numpy wheels' prefixed names, and their ILP64 builds */
  static const char* const gemm32[] = {"cblas_sgemm", "scipy_cblas_sgemm", NULL};
  static const char* const gemm64[] = {"cblas_sgemm64_", "scipy_cblas_sgemm64_", NULL};
  const char* sym = NULL;
  g_sgemm32 = (sgemm32_fn)first_symbol(g_lib, gemm32, &sym);
  if (!g_sgemm32) g_sgemm64 = (sgemm64_fn)first_symbol(g_lib, gemm64, &sym);
  if (g_sgemm32 || g_sgemm64) snprintf(g_backend, sizeof(g_backend), "%s:%s", path, sym);
  static const char* const qrf32[] = {"sgeqrf_", "scipy_sgeqrf_", NULL};
  static const char* const qrf64[] = {"sgeqrf_64_", "scipy_sgeqrf_64_", NULL};
  static const char* const gqr32[] = {"sorgqr_", "scipy_sorgqr_", NULL};
  static const char* const gqr64[] = {"sorgqr_64_", "scipy_sorgqr_64_", NULL};
  static const char* const svd32[] = {"sgesvd_", "scipy_sgesvd_", NULL};
  static const char* const svd64[] = {"sgesvd_64_", "scipy_sgesvd_64_", NULL};
  g_sgeqrf = first_symbol(g_lib, qrf32, NULL);
  if (g_sgeqrf && (void*)g_sgeqrf != (void*)sgeqrf_) {
    g_sorgqr = first_symbol(g_lib, gqr32, NULL);
    g_sgesvd = first_symbol(g_lib, svd32, NULL);
  } else {
    g_sgeqrf = first_symbol(g_lib, qrf64, NULL);
    g_sorgqr = first_symbol(g_lib, gqr64, NULL);
    g_sgesvd = first_symbol(g_lib, svd64, NULL);
    g_lapack_ilp64 = g_sgeqrf != NULL;
  }
  static const char* const threads[] = {"openblas_get_num_threads", "scipy_openblas_get_num_threads",
                                        "openblas_get_num_threads64_", "scipy_openblas_get_num_threads64_", NULL};
  g_get_threads = (int (*)(void))first_symbol(g_lib, threads, NULL);
}

const char* hc_accelerate_blas_backend(void) {
  pthread_once(&g_once, bind_library);
  return g_backend;
}

int hc_accelerate_blas_threads(void) {
  pthread_once(&g_once, bind_library);
  if (!g_sgemm32 && !g_sgemm64) return 1;
  return g_get_threads ? g_get_threads() : 0;
}

/* Built-in sgemm: row-major C[m x n] = A[m x p] B[p x n], blocked over k and n so that a panel of
 * B stays in cache, inner loop along n (unit stride, vectorisable). */
static void builtin_sgemm(const float* a, const float* b, float* c, size_t m, size_t n, size_t p) {
  enum { KB = 256, NB = 1024 };
  for (size_t i = 0; i < m * n; i++) c[i] = 0.0f;
  for (size_t k0 = 0; k0 < p; k0 += KB) {
    const size_t k1 = k0 + KB < p ? k0 + KB : p;
    for (size_t j0 = 0; j0 < n; j0 += NB) {
      const size_t j1 = j0 + NB < n ? j0 + NB : n;
      for (size_t i = 0; i < m; i++) {
        float* crow = c + i * n;
        for (size_t k = k0; k < k1; k++) {
          const float av = a[i * p + k];
          const float* brow = b + k * n;
          for (size_t j = j0; j < j1; j++) crow[j] += av * brow[j];
        }
      }
    }
  }
}

void vDSP_mmul(const float* a, vDSP_Stride ia, const float* b, vDSP_Stride ib, float* c, vDSP_Stride ic,
               vDSP_Length m, vDSP_Length n, vDSP_Length p) {
  if (m == 0 || n == 0) return;
  if (ia != 1 || ib != 1 || ic != 1) {
    /* strided elements: the reference never asks for this (BackendCPU.swift:1256 passes 1, 1, 1) */
    for (vDSP_Length i = 0; i < m; i++)
      for (vDSP_Length j = 0; j < n; j++) {
        float acc = 0.0f;
        for (vDSP_Length k = 0; k < p; k++) acc += a[(long)(i * p + k) * ia] * b[(long)(k * n + j) * ib];
        c[(long)(i * n + j) * ic] = acc;
      }
    return;
  }
  pthread_once(&g_once, bind_library);
  if (p == 0) {
    memset(c, 0, (size_t)m * n * sizeof(float));
  } else if (g_sgemm32 && m <= 0x7fffffff && n <= 0x7fffffff && p <= 0x7fffffff) {
    g_sgemm32(CblasRowMajor, CblasNoTrans, CblasNoTrans, (int)m, (int)n, (int)p, 1.0f, a, (int)p, b, (int)n, 0.0f, c, (int)n);
  } else if (g_sgemm64) {
    g_sgemm64(CblasRowMajor, CblasNoTrans, CblasNoTrans, (int64_t)m, (int64_t)n, (int64_t)p, 1.0f, a, (int64_t)p, b,
              (int64_t)n, 0.0f, c, (int64_t)n);
  } else {
    builtin_sgemm(a, b, c, m, n, p);
  }
}

/* ---- vImage half conversion (TensorElement.swift:262-338) ---- */

static uint16_t f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t absx = x & 0x7fffffffu;
  if (absx > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((absx >> 13) & 0x3ffu)); /* NaN, quiet */
  if (absx >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);                            /* >= 65536: inf */
  if (absx < 0x38800000u) {
    /* below the smallest normal half: the result is a multiple of 2^-24, rounded to nearest even */
    if (absx < 0x33000000u) return (uint16_t)sign; /* < 2^-25 rounds to zero */
    const uint32_t e = absx >> 23;                 /* 102 .. 112 */
    const uint32_t mant = (absx & 0x7fffffu) | 0x800000u;
    const uint32_t shift = 126u - e;               /* 14 .. 24 */
    uint32_t res = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (res & 1u))) res++;
    return (uint16_t)(sign | res);
  }
  uint32_t res = ((absx >> 23) - 112u) << 10 | ((absx & 0x7fffffu) >> 13);
  const uint32_t rem = absx & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (res & 1u))) res++; /* may carry into the exponent, up to inf */
  return (uint16_t)(sign | res);
}

static float f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t e = (h >> 10) & 31u, m = h & 0x3ffu;
  uint32_t bits;
  if (e == 31u) {
    bits = sign | 0x7f800000u | (m << 13);
  } else if (e != 0u) {
    bits = sign | ((e + 112u) << 23) | (m << 13);
  } else if (m == 0u) {
    bits = sign;
  } else {
    int shift = 0;
    uint32_t mm = m;
    while (!(mm & 0x400u)) {
      mm <<= 1;
      shift++;
    }
    bits = sign | ((uint32_t)(113 - shift) << 23) | ((mm & 0x3ffu) << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

vImage_Error vImageConvert_PlanarFtoPlanar16F(const vImage_Buffer* src, const vImage_Buffer* dest, vImage_Flags flags) {
  (void)flags;
  if (!src || !dest) return kvImageNullPointerArgument;
  if (src->height != dest->height || src->width != dest->width) return kvImageBufferSizeMismatch;
  if (src->width && src->height && (!src->data || !dest->data)) return kvImageNullPointerArgument;
  for (vImagePixelCount r = 0; r < src->height; r++) {
    const float* in = (const float*)((const char*)src->data + r * src->rowBytes);
    uint16_t* out = (uint16_t*)((char*)dest->data + r * dest->rowBytes);
    for (vImagePixelCount i = 0; i < src->width; i++) out[i] = f32_to_f16(in[i]);
  }
  return kvImageNoError;
}

vImage_Error vImageConvert_Planar16FtoPlanarF(const vImage_Buffer* src, const vImage_Buffer* dest, vImage_Flags flags) {
  (void)flags;
  if (!src || !dest) return kvImageNullPointerArgument;
  if (src->height != dest->height || src->width != dest->width) return kvImageBufferSizeMismatch;
  if (src->width && src->height && (!src->data || !dest->data)) return kvImageNullPointerArgument;
  for (vImagePixelCount r = 0; r < src->height; r++) {
    const uint16_t* in = (const uint16_t*)((const char*)src->data + r * src->rowBytes);
    float* out = (float*)((char*)dest->data + r * dest->rowBytes);
    for (vImagePixelCount i = 0; i < src->width; i++) out[i] = f16_to_f32(in[i]);
  }
  return kvImageNoError;
}

/* ---- LAPACK forwarding (QR / SVD, BackendCPU.swift:1382-1546) ----
 * Fortran symbols of the bound library: 32-bit integers as they come, or widened for an ILP64
 * build. Character arguments carry a hidden trailing length in the Fortran ABI. Without a LAPACK
 * the calls report info = -1000 (the reference turns a non-zero info into BackendError.lapackError). */

static void no_lapack(const char* name, __LAPACK_int* info) {
  fprintf(stderr, "Accelerate shim: %s needs a LAPACK library (OpenBLAS, or HC_ACCELERATE_BLAS=<path>)\n", name);
  *info = -1000;
}

void sgeqrf_(const __LAPACK_int* m, const __LAPACK_int* n, float* a, const __LAPACK_int* lda, float* tau, float* work,
             const __LAPACK_int* lwork, __LAPACK_int* info) {
  pthread_once(&g_once, bind_library);
  if (!g_sgeqrf) {
    no_lapack("sgeqrf_", info);
    return;
  }
  if (g_lapack_ilp64) {
    int64_t m8 = *m, n8 = *n, lda8 = *lda, lwork8 = *lwork, info8 = 0;
    ((void (*)(int64_t*, int64_t*, float*, int64_t*, float*, float*, int64_t*, int64_t*))g_sgeqrf)(&m8, &n8, a, &lda8, tau,
                                                                                                   work, &lwork8, &info8);
    *info = (__LAPACK_int)info8;
  } else {
    ((void (*)(const int32_t*, const int32_t*, float*, const int32_t*, float*, float*, const int32_t*, int32_t*))g_sgeqrf)(
        m, n, a, lda, tau, work, lwork, info);
  }
}

void sorgqr_(const __LAPACK_int* m, const __LAPACK_int* n, const __LAPACK_int* k, float* a, const __LAPACK_int* lda,
             const float* tau, float* work, const __LAPACK_int* lwork, __LAPACK_int* info) {
  pthread_once(&g_once, bind_library);
  if (!g_sorgqr) {
    no_lapack("sorgqr_", info);
    return;
  }
  if (g_lapack_ilp64) {
    int64_t m8 = *m, n8 = *n, k8 = *k, lda8 = *lda, lwork8 = *lwork, info8 = 0;
    ((void (*)(int64_t*, int64_t*, int64_t*, float*, int64_t*, const float*, float*, int64_t*, int64_t*))g_sorgqr)(
        &m8, &n8, &k8, a, &lda8, tau, work, &lwork8, &info8);
    *info = (__LAPACK_int)info8;
  } else {
    ((void (*)(const int32_t*, const int32_t*, const int32_t*, float*, const int32_t*, const float*, float*,
               const int32_t*, int32_t*))g_sorgqr)(m, n, k, a, lda, tau, work, lwork, info);
  }
}

void sgesvd_(const char* jobu, const char* jobvt, const __LAPACK_int* m, const __LAPACK_int* n, float* a,
             const __LAPACK_int* lda, float* s, float* u, const __LAPACK_int* ldu, float* vt, const __LAPACK_int* ldvt,
             float* work, const __LAPACK_int* lwork, __LAPACK_int* info) {
  pthread_once(&g_once, bind_library);
  if (!g_sgesvd) {
    no_lapack("sgesvd_", info);
    return;
  }
  if (g_lapack_ilp64) {
    int64_t m8 = *m, n8 = *n, lda8 = *lda, ldu8 = *ldu, ldvt8 = *ldvt, lwork8 = *lwork, info8 = 0;
    ((void (*)(const char*, const char*, int64_t*, int64_t*, float*, int64_t*, float*, float*, int64_t*, float*,
               int64_t*, float*, int64_t*, int64_t*, size_t, size_t))g_sgesvd)(jobu, jobvt, &m8, &n8, a, &lda8, s, u, &ldu8,
                                                                               vt, &ldvt8, work, &lwork8, &info8, 1, 1);
    *info = (__LAPACK_int)info8;
  } else {
    ((void (*)(const char*, const char*, const int32_t*, const int32_t*, float*, const int32_t*, float*, float*,
               const int32_t*, float*, const int32_t*, float*, const int32_t*, int32_t*, size_t, size_t))g_sgesvd)(
        jobu, jobvt, m, n, a, lda, s, u, ldu, vt, ldvt, work, lwork, info, 1, 1);
  }
}
