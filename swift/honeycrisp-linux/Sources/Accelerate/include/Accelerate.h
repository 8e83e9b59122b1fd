/*
 * Accelerate - Linux stand-in for the part of Apple's Accelerate framework that Honeycrisp's
 * CPUBackend calls, so that `import Accelerate` resolves on Linux and the reference sources stay
 * untouched. A SwiftPM C target (module name "Accelerate").
 *
 * Every symbol the reference uses, with the operand order of its call site
 * (Sources/Honeycrisp/BackendCPU.swift:284-2066, TensorElement.swift:262-338):
 *
 *   vDSP_vadd(A,1,B,1,C,1,n)       C = A + B                         BackendCPU.swift:284
 *   vDSP_vmul(A,1,B,1,C,1,n)       C = A * B (C may alias A)         :286 :666 :680
 *   vDSP_vsub(B,1,A,1,C,1,n)       C = A - B  (second minus first)   :290
 *   vDSP_vdiv(B,1,A,1,C,1,n)       C = A / B  (second over first)    :288
 *   vDSP_vsadd(A,1,&s,C,1,n)       C = A + s                         :337 :378
 *   vDSP_vsmul(A,1,&s,C,1,n)       C = A * s (C may alias A)         :339 :380 :668 :673
 *   vDSP_svdiv(&s,A,1,C,1,n)       C = s / A                         :382 :671
 *   vDSP_vsmsa(A,1,&m,&a,C,1,n)    C = A * m + a                     :384
 *   vDSP_vma(A,1,B,1,C,1,D,1,n)    D = A * B + C                     :464
 *   vDSP_vam(A,1,B,1,C,1,D,1,n)    D = (A + B) * C                   :512
 *   vDSP_sve(A,stride,&out,n)      out = sum of A[i * stride]        :802
 *   vDSP_mmul(A,1,B,1,C,1,M,N,P)   row-major C[M x N] = A[M x P] B[P x N]   :1256
 *   vDSP_mtrans(A,1,C,1,M,N)       C[M x N] = transpose of A[N x M]  :2066
 *   vImageConvert_PlanarFtoPlanar16F / Planar16FtoPlanarF            TensorElement.swift:273, :334
 *   sgeqrf_, sorgqr_, sgesvd_ (LAPACK, column-major, __LAPACK_int)   BackendCPU.swift:1401-1546
 *
 * Arithmetic is plain IEEE single precision, one rounding per operation (the file is built with
 * -ffp-contract=off: a*b+c is two roundings, as vDSP documents for vma / vsmsa / vam). vDSP_sve
 * adds sequentially. vDSP_mmul goes to a cblas_sgemm found at run time (OpenBLAS under its usual
 * names, or the library named by HC_ACCELERATE_BLAS), else to a built-in blocked loop; the LAPACK
 * entry points forward to the same library and report an illegal-argument code when there is none.
 */
#ifndef HC_ACCELERATE_SHIM_H
#define HC_ACCELERATE_SHIM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef unsigned long vDSP_Length;
typedef long vDSP_Stride;

void vDSP_vadd(const float* a, vDSP_Stride ia, const float* b, vDSP_Stride ib, float* c, vDSP_Stride ic, vDSP_Length n);
void vDSP_vmul(const float* a, vDSP_Stride ia, const float* b, vDSP_Stride ib, float* c, vDSP_Stride ic, vDSP_Length n);
void vDSP_vsub(const float* b, vDSP_Stride ib, const float* a, vDSP_Stride ia, float* c, vDSP_Stride ic, vDSP_Length n);
void vDSP_vdiv(const float* b, vDSP_Stride ib, const float* a, vDSP_Stride ia, float* c, vDSP_Stride ic, vDSP_Length n);
void vDSP_vsadd(const float* a, vDSP_Stride ia, const float* s, float* c, vDSP_Stride ic, vDSP_Length n);
void vDSP_vsmul(const float* a, vDSP_Stride ia, const float* s, float* c, vDSP_Stride ic, vDSP_Length n);
void vDSP_svdiv(const float* s, const float* a, vDSP_Stride ia, float* c, vDSP_Stride ic, vDSP_Length n);
void vDSP_vsmsa(const float* a, vDSP_Stride ia, const float* m, const float* add, float* c, vDSP_Stride ic,
                vDSP_Length n);
void vDSP_vma(const float* a, vDSP_Stride ia, const float* b, vDSP_Stride ib, const float* c, vDSP_Stride ic,
              float* d, vDSP_Stride id, vDSP_Length n);
void vDSP_vam(const float* a, vDSP_Stride ia, const float* b, vDSP_Stride ib, const float* c, vDSP_Stride ic,
              float* d, vDSP_Stride id, vDSP_Length n);
void vDSP_sve(const float* a, vDSP_Stride ia, float* out, vDSP_Length n);
void vDSP_mmul(const float* a, vDSP_Stride ia, const float* b, vDSP_Stride ib, float* c, vDSP_Stride ic,
               vDSP_Length m, vDSP_Length n, vDSP_Length p);
void vDSP_mtrans(const float* a, vDSP_Stride ia, float* c, vDSP_Stride ic, vDSP_Length m, vDSP_Length n);

/* vImage: planar float <-> planar IEEE binary16, round to nearest even, overflow to infinity,
 * subnormals kept, NaN stays NaN. */
typedef unsigned long vImagePixelCount;
typedef long vImage_Error;
typedef uint32_t vImage_Flags;
typedef struct vImage_Buffer {
  void* data;
  vImagePixelCount height;
  vImagePixelCount width;
  size_t rowBytes;
} vImage_Buffer;
enum { kvImageNoError = 0, kvImageBufferSizeMismatch = -21774, kvImageNullPointerArgument = -21772 };
vImage_Error vImageConvert_PlanarFtoPlanar16F(const vImage_Buffer* src, const vImage_Buffer* dest, vImage_Flags flags);
vImage_Error vImageConvert_Planar16FtoPlanarF(const vImage_Buffer* src, const vImage_Buffer* dest, vImage_Flags flags);

/* LAPACK with the ACCELERATE_NEW_LAPACK interface (32-bit integers, no hidden string lengths in
 * the prototypes), column-major. */
typedef int32_t __LAPACK_int;
void sgeqrf_(const __LAPACK_int* m, const __LAPACK_int* n, float* a, const __LAPACK_int* lda, float* tau, float* work,
             const __LAPACK_int* lwork, __LAPACK_int* info);
void sorgqr_(const __LAPACK_int* m, const __LAPACK_int* n, const __LAPACK_int* k, float* a, const __LAPACK_int* lda,
             const float* tau, float* work, const __LAPACK_int* lwork, __LAPACK_int* info);
void sgesvd_(const char* jobu, const char* jobvt, const __LAPACK_int* m, const __LAPACK_int* n, float* a,
             const __LAPACK_int* lda, float* s, float* u, const __LAPACK_int* ldu, float* vt, const __LAPACK_int* ldvt,
             float* work, const __LAPACK_int* lwork, __LAPACK_int* info);

/* Which sgemm vDSP_mmul runs on: the path of the library it found and the symbol it bound, or
 * "built-in". For benchmark reports. */
const char* hc_accelerate_blas_backend(void);
/* Threads of the bound BLAS (1 for the built-in loop, 0 if the library does not say). */
int hc_accelerate_blas_threads(void);

#ifdef __cplusplus
}
#endif
#endif /* HC_ACCELERATE_SHIM_H */
