/*
 * TEST INFRASTRUCTURE ONLY - never shipped, never on the product path.
 *
 * CPU restatement of the reference CPUBackend arithmetic for the ops the HIP
 * backend accelerates. Each function names the reference lines it follows
 * (paths relative to the reference checkout, Sources/Honeycrisp/...).
 *
 * Only tests, the smoke check and the bench's cpu_baseline leg may link this.
 *
 * How each function is pinned (besides being compared with the GPU):
 *   matmul            reference known answers (BackendTests.swift:684-725,
 *                     769-783), batched == per-matrix invariant (:728-767),
 *                     numpy float64 product on random inputs
 *   binary ops        testAdd/Sub/Mul/Div/Mod vectors (:86-152, :221-252),
 *                     implicit == explicit broadcast (:1461-1502), brute-force
 *                     stride map against numpy broadcasting
 *   elemwise / pow    golden tables (:1074-1232), closed forms via numpy/libm
 *   reduce sum/prod   testSum vectors (:335-434), numpy sums
 *   argmax / argmin   testMinMax (:1325-1362); tie and NaN rules have no
 *                     reference vector and are pinned by hand-derived cases
 *                     from BackendCPU.swift:848-877 (strict compare from k=0)
 *   gather / permute  testGather (:585-682), testIndexing 5-D permutations
 *                     (:991-1029), numpy take/transposition
 *   logSoftmax        3x5 golden (:1552-1610), scipy.special.log_softmax
 *   cast              testCast (:70-84), numpy float16 conversion (all 65536
 *                     half patterns, and random float32 -> half)
 *   mulAdd / addMul   fused == composed (:154-191)
 *   normalize         fused == composed formula (:193-219), numpy two-pass
 *   scatter           input gradients of testGather (:585-650) and the direct scatter
 *                     permutation (:626-633); numpy np.add.at on random indices
 *   logSoftmaxGrad    3x5 gradient goldens for both axes (:1552-1610); closed form
 *                     g - sum(g) * softmax(x) in float64; rows of the result sum to ~0
 *                     when weighted appropriately (sum_k out = sum(g) * (1 - 1) = 0)
 *   clamp             testClamp (:1235-1323), numpy clip / minimum / maximum
 *   cumulative ops    testCumulativeSum / testCumulativeProd vectors (:466-524), numpy cumsum /
 *                     cumprod incl. exclusive and reversed forms
 *   argsort           testArgsort (:526-564) incl. its stable-order vectors, numpy stable argsort
 *   bitwiseOp         testBitwise (:312-333), numpy bitwise ops on int64 / bool / half bits
 */
#ifndef HC_ORACLE_CPU_REF_H
#define HC_ORACLE_CPU_REF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Tensor.DType order (Tensor.swift:24-28). */
enum { REF_I64 = 0, REF_BOOL = 1, REF_F16 = 2, REF_F32 = 3 };
/* NumericBinaryOp order (BinaryOps.swift:2-8). */
enum { REF_ADD = 0, REF_MUL = 1, REF_SUB = 2, REF_DIV = 3, REF_MOD = 4 };
/* ReduceOp order (ReduceRepeat.swift:53-58). */
enum { REF_SUM = 0, REF_PROD = 1, REF_ARGMAX = 2, REF_ARGMIN = 3 };
/* ComparisonOp order (Comparison.swift:4-10). */
enum { REF_EQ = 0, REF_NE = 1, REF_LT = 2, REF_LE = 3, REF_GT = 4, REF_GE = 5 };
/* ElemwiseOp order (Elemwise.swift:13-43). */
enum {
  REF_SIN = 0, REF_COS, REF_MINUS_SIN, REF_TAN, REF_TAN_GRAD, REF_ATAN, REF_ATAN_GRAD,
  REF_ACOS, REF_ACOS_GRAD, REF_ASIN, REF_ASIN_GRAD, REF_EXP, REF_LOG, REF_RECIP,
  REF_SIGMOID, REF_SIGMOID_GRAD, REF_RELU, REF_RELU_GRAD, REF_ABS, REF_ABS_GRAD,
  REF_GELU_APPROX, REF_GELU_APPROX_GRAD, REF_GELU_EXACT, REF_GELU_EXACT_GRAD,
  REF_ERF, REF_ERF_GRAD, REF_FLOOR, REF_CEIL, REF_ROUND, REF_ELEMWISE_COUNT
};

#define REF_MAX_DIMS 8

/* BroadcastStrides (Broadcast.swift:9-30): virtual shape + data strides. */
typedef struct {
  uint32_t ndim;
  uint32_t reserved;
  int64_t shape[REF_MAX_DIMS];
  int64_t strides[REF_MAX_DIMS];
} ref_strides;

void ref_set_threads(int n);

uint16_t ref_f32_to_f16(float f);
float ref_f16_to_f32(uint16_t h);
void ref_f32_to_f16_n(const float* in, uint16_t* out, size_t n);
void ref_f16_to_f32_n(const uint16_t* in, float* out, size_t n);

int64_t ref_strides_index(const ref_strides* s, int64_t i);

void ref_broadcast(int dtype, const void* a, const ref_strides* as, void* out);
void ref_binary_op(int op, int dtype, const void* a, const ref_strides* as, const void* b,
                   const ref_strides* bs, void* out);
void ref_binary_op_scalar(int op, int dtype, const void* a, float sf, int64_t si,
                          int scalar_first, void* out, size_t count);
void ref_mul_add(int dtype, const void* in, const ref_strides* is, const void* coeff,
                 const ref_strides* cs, const void* bias, const ref_strides* bs, void* out);
void ref_add_mul(int dtype, const void* in, const ref_strides* is, const void* bias,
                 const ref_strides* bs, const void* coeff, const ref_strides* cs, void* out);
void ref_compare(int op, int dtype, const void* a, const ref_strides* as, const void* b,
                 const ref_strides* bs, uint8_t* out);
void ref_compare_scalar(int op, int dtype, const void* a, float sf, int64_t si, int scalar_first,
                        uint8_t* out, size_t count);
void ref_cast(const void* in, int in_type, void* out, int out_type, size_t count);
void ref_pow(int dtype, const void* in, float bf, float scalef, int64_t bi, int64_t scalei,
             const void* scales, void* out, size_t count);
void ref_elemwise(int op, int dtype, const void* in, const void* scales, void* out, size_t count);
void ref_reduce(int op, int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
                int64_t inner);
void ref_log_softmax(int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
                     int64_t inner);
void ref_gather(int dtype, const void* in, const int64_t* idx, const ref_strides* idx_strides,
                void* out, int64_t outer, int64_t middle, int64_t out_count, int64_t inner);
/* BackendCPU.swift:407-425: byte-wise or (0) / and (1) / xor (2) over the broadcast shape. */
void ref_bitwise_op(int op, int dtype, const void* a, const ref_strides* as, const void* b,
                    const ref_strides* bs, void* out);
/* BackendCPU.swift:922-998: running sum (op 0) or product (op 1) along the middle axis of
 * [outer, reduce, inner] in Float / Int64, optionally exclusive and / or from the far end. */
void ref_cumulative(int op, int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
                    int64_t inner, int exclusive, int reverse);
/* BackendCPU.swift:888-920: for every (outer, inner) pair the permutation (int64) that sorts the
 * reduce axis. The reference's comparison sort leaves the order of equal keys open; this one
 * is stable (equal keys keep their source order), which the `stable` flag asks for. */
void ref_argsort(int dtype, const void* in, int64_t* out, int64_t outer, int64_t reduce, int64_t inner,
                 int descending);
/* BackendCPU.swift:1149-1188. `in` holds outer*out_count*inner elements, `out` receives
 * outer*middle*inner; contributions to one output add up in (i, j, k) order in Float/Int64. */
void ref_scatter(int dtype, const void* in, const int64_t* idx, const ref_strides* idx_strides,
                 void* out, int64_t outer, int64_t middle, int64_t out_count, int64_t inner);
/* BackendCPU.swift:1040-1085. */
void ref_log_softmax_grad(int dtype, const void* in, const void* out_grad, void* out, int64_t outer,
                          int64_t reduce, int64_t inner);
/* BackendCPU.swift:704-782: out = min(hi, max(lo, a)); lo or hi may be NULL (not both). */
void ref_clamp(int dtype, const void* a, const ref_strides* as, const void* lo, const ref_strides* ls,
               const void* hi, const ref_strides* hs, void* out);
void ref_when(int dtype, const uint8_t* mask, const ref_strides* ms, const void* a,
              const ref_strides* as, const void* b, const ref_strides* bs, void* out);
void ref_matmul(int dtype, int64_t batch, const void* a, int trans_a, const void* b, int trans_b,
                int trans_out, int64_t rows, int64_t inner, int64_t cols, void* out);
/* Rows [row0, row1) of one fp16/fp32 product, single thread: the bounded CPU-baseline sample. */
void ref_matmul_rows(int dtype, const void* a, int trans_a, const void* b, int trans_b,
                     int64_t rows, int64_t inner, int64_t cols, int64_t row0, int64_t row1,
                     float* out_f32);
void ref_triangular(int dtype, const void* in, void* out, int64_t batch, int64_t rows,
                    int64_t cols, int upper, int64_t offset);
void ref_fill(int dtype, float vf, int64_t vi, void* out, size_t count);
void ref_axis_permutation(const int64_t* perm, const int64_t* shape, int ndim, int64_t* out);
void ref_normalize(int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
                   int64_t inner, float eps);
void ref_concat(int dtype, const void* const* inputs, const int64_t* inner_counts, int n_inputs,
                int64_t outer, void* out);

#ifdef __cplusplus
}
#endif
#endif
