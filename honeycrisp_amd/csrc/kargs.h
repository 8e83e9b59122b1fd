/*
 * Kernel argument blocks shared by the host launcher (hchip.cpp) and the gfx950
 * kernels. Every kernel takes exactly one of these structs by value, so the
 * host hands the struct itself to hipModuleLaunchKernel as the kernarg buffer.
 * Plain C layout, natural alignment, no pointers-to-host.
 */
#ifndef HC_KARGS_H
#define HC_KARGS_H

#include <stdint.h>

#define HCK_MAX_DIMS 8
#define HCK_BLOCK 256

/* Joint broadcast descriptor for up to three operands after the host has dropped
 * size-1 axes and merged axes that are mergeable for every operand. The innermost
 * axis is split off: a thread handles `vec` consecutive inner elements, the rest of
 * the flat index ("row") is unravelled over outer_shape. Strides are in elements;
 * inner strides are 0 or 1. */
typedef struct {
  uint32_t n_outer;
  uint32_t inner;
  uint32_t inner_vecs; /* inner / vec */
  uint32_t total_vecs; /* rows * inner_vecs */
  uint32_t outer_shape[HCK_MAX_DIMS - 1];
  uint32_t outer_stride[3][HCK_MAX_DIMS - 1];
  uint32_t inner_stride[3];
  /* division by inner_vecs and by outer_shape[k] as multiply-high and shifts (hck_fast_div) */
  uint32_t inner_magic, inner_sh;
  uint32_t outer_magic[HCK_MAX_DIMS - 1];
  uint32_t outer_sh[HCK_MAX_DIMS - 1];
  uint32_t pad;
} hck_bcast;

/* n / d for any 32-bit n with d's precomputed (magic, sh): l = ceil(log2 d),
 * magic = floor(2^32 (2^l - d) / d) + 1, sh = min(l, 1) | max(l - 1, 0) << 8;
 * t = high half of magic * n, quotient = (t + ((n - t) >> min(l, 1))) >> max(l - 1, 0). */
static inline void hck_fast_div_setup(uint32_t d, uint32_t* magic, uint32_t* sh) {
  uint32_t l = 0;
  while ((1ull << l) < d) l++;
  *magic = (uint32_t)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
  *sh = (l < 1 ? l : 1u) | ((l > 1 ? l - 1 : 0u) << 8);
}

/* out = a (op) b, broadcast; also compare (bool out) and broadcast copy (a only). */
typedef struct {
  const void* a;
  const void* b;
  void* out;
  hck_bcast d;
} hck_binary_args;

/* out = f(in, coeff, bias) for mulAdd / addMul; out = mask ? a : b for when. */
typedef struct {
  const void* x;
  const void* y;
  const void* z;
  void* out;
  hck_bcast d;
} hck_ternary_args;

/* Contiguous tensor (op) scalar. */
typedef struct {
  const void* in;
  void* out;
  uint64_t count;
  float sf;
  int32_t pad;
  int64_t si;
} hck_scalar_args;

/* Contiguous unary map with optional per-element scales: elemwise, pow, cast, fill. */
typedef struct {
  const void* in;
  const void* scales;
  void* out;
  uint64_t count;
  float p0; /* pow: exponent / fill: value */
  float p1; /* pow: scale */
  int64_t i0;
  int64_t i1;
} hck_map_args;

/* Input viewed as [outer, reduce, inner]. */
typedef struct {
  const void* in;
  void* out;
  uint32_t outer;
  uint32_t reduce;
  uint32_t inner;
  float eps;
  const void* in2; /* logSoftmaxGrad: the output gradient */
  /* reduce, few long rows: every row is cut into `segs` segments of `seg_len` elements, one
   * workgroup each, which leave [outer, segs] partials (accumulator type; arg-reductions: the
   * ordering key and the index within the row) for hc_reduce_cols_final_* with inner = 1 */
  uint32_t segs, seg_len;
  void* pvals;
  uint32_t* pidx;
} hck_reduce_args;

/* Row kernels that a recording's rewrite substitutes for chains of launches (same arithmetic,
 * intermediate by intermediate). */
typedef struct {
  /* [cast to fp32 ->] normalize rows in fp32 [-> x * (gain [+ gain_add]) + bias] [-> cast] */
  const void* in;
  void* out;
  const void* gain; /* `reduce` fp32 elements */
  const void* bias;
  uint32_t outer;
  uint32_t reduce;
  float eps;
  float gain_add;
  uint32_t flags; /* HCK_LN_* */
  uint32_t pad;
} hck_layernorm_args;
#define HCK_LN_AFFINE 1u   /* x * gain + bias follows */
#define HCK_LN_GAIN_ADD 2u /* ... with gain + gain_add formed first */

typedef struct {
  /* [x * scale ->] [+ mask ->] logSoftmax over rows [-> exp] */
  const void* in;
  void* out;
  const void* mask; /* [mask_rows, reduce]; row r of the input takes mask row r % mask_rows */
  uint32_t outer;
  uint32_t reduce;
  uint32_t mask_rows;
  float scale;
  uint32_t flags; /* HCK_SM_* */
  uint32_t pad;
} hck_softmax_chain_args;
#define HCK_SM_SCALE 1u
#define HCK_SM_MASK 2u
#define HCK_SM_EXP 4u

/* One attention head per workgroup column: out = softmax-chain(q k^T) v with 64-wide heads, fp16.
 * q, out: [T, 64] rows at row strides q_rs / o_rs; k: [T, 64] at k_rs; v: [T, 64] at v_rs (all
 * contiguous along the 64). Slice z of an operand starts at z * bs, or with bdiv != 0 at
 * (z / bdiv) * bs + (z % bdiv) * bs2 (heads that are an inner axis of [B, T, H, 64]). The chain
 * between the two products is that of hck_softmax_chain_args (flags, scale, mask, mask_rows: row
 * r of all batch * T score rows takes mask row r % mask_rows). */
typedef struct {
  const void* q;
  const void* k;
  const void* v;
  const void* mask;
  void* out;
  uint32_t T;      /* queries = keys per head, a multiple of 64 */
  uint32_t bdiv;
  uint32_t q_rs, k_rs, v_rs, o_rs;
  uint64_t q_bs, q_bs2, k_bs, k_bs2, v_bs, v_bs2, o_bs, o_bs2;
  uint32_t mask_rows;
  uint32_t flags; /* HCK_SM_* */
  float scale;
  uint32_t pad;
} hck_attention_args;

/* Column reduction ([outer, reduce, inner], inner > 1) in up to two passes: the reduce axis is
 * cut into `splits` ranges of `chunk` rows; with splits > 1 each range leaves a partial value
 * (and, for arg-reductions, its index) per column, combined by a second kernel. */
typedef struct {
  const void* in;
  void* out;
  void* pvals;    /* [outer, splits, inner] accumulators (float or int64) */
  uint32_t* pidx; /* [outer, splits, inner] indices (arg-reductions) */
  uint32_t outer;
  uint32_t reduce;
  uint32_t inner;
  uint32_t splits;
  uint32_t chunk;
  /* lanes of a wave along inner (a power of two <= 64); the other 64 / jl lanes of the wave
   * take further rows. 0 = 64. The final pass over the partials uses jl_final. */
  uint32_t jl;
  const float* aux; /* exp-sum: the per-column maximum, [outer, inner] */
  uint32_t jl_final;
  uint32_t pad;
} hck_reduce_cols_args;

/* Column logSoftmax / logSoftmaxGrad, last step: every element combined with per-column
 * statistics ([outer, inner] floats). */
typedef struct {
  const void* in;
  const void* grad; /* logSoftmaxGrad only */
  void* out;
  const float* col_max;
  const float* col_expsum;  /* hc_log_softmax_cols_logsum turns it into logf(exp-sum) + maximum in place */
  const float* col_gradsum; /* logSoftmaxGrad only */
  uint32_t outer, reduce, inner, pad;
} hck_softmax_cols_args;

/* cumulativeSum / cumulativeProd / argsort along the middle axis of [outer, reduce, inner].
 * reverse: scan from the far end (cumulative ops) or sort in descending order (argsort). */
typedef struct {
  const void* in;
  void* out;
  /* cumulative ops on few, long lines: the axis is cut into `segs` segments of `seg_len`
   * positions (in scan order) that are scanned independently; carry[(i * segs + s) * inner + j]
   * (float for float types, int64 otherwise) first receives the segments' totals, then what
   * precedes each segment. segs <= 1: unused. */
  void* carry;
  uint32_t outer, reduce, inner;
  uint32_t exclusive, reverse;
  uint32_t segs, seg_len, pad;
} hck_scan_args;

/* argsort of axes longer than one block sorts at once: sorted runs of (key, index) pairs, one
 * array of each per line ([lines, reduce], line = outer * inner + inner index), merged pairwise. */
typedef struct {
  const void* in;          /* chunk pass: the tensor; emit pass: unused */
  void* out;               /* emit pass: int64 result */
  const uint64_t* keys_in; /* merge pass: runs of length `run` */
  const uint32_t* idx_in;
  uint64_t* keys_out;      /* chunk and merge passes */
  uint32_t* idx_out;
  uint32_t outer, reduce, inner;
  uint32_t run, descending, pad;
} hck_sort_args;

/* Fused AdamW step over `count` contiguous elements; the scalars are the ones the op-by-op
 * composition would pass to its tensor-scalar ops. */
typedef struct {
  const void* param;
  const void* grad;
  const void* m1;
  const void* m2;
  void* out_param;
  void* out_m1;
  void* out_m2;
  uint64_t count;
  float beta1, one_minus_beta1, beta2, one_minus_beta2;
  float bias1, bias2; /* 1 / (1 - beta^step) */
  float eps, lr, decay; /* decay = 1 - lr * weightDecay */
  float exp_square, exp_root; /* 2 and 0.5, passed at run time so that powf is called exactly
                                 as in the pow kernels (no folding into x*x or sqrt) */
} hck_adamw_args;

/* Row gather: every output row of row_vecs 16-byte (or narrower) vectors comes from
 * one source row chosen by an index that only depends on the row. */
typedef struct {
  const void* in;
  const int64_t* indices;
  void* out;
  uint32_t out_count; /* rows per outer slice (indices.shape[axis]) */
  uint32_t middle;    /* source rows per outer slice */
  uint32_t row_vecs;  /* vectors per row */
  uint32_t total_rows;
  hck_bcast idx; /* operand 0 = index offset for a flat row number, vec = 1 */
} hck_gather_rows_args;

/* Row scatter with repeated indices, without atomics on the data: source rows are grouped by
 * destination row (count, scan, fill), every destination row then adds its sources in
 * ascending source order. Row numbers are flat over the outer axis. */
typedef struct {
  const void* in;          /* [outer, n_src, row] */
  const int64_t* indices;
  void* out;               /* [outer, n_dst, row] */
  int64_t* counts;         /* [outer * n_dst] sources per destination row */
  const int64_t* starts;   /* exclusive running sum of counts */
  int64_t* cursor;         /* [outer * n_dst] fill positions, zero before the fill pass */
  uint32_t* list;          /* [outer * n_src] source rows, grouped by destination */
  uint32_t n_src, n_dst;
  uint32_t row_vecs;       /* 16-byte vectors per row */
  uint32_t total_src;      /* outer * n_src */
  hck_bcast idx;           /* operand 0 = index offset for a flat source row, vec = 1 */
} hck_scatter_rows_args;

/* Element gather: general index map over the flat output index. */
typedef struct {
  const void* in;
  const int64_t* indices;
  void* out;
  uint32_t out_count;
  uint32_t middle;
  uint32_t inner;
  uint32_t total;
  hck_bcast idx; /* operand 0 = index offset for a flat output element, vec = 1 */
} hck_gather_elems_args;

typedef struct {
  int64_t* out;
  uint32_t total;
  uint32_t ndim;
  uint32_t new_shape[HCK_MAX_DIMS];
  uint32_t new_strides[HCK_MAX_DIMS];
  uint32_t permuted_strides[HCK_MAX_DIMS];
} hck_axis_perm_args;

/* Direct axis permutation (the gather that follows an axisPermutation, without its index vector).
 * Axes are the output's, outermost first, after the host dropped unit axes and merged axes that are
 * adjacent in both orders; strides in elements.
 * Row form: the innermost axis is contiguous in both; a lane moves `vec` of its `inner` elements, the
 * row number is unravelled over shape[0..ndim) (divisions by multiply-high, hck_fast_div_setup).
 * Tile form: the output's innermost axis (extent tile_a, source stride a_stride) differs from the
 * source's (extent tile_c, output stride c_out_stride): tiles of 2^ta_log2 x 2^tc_log2 elements go
 * through LDS, read along the source's innermost axis and written along the output's; shape[]/in_stride[]/out_stride[] then
 * describe the remaining axes. */
typedef struct {
  const void* in;
  void* out;
  uint32_t ndim;
  uint32_t inner;
  uint32_t inner_vecs;
  uint32_t total; /* row form: vectors; tile form: tiles */
  uint32_t shape[HCK_MAX_DIMS];
  uint32_t in_stride[HCK_MAX_DIMS];
  uint32_t out_stride[HCK_MAX_DIMS];
  uint32_t magic[HCK_MAX_DIMS];
  uint32_t sh[HCK_MAX_DIMS];
  uint32_t inner_magic, inner_sh;
  uint32_t tile_a, tile_c, a_stride, c_out_stride;
  uint32_t tiles_a, tiles_c;
  uint32_t tiles_a_magic, tiles_a_sh, tiles_c_magic, tiles_c_sh;
  uint32_t ta_log2, tc_log2; /* tile extents along a and c: powers of two, product <= 4096 */
} hck_permute_args;

typedef struct {
  const void* in;
  void* out;
  uint32_t total; /* batch * rows * cols */
  uint32_t rows;
  uint32_t cols;
  int32_t upper;
  int64_t offset;
} hck_triangular_args;

/* One input of a concat: out[o, out_off + c] = in[o, c], c < inner. */
typedef struct {
  const void* in;
  void* out;
  uint32_t outer;
  uint32_t inner;       /* bytes per outer slice of this input */
  uint32_t total_inner; /* bytes per outer slice of the output */
  uint32_t out_off;     /* byte offset inside the output slice */
} hck_concat_args;

/* C[M,N] = op(A) * op(B) per batch element; logical element (i,k) of A is at
 * a[i*a_rs + k*a_cs], (k,j) of B at b[k*b_rs + j*b_cs], (i,j) of C at c[i*c_rs + j*c_cs]
 * (strides in elements), batch element m at offsets m*a_bs, m*b_bs, m*c_bs. */
typedef struct {
  const void* a;
  const void* b;
  void* c;
  uint32_t M, N, K;
  uint32_t batch;
  uint32_t a_rs, a_cs, b_rs, b_cs, c_rs, c_cs;
  uint64_t a_bs, b_bs, c_bs;
  uint32_t tiles_m, tiles_n;
  /* Tile order of the direct-to-LDS kernels. xcd_gn == 0: block ids equal mod 8 (one XCD)
   * get a contiguous band of tiles. Otherwise the tile grid is cut into super-blocks of
   * (8/xcd_gn * xcd_sm) x (xcd_gn * xcd_sn) tiles, visited one after the other; inside one,
   * the 8 XCDs form an (8/xcd_gn) x xcd_gn grid and each owns xcd_sm x xcd_sn tiles. */
  uint32_t xcd_gn, xcd_sm, xcd_sn;
  /* edge kernels: rows (K-contiguous operand) or elements of a k-row (M/N-contiguous operand,
   * a multiple of 16 bytes) that may be fetched; anything beyond is clamped to the last one */
  uint32_t a_lim, b_lim;
  /* The fields from here on are read only by the second build of the direct-to-LDS kernels (names
   * ending in _m), which a recording's rewrite substitutes for the plain ones.
   * Operations applied to the finished tile before it is stored, in
   * order, each on the value rounded to the output type, i.e. with the arithmetic of the
   * separate kernels they replace: what a recording's rewrite merges into the product. */
  uint32_t ep_kind[3];    /* HCK_EP_* ; 0 ends the list */
  uint32_t ep_ld[3];      /* HCK_EP_ADD_MATRIX: leading dimension of the matrix, elements */
  const void* ep_ptr[3];  /* HCK_EP_ADD_ROW: N elements; HCK_EP_ADD_MATRIX: [M, ld] */
  /* Two-level batch (0 = off): slice z lies at
   * (z / bdiv) * x_bs + (z % bdiv) * x_bs2. What a batched product reads or writes when a
   * recording folds a swap of the batch axes ([B, T, H, d] <-> [B, H, T, d]) into it. */
  uint32_t bdiv;
  /* A group of up to HCK_GEMM_GROUP products over the same A with the same shape, operations and
   * strides in one launch (0 = off): blockIdx.y picks the member's B,
   * C and epilogue operands from the tables. What a recording makes of the q, k, v projections of
   * an attention layer. */
  uint32_t group;
  uint64_t a_bs2, b_bs2, c_bs2;
  const void* g_b[4];
  void* g_c[4];
  const void* g_ep[3][4];
} hck_gemm_args;
#define HCK_GEMM_GROUP 4

#define HCK_EP_NONE 0
#define HCK_EP_ADD_ROW 1     /* x + row[n]   (a bias broadcast over the rows) */
#define HCK_EP_ADD_MATRIX 2  /* x + other[m, n] (a residual connection) */
#define HCK_EP_GELU 3        /* ElemwiseOp.geluApprox; only as the last operation of the list */
#define HCK_EP_ADD_ROW_F32 4 /* x + T(row[n]) with the row held in fp32 (a parameter cast at call time) */

/* Copy of a batch of [rows, in_cols] matrices with leading dimension in_ld into [rows, out_cols]
 * with leading dimension out_ld; columns >= in_cols are written as zero. Element offsets. */
typedef struct {
  const void* in;
  void* out;
  uint32_t rows, in_cols, out_cols, pad;
  uint64_t in_ld, out_ld, in_bs, out_bs;
} hck_copy2d_args;

/* Skinny product C[p, q] = sum_k X[p, k] * Y[k, q]: p over a long extent L, q over a thin one
 * t <= 32 (a matrix-vector product, or the fringe of a ragged GEMM). Element strides; which of
 * A / B is X and whether C is stored [p, q] or [q, p] is folded into the strides by the host. */
typedef struct {
  const void* x;
  const void* y;
  void* c;
  float* acc;  /* split-K form: fp32 partial sums [batch, chunks, L, t], one slice per k-chunk */
  uint32_t L, t, K;
  uint32_t x_ps, x_ks, y_ks, y_qs, c_ps, c_qs;
  uint32_t kchunk; /* split-K form: k-range per workgroup */
  uint32_t chunks; /* split-K form: number of k-chunks */
  uint64_t x_bs, y_bs, c_bs;
} hck_skinny_args;

/* hc_gemm_skinny_pair_*: two independent skinny launches as one. Workgroups [0, split) run `a`,
 * [split, split + blocks_b) run `b`, each with the kernel its kind names. */
#define HCK_SKINNY_K 0u     /* hc_gemm_skinny_k_*    */
#define HCK_SKINNY_P 1u     /* hc_gemm_skinny_p_*    */
#define HCK_SKINNY_PACK 2u  /* hc_gemm_skinny_pack_* */
#define HCK_SKINNY_STORE 3u /* hc_gemm_skinny_store_* */
typedef struct {
  hck_skinny_args a, b;
  uint32_t split, blocks_b, kind_a, kind_b;
} hck_skinny_pair_args;

#endif
