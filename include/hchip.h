/*
 * hchip - C ABI of the MI355X (gfx950) compute backend for Honeycrisp.
 *
 * This is the whole boundary a `HIPBackend: Backend` subclass binds: a context
 * that owns one device, one in-order HIP stream, a caching device allocator
 * and the embedded gfx950 code objects, plus one entry point per backend
 * operation. Plain pointers and sizes only; every function returns 0 on
 * success or a non-zero hc_status / hipError_t-derived code and never throws
 * or aborts. hc_last_error_string() gives the message for the calling thread.
 *
 * Ordering: all work is enqueued on the context's single stream, so an
 * operation that consumes the output of an earlier call sees its result, and
 * hc_free() may be called as soon as the last consumer has been enqueued.
 * Entry points are thread-safe (one mutex around allocator + launch).
 *
 * Layout conventions follow the reference backend interface
 * (Sources/Honeycrisp/Backend.swift:170-815): dense row-major buffers,
 * dtype codes in Tensor.DType order (Tensor.swift:24-28), strides in elements.
 */
#ifndef HCHIP_H
#define HCHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct hc_ctx hc_ctx;
typedef struct hc_event hc_event;
typedef struct hc_module hc_module;
typedef struct hc_function hc_function;

/* Tensor.DType (Tensor.swift:24-28); byte sizes 8/1/2/4 (:42-53). */
typedef enum { HC_I64 = 0, HC_BOOL = 1, HC_F16 = 2, HC_F32 = 3 } hc_dtype;
/* NumericBinaryOp (BinaryOps.swift:2-8). */
typedef enum { HC_ADD = 0, HC_MUL = 1, HC_SUB = 2, HC_DIV = 3, HC_MOD = 4 } hc_binary;
/* ReduceOp (ReduceRepeat.swift:53-58). */
typedef enum { HC_SUM = 0, HC_PROD = 1, HC_ARGMAX = 2, HC_ARGMIN = 3 } hc_reduce_op;
/* ComparisonOp (Comparison.swift:4-10). */
typedef enum { HC_EQ = 0, HC_NE = 1, HC_LT = 2, HC_LE = 3, HC_GT = 4, HC_GE = 5 } hc_compare_op;
/* ElemwiseOp (Elemwise.swift:13-43), same order. */
typedef enum {
  HC_SIN = 0, HC_COS, HC_MINUS_SIN, HC_TAN, HC_TAN_GRAD, HC_ATAN, HC_ATAN_GRAD, HC_ACOS,
  HC_ACOS_GRAD, HC_ASIN, HC_ASIN_GRAD, HC_EXP, HC_LOG, HC_RECIP, HC_SIGMOID, HC_SIGMOID_GRAD,
  HC_RELU, HC_RELU_GRAD, HC_ABS, HC_ABS_GRAD, HC_GELU_APPROX, HC_GELU_APPROX_GRAD,
  HC_GELU_EXACT, HC_GELU_EXACT_GRAD, HC_ERF, HC_ERF_GRAD, HC_FLOOR, HC_CEIL, HC_ROUND,
  HC_ELEMWISE_COUNT
} hc_elemwise_op;

/* Status codes. Codes >= HC_ERR_HIP_BASE are HC_ERR_HIP_BASE + hipError_t. They map
 * onto BackendError (Backend.swift:6-16): ALLOC -> .allocationFailed, LOAD ->
 * .failedToLoadKernels, UNSUPPORTED -> .notImplemented, everything else ->
 * .kernelFailed(hc_last_error_string()). */
typedef enum {
  HC_OK = 0,
  HC_ERR_INVALID = 1,     /* bad argument (null pointer, negative count, ndim > 8 ...) */
  HC_ERR_ALLOC = 2,       /* device or pinned-host allocation failed */
  HC_ERR_LOAD = 3,        /* code object missing / not loadable / kernel symbol missing */
  HC_ERR_UNSUPPORTED = 4, /* dtype/op combination this backend leaves to the CPU fallback */
  HC_ERR_TOO_LARGE = 5,   /* element count beyond the kernel's 32-bit index range */
  HC_ERR_NO_DEVICE = 6,
  HC_ERR_HIP_BASE = 1000
} hc_status;

#define HC_MAX_DIMS 8

/* BroadcastStrides (Broadcast.swift:9-30): virtual shape and, per axis, the stride
 * into the data buffer in elements (0 on broadcast axes). Element i of the virtual
 * array maps to data index sum_d strides[d] * ((i / prod(shape[d+1:])) % shape[d])
 * (Broadcast.swift:72-90). */
typedef struct {
  uint32_t ndim;
  uint32_t reserved;
  int64_t shape[HC_MAX_DIMS];
  int64_t strides[HC_MAX_DIMS];
} hc_strides;

typedef struct {
  char name[256];
  char arch[64];
  int compute_units;
  int clock_mhz;
  int wavefront_size;
  int lds_bytes_per_block;
  size_t total_mem;
} hc_device_info;

/* ---- context, errors ---- */

/* Create a context on `device` (HIP ordinal): stream, allocator, code objects.
 * Replaces MPSBackend.init (BackendMPS.swift:373-466) for this backend. */
int hc_init(int device, hc_ctx** out);
void hc_shutdown(hc_ctx* ctx);
const char* hc_last_error_string(void);
int hc_get_device_info(hc_ctx* ctx, hc_device_info* out);

/* Switches for measurements and tests. No counterpart in the reference (its backends are
 * configured in code). A context takes the first value of each switch from the environment
 * variable of the same name when it is created; this call changes one afterwards, safely while
 * other threads launch through the context (an entry point works on a copy it takes when it
 * starts). `value` NULL or "" restores the default; for the on/off switches anything but "0"
 * means on. Names: HCHIP_GEMM_TILE (general | <BM>x<BN>), HCHIP_GEMM_KERNEL (dma | dma2 | mi16 |
 * staged), HCHIP_GEMM_RING (4 | 2), HCHIP_GEMM_ONE (0), and the on/off switches
 * HCHIP_GEMM_NO_PEEL, HCHIP_GEMM_NO_DIRECT, HCHIP_GEMM_NO_REPITCH, HCHIP_GEMM_BAND,
 * HCHIP_NO_FUSION (looked at when a capture begins), HCHIP_RECORDING_LOG,
 * HCHIP_GRAPH_AS_LAUNCHES (both looked at when a capture ends). HC_ERR_INVALID for any other name. */
int hc_debug_set(hc_ctx* ctx, const char* name, const char* value);

/* ---- memory: backs Tensor.Data (Tensor.swift:69-85) and DataAllocator
 * (Backend.swift:894-896; precedent BackendMPS.swift:468-556) ---- */

/* Size-bucketed caching allocator; bytes == 0 yields a valid 1-byte buffer. */
int hc_malloc(hc_ctx* ctx, size_t bytes, void** out);
/* Stream-ordered: the block becomes reusable by later hc_malloc calls on the
 * same stream, so freeing right after the last consumer was enqueued is safe. */
int hc_free(hc_ctx* ctx, void* ptr);
/* Return cached blocks to the driver (waits for the stream first). */
int hc_trim(hc_ctx* ctx);
/* Bytes currently handed out / held in the cache. */
int hc_mem_stats(hc_ctx* ctx, size_t* in_use, size_t* cached);
/* Pinned host staging memory (hipHostMalloc). */
int hc_host_alloc(hc_ctx* ctx, size_t bytes, void** out);
int hc_host_free(hc_ctx* ctx, void* ptr);
/* Copies ordered after everything already enqueued: what Tensor.Data.onCPU / mutateOnCPU need
 * (Tensor.swift:74-84). When a call returns the host buffer is the caller's again: d2h has
 * completed; h2d has completed, or (uploads up to 256 KiB) the bytes were taken into pinned
 * staging memory from which the stream copies them in order, so that small uploads in the middle
 * of a forward pass (index vectors of slices, constants) do not make the host wait for the
 * device. */
int hc_memcpy_h2d(hc_ctx* ctx, void* dst, const void* src, size_t bytes);
int hc_memcpy_d2h(hc_ctx* ctx, void* dst, const void* src, size_t bytes);
int hc_memcpy_d2d(hc_ctx* ctx, void* dst, const void* src, size_t bytes);
/* Enqueue-only copies; the host pointer must be pinned and stay valid until a sync. */
int hc_memcpy_h2d_async(hc_ctx* ctx, void* dst, const void* src, size_t bytes);
int hc_memcpy_d2h_async(hc_ctx* ctx, void* dst, const void* src, size_t bytes);

/* ---- stream, events: Tensor.Data.wait() (Tensor.swift:72) and timing ---- */

int hc_sync(hc_ctx* ctx);
int hc_event_create(hc_ctx* ctx, hc_event** out);
int hc_event_record(hc_ctx* ctx, hc_event* ev);
int hc_event_sync(hc_event* ev);
/* 0 = complete, 1 = still pending, other = error. */
int hc_event_query(hc_event* ev);
int hc_event_elapsed_ms(hc_event* start, hc_event* stop, float* ms);
int hc_event_destroy(hc_event* ev);
/* Run fn(user) on a runtime thread once prior work completes: the hook a Swift
 * continuation resumes from (precedent BackendMPS.swift:2663-2720). */
int hc_launch_host_func(hc_ctx* ctx, void (*fn)(void*), void* user);

/* ---- stream capture and graph replay ----
 * No counterpart in the reference, which issues one backend call per op (one Task per op,
 * Tensor.swift:634-657): a model whose forward pass is a few hundred small ops is bound by
 * that per-op host cost. Between hc_capture_begin and hc_capture_end every op entry point
 * records its kernels into a graph instead of running them; hc_graph_launch replays the
 * whole recording with one call, in stream order with everything else.
 *  - Buffers obtained from hc_malloc during the capture stay reserved for the graph (also
 *    after hc_free) until hc_graph_destroy, so a replay never writes into memory that was
 *    handed to somebody else. Buffers allocated before the capture and read by it must be
 *    kept alive by the caller for as long as the graph is replayed; results are read from
 *    the buffers the captured ops returned.
 *  - Host transfers, hc_sync, event and host-function calls are refused while capturing
 *    (HC_ERR_INVALID). One capture at a time per context.
 *  - The launches of a capture are listed first and enqueued at hc_capture_end, after a
 *    rewrite. Every entry point declares the buffers it reads and writes, every buffer has
 *    an address of its own while the capture lasts, and hc_free says that a buffer has no
 *    further reader: from that alone the rewrite sees results with a single reader and
 *    replaces chains of launches by one launch that does the same arithmetic, intermediate
 *    by intermediate, so a replay returns the bits of the unmerged sequence:
 *      matmul -> + row -> [+ matrix | geluApprox]   one product with an epilogue (the row may
 *                                                    be an fp32 buffer cast to fp16 on the way)
 *      [cast ->] normalize -> [(gain + c) *, + bias] -> [cast]      one LayerNorm kernel
 *      [* s ->] [+ mask ->] logSoftmax -> [exp]                     one softmax kernel
 *      swap of two batch axes -> batchedMatmul -> swap back         read / written through strides
 *      q k^T -> that softmax kernel -> x v, 64-wide heads, T a
 *      multiple of 64 up to 512 (fp16) / 256 (fp32)                 one attention kernel
 *      products of one shape over the same input (q, k, v)          one launch
 *      argmax | argmin over rows -> gather of those indices from
 *      the same tensor (Tensor.max / min / all / some)              one row kernel
 *    Buffers that only held merged intermediates are never written by a replay.
 *    Switches (environment at hc_init, or hc_debug_set): HCHIP_RECORDING_LOG=1 lists the
 *    launches of the rewritten recording on stderr at hc_capture_end; HCHIP_GRAPH_AS_LAUNCHES=1
 *    makes hc_graph_launch issue them one by one instead of through hipGraphLaunch (for kernel
 *    traces); HCHIP_NO_FUSION=1 when a capture begins turns its rewrite off. */
typedef struct hc_graph hc_graph;
int hc_capture_begin(hc_ctx* ctx);
int hc_capture_end(hc_ctx* ctx, hc_graph** out);
/* Ends a capture and throws the recording away (error paths). */
int hc_capture_abort(hc_ctx* ctx);
int hc_graph_launch(hc_ctx* ctx, hc_graph* graph);
/* Number of nodes (kernel launches and copies) one replay of the graph issues. */
int hc_graph_node_count(hc_graph* graph, size_t* out);
int hc_graph_destroy(hc_ctx* ctx, hc_graph* graph);

/* ---- batching: the rewrite of a recording for ordinary, call-by-call use ----
 * No counterpart in the reference, whose API has no notion of a recording either: a program
 * written against it issues one backend call per op and never says where a forward pass begins
 * or ends (Tensor.swift:634-657). With max_launches > 0 the op entry points list their launches
 * instead of enqueueing them, exactly as inside a capture, and the list is rewritten (the same
 * passes, the same guarantee: the bits of the call-by-call result) and enqueued
 *  - when it holds max_launches launches (at the next hc_free that leaves the caller with at most one
 *    buffer allocated since the last batch, or a quarter of max_launches later at the latest: a
 *    list cut in the middle of a layer leaves the launches around the cut unmerged), or
 *    (idle_after > 0) at least idle_after launches
 *    while the device is past the middle of the last batch (or has had none): looked up in
 *    hc_free when the caller holds at most one buffer allocated since the last batch (between
 *    two layers of a model: every other intermediate is released, so no chain the rewrite could
 *    merge is cut). While the device has more than half a batch in front of it the list grows;
 *    after that it gets what there is, rewritten and enqueued while the rest still runs. Every
 *    batch that goes out early this way doubles the number of launches the next early one needs
 *    (up to max_launches); a call that waits or transfers starts over at idle_after: a program
 *    that reads a result after every pass gets its device started after idle_after launches,
 *    one that never waits and keeps the device short of work ends up with full batches,
 *  - before anything that must see or order against the results: hc_memcpy_d2h (Tensor.Data.onCPU),
 *    hc_sync, hc_event_record, hc_launch_host_func (Tensor.Data.wait), hc_graph_launch,
 *    hc_capture_begin, hc_trim, hc_flush; an upload is enqueued at once and overtakes the list
 *    when no listed launch uses the block it fills, else the list goes first,
 *  - when the blocks released since the last batch exceed 8 GiB, or an allocation fails.
 * A block released while its batch is listed is not handed out again before the batch has been
 * enqueued (the rewrite needs every buffer of a batch at an address of its own), so the
 * footprint of a batch is the sum of its intermediates. Errors of a listed launch surface in
 * the call that enqueues the batch; if that was not a call that waits or transfers (the batch
 * was full, or went out from hc_free), the next such call reports the failure once more, so a
 * caller that ignores the status of a release still learns of it. max_launches = 0 (the
 * default) enqueues what is listed and goes back to one launch per call. Refused during a
 * capture; a capture inside batching works (the list is enqueued first). HCHIP_BATCHING=<max>[,<idle_after>] in the environment at
 * hc_init starts a context with hc_set_batching(max, idle_after). */
int hc_set_batching(hc_ctx* ctx, size_t max_launches, size_t idle_after);
/* Enqueues what batching has listed so far. Nothing to do outside batching. */
int hc_flush(hc_ctx* ctx);
/* Launches and device-to-device copies that batches listed, and that were enqueued in their
 * place after the rewrite, since the context was created (either pointer may be NULL). */
int hc_batching_stats(hc_ctx* ctx, uint64_t* listed, uint64_t* enqueued);

/* ---- raw module API (thin wrappers over hipModuleLoadData / hipModuleGetFunction /
 * hipModuleLaunchKernel) for callers that bring their own gfx950 code objects ---- */

int hc_module_load(hc_ctx* ctx, const void* image, size_t bytes, hc_module** out);
int hc_module_unload(hc_ctx* ctx, hc_module* mod);
int hc_module_get_function(hc_module* mod, const char* name, hc_function** out);
int hc_launch(hc_ctx* ctx, hc_function* fn, const uint32_t grid[3], const uint32_t block[3],
              uint32_t shared_bytes, const void* kernarg, size_t kernarg_bytes);

/* ---- operations ----
 * Every pointer below is a device pointer from hc_malloc unless stated otherwise;
 * outputs are caller-allocated, dense, and never alias inputs.
 *
 * Alignment. hc_malloc returns 256-byte aligned blocks, which satisfies every entry point. A
 * pointer into the middle of a block (a view) must at least be aligned to its element size, and
 *  - the contiguous maps and row kernels require 16-byte aligned buffers and return
 *    HC_ERR_INVALID otherwise: hc_binary_op_scalar, hc_compare_scalar, hc_cast, hc_pow,
 *    hc_elemwise, hc_fill, hc_adamw, hc_log_softmax, hc_log_softmax_grad, hc_normalize, hc_reduce
 *    with inner == 1, and hc_scatter (whose output is cleared with hc_fill);
 *  - everything else takes any element-aligned pointer and only loses its 16-byte vector
 *    accesses: the broadcasting ops (hc_broadcast, hc_binary_op, hc_bitwise_op, hc_compare,
 *    hc_mul_add, hc_add_mul, hc_when, hc_clamp), hc_reduce with inner > 1, hc_cumulative,
 *    hc_argsort, hc_gather, hc_permute, hc_concat, hc_triangular and hc_matmul (whose tiled
 *    kernels fetch and store rows at any element alignment; an operand that does not leave 16
 *    readable bytes behind its last row inside its hc_malloc block, or that was not allocated by
 *    this context, goes through a zero-padded scratch copy instead). */

/* Backend.broadcast (Backend.swift:170-172; CPU BackendCPU.swift:255-265). */
int hc_broadcast(hc_ctx* ctx, int dtype, const void* a, const hc_strides* as, void* out);

/* Backend.binaryOp(BroadcastData, BroadcastData) (Backend.swift:178-185; CPU
 * BackendCPU.swift:267-314). Float dtypes compute in fp32 and round once; mod is
 * Python-style (TensorElement.swift:124-132, 214-222). */
int hc_binary_op(hc_ctx* ctx, int op, int dtype, const void* a, const hc_strides* as,
                 const void* b, const hc_strides* bs, void* out);

/* Backend.binaryOp(Tensor.Data, T) and (T, Tensor.Data) (Backend.swift:190-209; CPU
 * BackendCPU.swift:316-405). `sf` is used for float dtypes, `si` for int64. fp32
 * follows the CPU's vDSP forms: x / s == x * (1 / s), x - s == x + (-s),
 * s - x == x * -1 + s. */
int hc_binary_op_scalar(hc_ctx* ctx, int op, int dtype, const void* a, float sf, int64_t si,
                        int scalar_first, void* out, size_t count);

/* Backend.mulAdd / addMul (Backend.swift:240-257; CPU BackendCPU.swift:445-539). */
int hc_mul_add(hc_ctx* ctx, int dtype, const void* input, const hc_strides* is,
               const void* coeff, const hc_strides* cs, const void* bias, const hc_strides* bs,
               void* out);
int hc_add_mul(hc_ctx* ctx, int dtype, const void* input, const hc_strides* is, const void* bias,
               const hc_strides* bs, const void* coeff, const hc_strides* cs, void* out);

/* Backend.compare (Backend.swift:457-486; CPU BackendCPU.swift:541-624): bool (1 byte) out. */
int hc_compare(hc_ctx* ctx, int op, int dtype, const void* a, const hc_strides* as,
               const void* b, const hc_strides* bs, void* out);
int hc_compare_scalar(hc_ctx* ctx, int op, int dtype, const void* a, float sf, int64_t si,
                      int scalar_first, void* out, size_t count);

/* Backend.cast (Backend.swift:489-494; CPU BackendCPU.swift:626-646): f32->f16 is RNE
 * with overflow to inf; float->int64 truncates; anything->bool is (x != 0). */
int hc_cast(hc_ctx* ctx, const void* in, int in_type, void* out, int out_type, size_t count);

/* Backend.pow (Backend.swift:500-507; CPU BackendCPU.swift:648-702):
 * out = scale * scales[i] * x^b with the fp32 special cases b in {2, -1, 1}.
 * (bf, scalef) apply to float dtypes, (bi, scalei) to int64; scales may be NULL. */
int hc_pow(hc_ctx* ctx, int dtype, const void* in, float bf, float scalef, int64_t bi,
           int64_t scalei, const void* scales, void* out, size_t count);

/* Backend.elemwise (Backend.swift:770-774; CPU BackendCPU.swift:1748-1766; formulas
 * Elemwise.swift:44-183): out = f(x) * scales[i], float dtypes only; scales may be NULL. */
int hc_elemwise(hc_ctx* ctx, int op, int dtype, const void* in, const void* scales, void* out,
                size_t count);

/* Backend.reduce (Backend.swift:524-531; CPU BackendCPU.swift:784-886): input viewed as
 * [outer, reduce, inner]; sum/prod keep the dtype, argmax/argmin write int64 and return
 * the first extremum (strict compare from k = 0; a NaN at k > 0 never wins, a NaN at
 * k = 0 yields 0). */
int hc_reduce(hc_ctx* ctx, int op, int dtype, const void* in, void* out, int64_t outer,
              int64_t reduce, int64_t inner);

/* hc_reduce for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc. No counterpart in the reference. Same arguments,
 * kernels and results as hc_reduce, but the partial results of split reductions (a column
 * reduction cut into ranges, long rows cut into segments) live in a fixed array of
 * HC_NOALLOC_SCRATCH_BYTES of device memory that the library holds on every device it runs on
 * until the process ends, so the call allocates and frees nothing, not even from the context's
 * pool. A reduction whose partials need more returns HC_ERR_TOO_LARGE (the message says how
 * much). All calls on one GPU share that array, which keeps the last call's contents. Calls
 * through one context, from any number of threads, run one after the other: a per-device lock is
 * held while a call enqueues its (up to two) launches, and the context's stream keeps that order.
 * Calls that overlap on one GPU through two contexts (two streams) race on the array. */
#define HC_NOALLOC_SCRATCH_BYTES (8u << 20)
int hc_reduce_noalloc(hc_ctx* ctx, int op, int dtype, const void* in, void* out, int64_t outer,
                      int64_t reduce, int64_t inner);

/* Backend.cumulativeSum / cumulativeProd (Backend.swift:548-568; CPU BackendCPU.swift:922-998):
 * op 0 = running sum, 1 = running product along the middle axis of [outer, reduce, inner];
 * exclusive shifts the result by one position, reverse scans from the far end. */
int hc_cumulative(hc_ctx* ctx, int op, int dtype, const void* in, void* out, int64_t outer,
                  int64_t reduce, int64_t inner, int exclusive, int reverse);

/* Backend.argsort (Backend.swift:535-545; CPU BackendCPU.swift:888-920): int64 permutation that
 * sorts the middle axis, for every (outer, inner) pair. Always stable (equal keys keep their
 * source order). Axes up to 4096 elements are sorted in one pass in LDS; longer ones as runs of
 * 4096 merged pairwise, through scratch memory of 24 bytes per element from the context's pool. */
int hc_argsort(hc_ctx* ctx, int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
               int64_t inner, int descending);

/* Backend.logSoftmax (Backend.swift:571-575; CPU BackendCPU.swift:1000-1038). */
int hc_log_softmax(hc_ctx* ctx, int dtype, const void* in, void* out, int64_t outer,
                   int64_t reduce, int64_t inner);

/* Backend.normalize (Backend.swift:265-327: two-pass mean / biased variance,
 * (var + eps)^-0.5, every intermediate rounded to `dtype`). */
int hc_normalize(hc_ctx* ctx, int dtype, const void* in, void* out, int64_t outer,
                 int64_t reduce, int64_t inner, float eps);

/* Backend.gather (Backend.swift:609-616; CPU BackendCPU.swift:1108-1147) with
 * ScatterGatherIndices flattened (ScatterGather.swift:21-45):
 * out[(i*out_count + j)*inner + k] = in[(i*middle + idx)*inner + k],
 * idx = indices[idx_strides(flat out index)] (int64, no bounds check, no wrap). */
int hc_gather(hc_ctx* ctx, int dtype, const void* in, const void* indices,
              const hc_strides* idx_strides, void* out, int64_t outer, int64_t middle,
              int64_t out_count, int64_t inner);

/* Backend.bitwiseOp (Backend.swift:215-237; CPU BackendCPU.swift:407-443): or / and / xor of
 * the raw element bits over the broadcast shape, any dtype. The tensor-scalar form is the same
 * call with a 1-element buffer holding the scalar's bit pattern and all-zero strides. */
typedef enum { HC_BIT_OR = 0, HC_BIT_AND = 1, HC_BIT_XOR = 2 } hc_bitwise_op_kind; /* BitwiseOps.swift:38-41 */
int hc_bitwise_op(hc_ctx* ctx, int op, int dtype, const void* a, const hc_strides* as, const void* b,
                  const hc_strides* bs, void* out);

/* Backend.scatter (Backend.swift:621-626; CPU BackendCPU.swift:1149-1188), the adjoint of
 * gather: out[(i*middle + idx)*inner + k] += in[(i*out_count + j)*inner + k] over a zeroed
 * output of outer*middle*inner elements; numeric dtypes. Values sharing an index are added
 * with atomics (float sums in no fixed order; half values accumulate in float and are
 * rounded once). indices_are_unique != 0 (ScatterGatherIndices.indicesAreUnique,
 * ScatterGather.swift:4-19) lets the kernel store instead of add. */
int hc_scatter(hc_ctx* ctx, int dtype, const void* in, const void* indices,
               const hc_strides* idx_strides, void* out, int64_t outer, int64_t middle,
               int64_t out_count, int64_t inner, int indices_are_unique);

/* Backend.logSoftmaxGrad (Backend.swift:578-587; CPU BackendCPU.swift:1040-1085):
 * out = g - sum_k(g) * exp(logSoftmax(x)) over the reduce axis. */
int hc_log_softmax_grad(hc_ctx* ctx, int dtype, const void* in, const void* out_grad, void* out,
                        int64_t outer, int64_t reduce, int64_t inner);

/* Backend.clamp (Backend.swift:512-520; CPU BackendCPU.swift:704-782): min(hi, max(lo, a))
 * over the broadcast shape of `as`; lo or hi (with its strides) may be NULL, not both. A
 * scalar bound is a 1-element buffer with all-zero strides. */
int hc_clamp(hc_ctx* ctx, int dtype, const void* a, const hc_strides* as, const void* lo,
             const hc_strides* ls, const void* hi, const hc_strides* hs, void* out);

/* Backend.adamW (Backend.swift:818-892), one fused pass that reproduces the base class's
 * op-by-op composition bit for bit (every intermediate rounded to `dtype`); writes the new
 * parameter and both new moments. step is the 1-based update count as a Float. */
int hc_adamw(hc_ctx* ctx, int dtype, const void* param, const void* grad, const void* moment1,
             const void* moment2, float beta1, float beta2, float eps, float weight_decay, float lr,
             float step, size_t count, void* out_param, void* out_moment1, void* out_moment2);

/* Backend.when (Backend.swift:633-641; CPU BackendCPU.swift:1190-1220); a scalar branch is
 * a 1-element buffer with all-zero strides, as CPUBackend.tensorOrScalarData makes it. */
int hc_when(hc_ctx* ctx, int dtype, const void* mask, const hc_strides* ms, const void* a,
            const hc_strides* as, const void* b, const hc_strides* bs, void* out);

/* Backend.matmul / batchedMatmul (Backend.swift:650-669; CPU BackendCPU.swift:1222-1313).
 * rows/inner/cols are M/K/N after the transposes; A is [M,K] ([K,M] if trans_a), B is
 * [K,N] ([N,K] if trans_b), C is [M,N] ([N,M] if trans_out); matrix m of the batch is at
 * element offsets m*M*K, m*K*N, m*M*N. fp16 accumulates in fp32 and rounds once; fp16 and fp32
 * run on the matrix cores, int64 (wrapping sums) on the vector ALU. */
int hc_matmul(hc_ctx* ctx, int dtype, int64_t batch, const void* a, int trans_a, const void* b,
              int trans_b, int trans_out, int64_t rows, int64_t inner, int64_t cols, void* out);

/* Backend.triangular (Backend.swift:674-680; CPU BackendCPU.swift:1315-1348). */
int hc_triangular(hc_ctx* ctx, int dtype, const void* in, void* out, int64_t batch,
                  int64_t rows, int64_t cols, int upper, int64_t offset);

/* Backend.constant (Backend.swift:787-791; CPU BackendCPU.swift:1796-1815). */
int hc_fill(hc_ctx* ctx, int dtype, float vf, int64_t vi, void* out, size_t count);

/* Backend.axisPermutation (Backend.swift:803-805; CPU BackendCPU.swift:1831-1849):
 * `perm` and `shape` are host arrays of ndim entries; out is int64[prod(shape)]. */
int hc_axis_permutation(hc_ctx* ctx, const int64_t* perm, const int64_t* shape, int ndim,
                        void* out);

/* The gather that Tensor.t / swap / move / PermuteAxes issue right after axisPermutation
 * (Index.swift:238-266: gather(axis 0 of [count, inner], indices = the permutation vector)), as one
 * direct copy: out[new axes..., k] = in[old axes..., k] with new axis d = old axis perm[d], `shape`
 * the extents of the permuted (leading) old axes and `inner` the number of untouched trailing
 * elements per position. Same bytes as hc_axis_permutation + hc_gather, without the 8-byte index
 * per element: rows move as 16-byte vectors, a moved innermost axis goes through 64 x 64 LDS tiles.
 * A backend may hand out the index vector lazily and call this when the consumer is that gather. */
int hc_permute(hc_ctx* ctx, int dtype, const void* in, const int64_t* perm, const int64_t* shape,
               int ndim, int64_t inner, void* out);

/* Backend.concat (Backend.swift:777-784; CPU BackendCPU.swift:1768-1794): `inputs` and
 * `inner_counts` are host arrays of n_inputs entries (device pointers / element counts). */
int hc_concat(hc_ctx* ctx, int dtype, const void* const* inputs, const int64_t* inner_counts,
              int n_inputs, int64_t outer, void* out);

#ifdef __cplusplus
}
#endif
#endif /* HCHIP_H */
