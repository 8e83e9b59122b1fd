// Host side of the hchip C ABI (include/hchip.h): context, caching allocator, code-object
// loading and the per-operation launchers. Talks to the HIP runtime only through
// hipMalloc / hipMemcpyAsync / hipModuleLoadData / hipModuleLaunchKernel and friends; the
// kernels are gfx950 code objects built with `hipcc --genco` and embedded in this library
// (embed.S), so this file compiles with any host C++ compiler.
#ifndef __HIP_PLATFORM_AMD__
#define __HIP_PLATFORM_AMD__ 1
#endif
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <cmath>
#include <map>
#include <unordered_set>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/hchip.h"
#include "kargs.h"

extern "C" {
extern const unsigned char hc_image_elementwise[], hc_image_elementwise_end[];
extern const unsigned char hc_image_reduce[], hc_image_reduce_end[];
extern const unsigned char hc_image_gather[], hc_image_gather_end[];
extern const unsigned char hc_image_scan[], hc_image_scan_end[];
extern const unsigned char hc_image_attention[], hc_image_attention_end[];
extern const unsigned char hc_image_gemm[], hc_image_gemm_end[];
extern const unsigned char hc_image_gemm_f16_fast[], hc_image_gemm_f16_fast_end[];
extern const unsigned char hc_image_gemm_dma[], hc_image_gemm_dma_end[];
extern const unsigned char hc_image_gemm_dma2[], hc_image_gemm_dma2_end[];
extern const unsigned char hc_image_gemm_mi16[], hc_image_gemm_mi16_end[];
extern const unsigned char hc_image_gemm_dma_m[], hc_image_gemm_dma_m_end[];
extern const unsigned char hc_image_gemm_dma2_m_f16[], hc_image_gemm_dma2_m_f16_end[];
extern const unsigned char hc_image_gemm_dma2_m_f32[], hc_image_gemm_dma2_m_f32_end[];
extern const unsigned char hc_image_gemm_mi16_m[], hc_image_gemm_mi16_m_end[];
}

// noalloc.hip: looks up this device's copy of the library's fixed scratch array (device current)
int hc_noalloc_setup(int device);

struct hc_module {
  hipModule_t mod;
};
struct hc_function {
  hipFunction_t fn;
};
struct hc_event {
  hipEvent_t ev;
};

// A captured recording plus the buffers it owns: `parked` holds, by bucket size, blocks that
// were freed but must stay out of the general pool while the graph exists.
// One entry of a recording in progress. While a capture runs, kernels are not handed to the
// stream one by one: they are listed here, in call order, with the caller-visible buffers they
// read and write, and hc_capture_end rewrites the list (producer / consumer chains whose
// intermediate results nobody else reads become one kernel, see fuse_recording) before it
// enqueues what is left on the capturing stream.
struct hc_pending {
  enum Kind { KERNEL, RAW_KERNEL, COPY_D2D, FREE } kind = KERNEL;
  hipFunction_t fn = nullptr;
  std::string name;                    // KERNEL: the built-in kernel's name
  uint32_t grid[3] = {1, 1, 1}, block[3] = {HCK_BLOCK, 1, 1}, shared = 0;
  std::vector<char> args;              // the kernel's by-value argument struct
  void* dst = nullptr;                 // COPY_D2D / FREE
  const void* src = nullptr;
  size_t bytes = 0;
  // Buffers of the operation this launch belongs to (OpNote). known == false: the entry point
  // declared nothing, so the launch may touch anything and nothing is moved across it.
  bool known = false;
  std::vector<const void*> reads;
  std::vector<const void*> writes;
  // what the rewrite needs to know about the operations it can merge
  enum Tag { NONE, GEMM, PRODUCT, BMM, PERMUTE, ADD, GELU, CAST, NORMALIZE, LOG_SOFTMAX, SCALAR, MUL_ADD, EXP, SOFTMAX_CHAIN, ARG_REDUCE, GATHER_ONE } tag = NONE;
  int dtype = 0;                       // element type of the output
  int src_dtype = 0;                   // CAST: element type of the input
  uint64_t rows = 0, cols = 0;         // GEMM: M, N; ADD: leading x trailing extent; GELU, CAST: 1 x count
  const void* in0 = nullptr;           // ADD: a; GELU, CAST: input
  const void* in1 = nullptr;           // ADD: b
  int add_form = 0;                    // ADD: 1 = b is a row of `cols` elements repeated over the rows,
                                       //      2 = a is such a row, 3 = both dense
  // NORMALIZE (fp32, a wave per row) / LOG_SOFTMAX: rows x cols, in0; sf = eps; lanes of a row's team
  // SCALAR: out = in0 (op) sf over `cols` elements, op = HC_ADD or HC_MUL as the kernel computes it
  // MUL_ADD: out = in0 * in1 + in2 with in0 dense [rows, cols] and in1, in2 rows of `cols` elements
  // EXP: ElemwiseOp.exp over `cols` elements of in0
  // BMM: a batched product in one launch of a direct-to-LDS kernel (operands in the argument struct);
  //   stays a BMM when the rewrite has made it read or write through a swap of the batch axes
  // ARG_REDUCE: argmax / argmin (op) over the rows of a dense rows x cols input (in0, of type dtype) by one
  //   launch of a row kernel with teams of `lanes` lanes; out holds rows int64 indices
  // GATHER_ONE: out[r] = in0[r * cols + in1[r]] for rows rows, in1 dense int64 indices
  // SOFTMAX_CHAIN: the merged [scale] [mask] logSoftmax [exp] row kernel (rows x cols, lanes; args hck_softmax_chain_args)
  // PERMUTE (row form): in0 -> out; axis d of the dense output has extent pext[d] and lies at
  // stride pstr[d] (elements) in the source, the last axis contiguous in both
  int pn = 0;
  uint64_t pext[HC_MAX_DIMS + 1] = {0}, pstr[HC_MAX_DIMS + 1] = {0};
  const void* in2 = nullptr;
  float sf = 0.0f;
  int op = 0;
  int lanes = 0;
  void* out = nullptr;
  bool dropped = false;                // merged into another entry
  bool merged = false;                 // the rewrite's own launch: stands where the last entry of its chain stood
};

struct hc_graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  std::unordered_map<size_t, std::vector<void*>> parked;
  // HCHIP_GRAPH_AS_LAUNCHES=1 at hc_capture_end: the rewritten list, replayed launch by launch
  // instead of through hipGraphLaunch (for kernel traces: the tracer of this ROCm release aborts
  // inside hipGraphLaunch)
  std::vector<hc_pending> launches;
};

// Switches for measurements and tests (the names are those of the environment variables that
// give them their first value when a context is created; hc_debug_set changes one later). Plain
// data: an entry point copies the struct under the context's mutex and works on its copy, so a
// thread that flips a switch never races a thread that launches.
struct hc_switches {
  char gemm_tile[16] = "";      // HCHIP_GEMM_TILE=general|<BM>x<BN>: overrides the tile choice
  char gemm_kernel[16] = "";    // HCHIP_GEMM_KERNEL=dma|dma2|mi16|staged: the pipeline
  char gemm_ring[8] = "";       // HCHIP_GEMM_RING=4|2: ring-of-four variant of the smallest tiles forced / off
  char gemm_one[8] = "";        // HCHIP_GEMM_ONE=0: no single-slice variants
  bool gemm_no_peel = false;    // HCHIP_GEMM_NO_PEEL: no body-plus-fringes split
  bool gemm_no_direct = false;  // HCHIP_GEMM_NO_DIRECT: unaligned operands through padded copies
  bool gemm_no_repitch = false; // HCHIP_GEMM_NO_REPITCH: ... or not even those (general kernel)
  bool gemm_band = false;       // HCHIP_GEMM_BAND: plain band order of tiles instead of XCD rectangles
  bool no_fusion = false;       // HCHIP_NO_FUSION: recordings are enqueued as they were issued
  bool recording_log = false;   // HCHIP_RECORDING_LOG: the launches of a recording, to stderr
  bool graph_as_launches = false;  // HCHIP_GRAPH_AS_LAUNCHES: replays issue their launches one by one
};

static bool switch_is_on(const char* v) { return v && *v && strcmp(v, "0") != 0; }

// Sets the switch called `name` from `value` (NULL or "" = default). False for an unknown name.
static bool set_switch(hc_switches& sw, const char* name, const char* value) {
  struct Text { const char* name; char* dst; size_t cap; };
  const Text texts[] = {{"HCHIP_GEMM_TILE", sw.gemm_tile, sizeof(sw.gemm_tile)},
                        {"HCHIP_GEMM_KERNEL", sw.gemm_kernel, sizeof(sw.gemm_kernel)},
                        {"HCHIP_GEMM_RING", sw.gemm_ring, sizeof(sw.gemm_ring)},
                        {"HCHIP_GEMM_ONE", sw.gemm_one, sizeof(sw.gemm_one)}};
  for (const Text& t : texts)
    if (strcmp(name, t.name) == 0) {
      snprintf(t.dst, t.cap, "%s", value ? value : "");
      return true;
    }
  struct Flag { const char* name; bool* dst; };
  const Flag flags[] = {{"HCHIP_GEMM_NO_PEEL", &sw.gemm_no_peel},     {"HCHIP_GEMM_NO_DIRECT", &sw.gemm_no_direct},
                        {"HCHIP_GEMM_NO_REPITCH", &sw.gemm_no_repitch}, {"HCHIP_GEMM_BAND", &sw.gemm_band},
                        {"HCHIP_NO_FUSION", &sw.no_fusion},           {"HCHIP_RECORDING_LOG", &sw.recording_log},
                        {"HCHIP_GRAPH_AS_LAUNCHES", &sw.graph_as_launches}};
  for (const Flag& f : flags)
    if (strcmp(name, f.name) == 0) {
      *f.dst = switch_is_on(value);
      return true;
    }
  return false;
}
static const char* const kSwitchNames[] = {"HCHIP_GEMM_TILE",      "HCHIP_GEMM_KERNEL",     "HCHIP_GEMM_RING",
                                           "HCHIP_GEMM_ONE",       "HCHIP_GEMM_NO_PEEL",    "HCHIP_GEMM_NO_DIRECT",
                                           "HCHIP_GEMM_NO_REPITCH", "HCHIP_GEMM_BAND",       "HCHIP_NO_FUSION",
                                           "HCHIP_RECORDING_LOG",  "HCHIP_GRAPH_AS_LAUNCHES"};

struct hc_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  std::mutex mu;
  hc_switches sw;                        // guarded by mu
  std::vector<hipModule_t> modules;
  std::unordered_map<std::string, hipFunction_t> functions;
  std::unordered_set<std::string> functions_missing;   // names no embedded code object has
  std::unordered_map<size_t, std::vector<void*>> free_blocks;
  std::map<void*, size_t> live;          // blocks handed out: base -> bucket size, ordered by address
  size_t bytes_in_use = 0, bytes_cached = 0;
  hipDeviceProp_t props;
  hc_graph* capturing = nullptr;                      // the recording in progress, if any
  std::unordered_map<void*, hc_graph*> block_owner;   // blocks reserved for a graph
  std::vector<hc_graph*> graphs;
  std::vector<hc_graph*> doomed;   // hc_graph_destroy during a capture: destroyed when the capture ends
  // Small host-to-device uploads go through pinned memory so that they need no host-side wait:
  // two halves used in turn, each guarded by an event recorded when the upload path leaves it.
  char* stage = nullptr;
  size_t stage_off = 0;
  int stage_cur = 0;
  hipEvent_t stage_ev[2] = {nullptr, nullptr};
  bool stage_busy[2] = {false, false};
  std::vector<hipEvent_t> wait_events;  // spare events of blocking transfers (waited for outside the mutex)
  bool lazy = false;                    // launches are listed, not enqueued (see hc_pending): a capture, or batching
  bool rewrite = false;                 // the capture in progress will rewrite its list (decided when it begins)
  std::vector<hc_pending> pending;
  // hc_set_batching: outside a capture, launches are listed too and enqueued batch by batch, each
  // batch rewritten like a recording. Blocks released while their batch is listed wait here, by
  // bucket size, and go back to the pool when the batch has been enqueued.
  size_t batch_limit = 0;               // launches per batch at most; 0 = every launch is enqueued at once
  size_t batch_idle_after = 0;          // > 0: a list this long is also enqueued when the stream has run dry (see hc_free)
  size_t batch_idle_now = 0;            // ... the length that applies at the moment (see flush_batch_locked)
  std::unordered_set<void*> batch_born; // blocks handed out since the last batch was enqueued and still in use
  // "has the stream run dry" without a call into the runtime: behind every batch a one-lane
  // kernel stores the batch's number into pinned host memory, which hc_free compares with the
  // number of the last batch it enqueued
  uint64_t* batch_done = nullptr;
  uint64_t batch_seq = 0;
  size_t batch_launches = 0;            // launches in the list now
  std::unordered_map<size_t, std::vector<void*>> batch_parked;
  size_t batch_parked_bytes = 0;
  uint64_t batch_listed = 0, batch_enqueued = 0;   // launches and copies, since the context was created
  int batch_failed = 0;                 // status of a batch that could not be enqueued, until a call has reported it
  std::string batch_failed_why;
  // buffers whose only writer and only reader were merged away by the rewrite of the recording in
  // progress: no launch of the graph touches them, so they need not stay reserved for it
  std::vector<std::pair<void*, size_t>> dead;
};
static const size_t kStageHalf = 2u << 20;    // bytes per half of the staging buffer
static const size_t kStageMax = 256u << 10;   // largest upload that is staged
static const size_t kBatchParkedMax = (size_t)8 << 30;   // batching: released bytes a listed batch may hold back

static thread_local std::string g_last_error;
static int alloc_batch_flag_locked(hc_ctx* ctx);

static int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

static int hip_fail(hipError_t e, const char* what) {
  return fail(HC_ERR_HIP_BASE + (int)e, "%s: %s (%s)", what, hipGetErrorString(e), hipGetErrorName(e));
}

#define HIP_TRY(expr)                              \
  do {                                             \
    hipError_t _e = (expr);                        \
    if (_e != hipSuccess) return hip_fail(_e, #expr); \
  } while (0)

#define HC_TRY(expr)          \
  do {                        \
    int _s = (expr);          \
    if (_s != HC_OK) return _s; \
  } while (0)

#define REQUIRE(cond, ...)                                   \
  do {                                                       \
    if (!(cond)) return fail(HC_ERR_INVALID, __VA_ARGS__);   \
  } while (0)

extern "C" const char* hc_last_error_string(void) { return g_last_error.c_str(); }

// ------------------------------------------------------------------ context

static int load_image(hc_ctx* ctx, const unsigned char* begin, const unsigned char* end, const char* name) {
  if (end <= begin) return fail(HC_ERR_LOAD, "embedded code object '%s' is empty", name);
  hipModule_t mod;
  hipError_t e = hipModuleLoadData(&mod, begin);
  if (e != hipSuccess)
    return fail(HC_ERR_LOAD, "hipModuleLoadData(%s): %s", name, hipGetErrorString(e));
  ctx->modules.push_back(mod);
  return HC_OK;
}

extern "C" int hc_init(int device, hc_ctx** out) {
  REQUIRE(out != nullptr, "hc_init: out is null");
  *out = nullptr;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0)
    return fail(HC_ERR_NO_DEVICE, "no HIP device available (%s)", hipGetErrorString(e));
  REQUIRE(device >= 0 && device < count, "hc_init: device %d out of range (have %d)", device, count);
  HIP_TRY(hipSetDevice(device));
  hc_ctx* ctx = new hc_ctx();
  ctx->device = device;
  for (const char* name : kSwitchNames) set_switch(ctx->sw, name, getenv(name));
  if (const char* v = getenv("HCHIP_BATCHING")) {   // hc_set_batching from the environment: <max>[,<idle_after>]
    char* end = nullptr;
    ctx->batch_limit = (size_t)strtoull(v, &end, 10);
    ctx->batch_idle_after = end && *end == ',' ? (size_t)strtoull(end + 1, nullptr, 10) : 0;
    ctx->batch_idle_now = ctx->batch_idle_after;
    ctx->lazy = ctx->batch_limit > 0;
  }
  e = hipGetDeviceProperties(&ctx->props, device);
  if (e != hipSuccess) {
    delete ctx;
    return hip_fail(e, "hipGetDeviceProperties");
  }
  if (strncmp(ctx->props.gcnArchName, "gfx950", 6) != 0) {
    int s = fail(HC_ERR_LOAD, "device %d is %s; the embedded kernels are built for gfx950 only", device,
                 ctx->props.gcnArchName);
    delete ctx;
    return s;
  }
  {  // (after the architecture check: on another device the lookup fails with a less telling message)
    const int s = hc_noalloc_setup(device);
    if (s != HC_OK) {
      delete ctx;
      return s;
    }
  }
  e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
  if (e != hipSuccess) {
    delete ctx;
    return hip_fail(e, "hipStreamCreateWithFlags");
  }
  // (without the staging buffer uploads simply stay synchronous; HCHIP_NO_STAGING=1 asks for that)
  if (getenv("HCHIP_NO_STAGING")) {
    ctx->stage = nullptr;
  } else if (hipHostMalloc((void**)&ctx->stage, 2 * kStageHalf, hipHostMallocDefault) != hipSuccess) {
    ctx->stage = nullptr;
    (void)hipGetLastError();
  } else if (hipEventCreateWithFlags(&ctx->stage_ev[0], hipEventDisableTiming) != hipSuccess ||
             hipEventCreateWithFlags(&ctx->stage_ev[1], hipEventDisableTiming) != hipSuccess) {
    (void)hipHostFree(ctx->stage);
    ctx->stage = nullptr;
    (void)hipGetLastError();
  }
  int s = load_image(ctx, hc_image_elementwise, hc_image_elementwise_end, "elementwise");
  if (s == HC_OK) s = load_image(ctx, hc_image_reduce, hc_image_reduce_end, "reduce");
  if (s == HC_OK) s = load_image(ctx, hc_image_gather, hc_image_gather_end, "gather");
  if (s == HC_OK) s = load_image(ctx, hc_image_scan, hc_image_scan_end, "scan");
  if (s == HC_OK) s = load_image(ctx, hc_image_attention, hc_image_attention_end, "attention");
  if (s == HC_OK) s = load_image(ctx, hc_image_gemm, hc_image_gemm_end, "gemm");
  if (s == HC_OK) s = load_image(ctx, hc_image_gemm_f16_fast, hc_image_gemm_f16_fast_end, "gemm_f16_fast");
  if (s == HC_OK) s = load_image(ctx, hc_image_gemm_dma, hc_image_gemm_dma_end, "gemm_dma");
  if (s == HC_OK) s = load_image(ctx, hc_image_gemm_dma2, hc_image_gemm_dma2_end, "gemm_dma2");
  if (s == HC_OK) s = load_image(ctx, hc_image_gemm_mi16, hc_image_gemm_mi16_end, "gemm_mi16");
  if (s == HC_OK) s = load_image(ctx, hc_image_gemm_dma_m, hc_image_gemm_dma_m_end, "gemm_dma_m");
  if (s == HC_OK) s = load_image(ctx, hc_image_gemm_dma2_m_f16, hc_image_gemm_dma2_m_f16_end, "gemm_dma2_m_f16");
  if (s == HC_OK) s = load_image(ctx, hc_image_gemm_dma2_m_f32, hc_image_gemm_dma2_m_f32_end, "gemm_dma2_m_f32");
  if (s == HC_OK) s = load_image(ctx, hc_image_gemm_mi16_m, hc_image_gemm_mi16_m_end, "gemm_mi16_m");
  if (s == HC_OK && ctx->batch_idle_after > 0) s = alloc_batch_flag_locked(ctx);
  if (s != HC_OK) {
    hc_shutdown(ctx);
    return s;
  }
  *out = ctx;
  return HC_OK;
}

extern "C" void hc_shutdown(hc_ctx* ctx) {
  if (!ctx) return;
  (void)hipSetDevice(ctx->device);
  if (ctx->capturing) {
    hipGraph_t dropped = nullptr;
    (void)hipStreamEndCapture(ctx->stream, &dropped);
    if (dropped) (void)hipGraphDestroy(dropped);
    (void)hipGetLastError();
  }
  if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
  for (hc_graph* g : ctx->graphs) {
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    for (auto& kv : g->parked)
      for (void* p : kv.second) (void)hipFree(p);
    delete g;
  }
  for (auto& kv : ctx->free_blocks)
    for (void* p : kv.second) (void)hipFree(p);
  for (auto& kv : ctx->batch_parked)   // (a batch still listed is dropped: nobody can read its results any more)
    for (void* p : kv.second) (void)hipFree(p);
  for (auto& kv : ctx->live) (void)hipFree(kv.first);
  for (hipModule_t m : ctx->modules) (void)hipModuleUnload(m);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  for (hipEvent_t ev : ctx->stage_ev)
    if (ev) (void)hipEventDestroy(ev);
  for (hipEvent_t ev : ctx->wait_events) (void)hipEventDestroy(ev);
  if (ctx->stage) (void)hipHostFree(ctx->stage);
  if (ctx->batch_done) (void)hipHostFree(ctx->batch_done);
  delete ctx;
}

extern "C" int hc_debug_set(hc_ctx* ctx, const char* name, const char* value) {
  REQUIRE(ctx && name, "hc_debug_set: null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  REQUIRE(set_switch(ctx->sw, name, value), "hc_debug_set: no switch called '%s'", name);
  return HC_OK;
}

// The context's switches as they are now (a copy: see hc_switches).
static hc_switches switches_of(hc_ctx* ctx) {
  std::lock_guard<std::mutex> lock(ctx->mu);
  return ctx->sw;
}

// The block of this context that holds the address `p`: its base and size, or {nullptr, 0}.
// Caller holds the mutex.
static std::pair<void*, size_t> block_of_locked(const hc_ctx* ctx, const void* p) {
  auto it = ctx->live.upper_bound(const_cast<void*>(p));
  if (it == ctx->live.begin()) return {nullptr, 0};
  --it;
  if ((const char*)p < (const char*)it->first + it->second) return {it->first, it->second};
  return {nullptr, 0};
}

extern "C" int hc_get_device_info(hc_ctx* ctx, hc_device_info* out) {
  REQUIRE(ctx && out, "hc_get_device_info: null argument");
  memset(out, 0, sizeof(*out));
  snprintf(out->name, sizeof(out->name), "%s", ctx->props.name);
  snprintf(out->arch, sizeof(out->arch), "%s", ctx->props.gcnArchName);
  out->compute_units = ctx->props.multiProcessorCount;
  out->clock_mhz = ctx->props.clockRate / 1000;
  out->wavefront_size = ctx->props.warpSize;
  out->lds_bytes_per_block = (int)ctx->props.sharedMemPerBlock;
  out->total_mem = ctx->props.totalGlobalMem;
  return HC_OK;
}

// ------------------------------------------------------------------ memory

// Bucket sizes: powers of two up to 1 MiB, multiples of 2 MiB above. A freed block goes
// back to its bucket and is handed out again by a later hc_malloc; both happen in host
// program order and all work runs on one in-order stream, so a kernel enqueued before the
// free always finishes before a kernel enqueued after the re-allocation touches the block.
static size_t bucket_size(size_t bytes) {
  if (bytes < 256) return 256;
  if (bytes <= ((size_t)1 << 20)) {
    size_t b = 256;
    while (b < bytes) b <<= 1;
    return b;
  }
  const size_t g = (size_t)2 << 20;
  return (bytes + g - 1) / g * g;
}

enum BatchEnd { BATCH_END_OTHER, BATCH_END_WAIT, BATCH_END_IDLE };
static int flush_batch_locked(hc_ctx* ctx, BatchEnd why = BATCH_END_OTHER);
static int batch_grew_locked(hc_ctx* ctx);

static void release_cache_locked(hc_ctx* ctx) {
  for (auto& kv : ctx->free_blocks)
    for (void* p : kv.second) (void)hipFree(p);
  ctx->free_blocks.clear();
  ctx->bytes_cached = 0;
}

extern "C" int hc_malloc(hc_ctx* ctx, size_t bytes, void** out) {
  REQUIRE(ctx && out, "hc_malloc: null argument");
  *out = nullptr;
  const size_t b = bucket_size(bytes);
  std::lock_guard<std::mutex> lock(ctx->mu);
  auto it = ctx->free_blocks.find(b);
  void* p = nullptr;
  if (ctx->capturing && !ctx->rewrite) {
    // blocks this recording already owns come first; anything else it takes becomes its own.
    // (Not while the recording's list is going to be rewritten: there every buffer stays a
    // buffer of its own until the recording ends, so that an operation can be moved next to its
    // consumer without running into a block that was handed out again in between. The price is a
    // footprint of the sum of all intermediates instead of their peak.)
    auto& parked = ctx->capturing->parked[b];
    if (!parked.empty()) {
      p = parked.back();
      parked.pop_back();
      ctx->live[p] = b;
      ctx->bytes_in_use += b;
      *out = p;
      return HC_OK;
    }
  }
  if (it != ctx->free_blocks.end() && !it->second.empty()) {
    p = it->second.back();
    it->second.pop_back();
    ctx->bytes_cached -= b;
  } else {
    (void)hipSetDevice(ctx->device);
    hipError_t e = hipMalloc(&p, b);
    if (e != hipSuccess && !ctx->capturing) {
      // Enqueue what is listed (its released blocks come back with it), give cached blocks back
      // to the driver and retry once.
      (void)hipGetLastError();
      (void)flush_batch_locked(ctx);
      (void)hipStreamSynchronize(ctx->stream);
      release_cache_locked(ctx);
      e = hipMalloc(&p, b);
    }
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return fail(HC_ERR_ALLOC, "hipMalloc(%zu bytes) failed: %s", b, hipGetErrorString(e));
    }
  }
  ctx->live[p] = b;
  ctx->bytes_in_use += b;
  if (ctx->capturing) ctx->block_owner[p] = ctx->capturing;
  else if (ctx->lazy && ctx->batch_idle_after > 0) ctx->batch_born.insert(p);
  *out = p;
  return HC_OK;
}

extern "C" int hc_free(hc_ctx* ctx, void* ptr) {
  REQUIRE(ctx, "hc_free: null context");
  if (!ptr) return HC_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  auto it = ctx->live.find(ptr);
  REQUIRE(it != ctx->live.end(), "hc_free: %p was not allocated by this context (or freed twice)", ptr);
  const size_t b = it->second;
  ctx->live.erase(it);
  ctx->bytes_in_use -= b;
  if (ctx->lazy) {   // from here on nobody reads this buffer: what the rewrite of the recording looks for
    hc_pending e;
    e.kind = hc_pending::FREE;
    e.dst = ptr;
    e.bytes = b;
    ctx->pending.push_back(std::move(e));
  }
  auto owner = ctx->block_owner.find(ptr);
  if (owner != ctx->block_owner.end()) {
    // recorded kernels keep using this block on every replay
    owner->second->parked[b].push_back(ptr);
  } else if (ctx->capturing) {
    // allocated before the capture, released inside it: the recording read (or wrote) it
    ctx->block_owner[ptr] = ctx->capturing;
    ctx->capturing->parked[b].push_back(ptr);
  } else if (ctx->lazy) {
    // batching: listed launches may still use it, so it stays out of the pool until they are enqueued
    ctx->batch_parked[b].push_back(ptr);
    ctx->batch_parked_bytes += b;
    ctx->batch_born.erase(ptr);
    if (ctx->batch_parked_bytes > kBatchParkedMax) return flush_batch_locked(ctx);
    if (ctx->batch_launches >= ctx->batch_limit && ctx->batch_born.size() <= 1) return flush_batch_locked(ctx);   // (a full list, see batch_grew_locked)
    // A device that has nothing left to do gains nothing from a longer list. The place to cut
    // the list is where the program holds at most one result of the listed launches (between
    // two layers of a model, say): every other intermediate has been released, so no chain that
    // the rewrite could merge is open. There, once the list is long enough to be worth a
    // rewrite, look whether the device is past the middle of the last batch (or has never had one): the
    // list then goes out while the rest of that batch runs.
    if (ctx->batch_idle_after > 0 && ctx->batch_launches >= ctx->batch_idle_now && ctx->batch_born.size() <= 1 &&
        ctx->batch_done && __atomic_load_n(ctx->batch_done, __ATOMIC_ACQUIRE) == ctx->batch_seq)
      return flush_batch_locked(ctx, BATCH_END_IDLE);
  } else {
    ctx->free_blocks[b].push_back(ptr);
    ctx->bytes_cached += b;
  }
  return HC_OK;
}

extern "C" int hc_trim(hc_ctx* ctx) {
  REQUIRE(ctx, "hc_trim: null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  REQUIRE(!ctx->capturing, "hc_trim: not allowed while capturing");
  HC_TRY(flush_batch_locked(ctx));
  HIP_TRY(hipStreamSynchronize(ctx->stream));
  release_cache_locked(ctx);
  return HC_OK;
}

extern "C" int hc_mem_stats(hc_ctx* ctx, size_t* in_use, size_t* cached) {
  REQUIRE(ctx, "hc_mem_stats: null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (in_use) *in_use = ctx->bytes_in_use;
  if (cached) *cached = ctx->bytes_cached;
  return HC_OK;
}

extern "C" int hc_host_alloc(hc_ctx* ctx, size_t bytes, void** out) {
  REQUIRE(ctx && out, "hc_host_alloc: null argument");
  *out = nullptr;
  hipError_t e = hipHostMalloc(out, bytes ? bytes : 1, hipHostMallocDefault);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(HC_ERR_ALLOC, "hipHostMalloc(%zu bytes) failed: %s", bytes, hipGetErrorString(e));
  }
  return HC_OK;
}

extern "C" int hc_host_free(hc_ctx* ctx, void* ptr) {
  REQUIRE(ctx, "hc_host_free: null context");
  if (ptr) HIP_TRY(hipHostFree(ptr));
  return HC_OK;
}

// An event recorded on the stream now (mutex held by the caller), from the context's spare list.
static int record_wait_event_locked(hc_ctx* ctx, hipEvent_t* out) {
  hipEvent_t ev = nullptr;
  if (!ctx->wait_events.empty()) {
    ev = ctx->wait_events.back();
    ctx->wait_events.pop_back();
  } else {
    HIP_TRY(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
  }
  hipError_t e = hipEventRecord(ev, ctx->stream);
  if (e != hipSuccess) {
    ctx->wait_events.push_back(ev);
    return hip_fail(e, "hipEventRecord");
  }
  *out = ev;
  return HC_OK;
}

// Waits for `ev` WITHOUT the mutex, so that other threads keep allocating and enqueueing while
// this one sleeps, then puts the event back.
static int wait_event_unlocked(hc_ctx* ctx, hipEvent_t ev) {
  hipError_t e = hipEventSynchronize(ev);
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    ctx->wait_events.push_back(ev);
  }
  if (e != hipSuccess) return hip_fail(e, "hipEventSynchronize");
  return HC_OK;
}

// Batching: whether a launch that is listed, not yet enqueued, may read or write the block that
// holds `p` (or `p` itself, for memory this context did not allocate). Caller holds the mutex.
static bool batch_touches_locked(const hc_ctx* ctx, const void* p) {
  std::pair<void*, size_t> blk = block_of_locked(ctx, p);
  if (!blk.first) blk = {const_cast<void*>(p), 1};
  for (const hc_pending& e : ctx->pending) {
    if (e.kind == hc_pending::FREE) continue;
    if (!e.known) return true;
    for (const void* q : e.reads)
      if ((const char*)q >= (const char*)blk.first && (const char*)q < (const char*)blk.first + blk.second) return true;
    for (const void* q : e.writes)
      if ((const char*)q >= (const char*)blk.first && (const char*)q < (const char*)blk.first + blk.second) return true;
  }
  return false;
}

static int copy(hc_ctx* ctx, void* dst, const void* src, size_t bytes, hipMemcpyKind kind, bool wait) {
  REQUIRE(ctx, "memcpy: null context");
  if (bytes == 0) return HC_OK;
  REQUIRE(dst && src, "memcpy: null pointer");
  hipEvent_t ev = nullptr;
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    REQUIRE(!ctx->capturing || kind == hipMemcpyDeviceToDevice,
            "memcpy: host transfers are not allowed while capturing (upload inputs before hc_capture_begin)");
    // Batching: a transfer is enqueued at once, ahead of the launches still listed. An upload
    // may overtake them when none of them uses the block it fills (a fresh buffer: constants and
    // index vectors in the middle of a forward pass); everything else enqueues the list first.
    if (!ctx->capturing && !ctx->pending.empty() && kind != hipMemcpyDeviceToDevice &&
        (kind != hipMemcpyHostToDevice || batch_touches_locked(ctx, dst)))
      HC_TRY(flush_batch_locked(ctx, BATCH_END_WAIT));
    if (kind == hipMemcpyHostToDevice && wait && bytes <= kStageMax && ctx->stage) {
      // The caller may reuse `src` as soon as this returns: copy it into pinned memory and let the
      // stream pick it up from there. No wait, so the device keeps running what is already queued
      // (index vectors of slices, small constants in the middle of a forward pass).
      if (ctx->stage_off + bytes > kStageHalf) {
        HIP_TRY(hipEventRecord(ctx->stage_ev[ctx->stage_cur], ctx->stream));
        ctx->stage_busy[ctx->stage_cur] = true;
        ctx->stage_cur ^= 1;
        ctx->stage_off = 0;
        if (ctx->stage_busy[ctx->stage_cur]) HIP_TRY(hipEventSynchronize(ctx->stage_ev[ctx->stage_cur]));
        ctx->stage_busy[ctx->stage_cur] = false;
      }
      char* slot = ctx->stage + (size_t)ctx->stage_cur * kStageHalf + ctx->stage_off;
      memcpy(slot, src, bytes);
      ctx->stage_off += (bytes + 63) & ~(size_t)63;
      HIP_TRY(hipMemcpyAsync(dst, slot, bytes, kind, ctx->stream));
      return HC_OK;
    }
    if (!wait) {
      if (ctx->lazy) {   // (only device-to-device copies get here while capturing)
        hc_pending e;
        e.kind = hc_pending::COPY_D2D;
        e.dst = dst;
        e.src = src;
        e.bytes = bytes;
        e.known = true;
        e.reads = {src};
        e.writes = {dst};
        ctx->pending.push_back(std::move(e));
        return batch_grew_locked(ctx);
      }
      HIP_TRY(hipMemcpyAsync(dst, src, bytes, kind, ctx->stream));
      return HC_OK;
    }
    // A blocking transfer first lets everything that is already enqueued finish, with the mutex
    // released (a readback at the end of a long queue would otherwise stall every other thread's
    // allocations and launches for the whole drain) ...
    HC_TRY(record_wait_event_locked(ctx, &ev));
  }
  HC_TRY(wait_event_unlocked(ctx, ev));
  {
    // ... and then holds it only for the copy itself. Work that other threads enqueued in the
    // meantime runs before the copy, which is what stream order promises anyway.
    std::lock_guard<std::mutex> lock(ctx->mu);
    REQUIRE(!ctx->capturing, "memcpy: host transfers are not allowed while capturing");
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, kind, ctx->stream));
    HC_TRY(record_wait_event_locked(ctx, &ev));
  }
  return wait_event_unlocked(ctx, ev);
}

extern "C" int hc_memcpy_h2d(hc_ctx* ctx, void* dst, const void* src, size_t bytes) {
  return copy(ctx, dst, src, bytes, hipMemcpyHostToDevice, true);
}
extern "C" int hc_memcpy_d2h(hc_ctx* ctx, void* dst, const void* src, size_t bytes) {
  return copy(ctx, dst, src, bytes, hipMemcpyDeviceToHost, true);
}
extern "C" int hc_memcpy_d2d(hc_ctx* ctx, void* dst, const void* src, size_t bytes) {
  return copy(ctx, dst, src, bytes, hipMemcpyDeviceToDevice, false);
}
extern "C" int hc_memcpy_h2d_async(hc_ctx* ctx, void* dst, const void* src, size_t bytes) {
  return copy(ctx, dst, src, bytes, hipMemcpyHostToDevice, false);
}
extern "C" int hc_memcpy_d2h_async(hc_ctx* ctx, void* dst, const void* src, size_t bytes) {
  return copy(ctx, dst, src, bytes, hipMemcpyDeviceToHost, false);
}

// ------------------------------------------------------------------ stream / events

extern "C" int hc_sync(hc_ctx* ctx) {
  REQUIRE(ctx, "hc_sync: null context");
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    REQUIRE(!ctx->capturing, "hc_sync: not allowed while capturing");
    HC_TRY(flush_batch_locked(ctx, BATCH_END_WAIT));
  }
  HIP_TRY(hipStreamSynchronize(ctx->stream));
  return HC_OK;
}

extern "C" int hc_event_create(hc_ctx* ctx, hc_event** out) {
  REQUIRE(ctx && out, "hc_event_create: null argument");
  hc_event* ev = new hc_event();
  hipError_t e = hipEventCreate(&ev->ev);
  if (e != hipSuccess) {
    delete ev;
    return hip_fail(e, "hipEventCreate");
  }
  *out = ev;
  return HC_OK;
}

extern "C" int hc_event_record(hc_ctx* ctx, hc_event* ev) {
  REQUIRE(ctx && ev, "hc_event_record: null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  REQUIRE(!ctx->capturing, "hc_event_record: not allowed while capturing");
  HC_TRY(flush_batch_locked(ctx, BATCH_END_WAIT));
  HIP_TRY(hipEventRecord(ev->ev, ctx->stream));
  return HC_OK;
}

extern "C" int hc_event_sync(hc_event* ev) {
  REQUIRE(ev, "hc_event_sync: null event");
  HIP_TRY(hipEventSynchronize(ev->ev));
  return HC_OK;
}

extern "C" int hc_event_query(hc_event* ev) {
  REQUIRE(ev, "hc_event_query: null event");
  hipError_t e = hipEventQuery(ev->ev);
  if (e == hipSuccess) return 0;
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();
    return 1;
  }
  return hip_fail(e, "hipEventQuery");
}

extern "C" int hc_event_elapsed_ms(hc_event* start, hc_event* stop, float* ms) {
  REQUIRE(start && stop && ms, "hc_event_elapsed_ms: null argument");
  HIP_TRY(hipEventElapsedTime(ms, start->ev, stop->ev));
  return HC_OK;
}

extern "C" int hc_event_destroy(hc_event* ev) {
  if (!ev) return HC_OK;
  hipError_t e = hipEventDestroy(ev->ev);
  delete ev;
  if (e != hipSuccess) return hip_fail(e, "hipEventDestroy");
  return HC_OK;
}

extern "C" int hc_launch_host_func(hc_ctx* ctx, void (*fn)(void*), void* user) {
  REQUIRE(ctx && fn, "hc_launch_host_func: null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  REQUIRE(!ctx->capturing, "hc_launch_host_func: not allowed while capturing");
  HC_TRY(flush_batch_locked(ctx, BATCH_END_WAIT));
  HIP_TRY(hipLaunchHostFunc(ctx->stream, fn, user));
  return HC_OK;
}

// ------------------------------------------------------------------ capture / graphs

extern "C" int hc_capture_begin(hc_ctx* ctx) {
  REQUIRE(ctx, "hc_capture_begin: null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  REQUIRE(!ctx->capturing, "hc_capture_begin: a capture is already in progress");
  HC_TRY(flush_batch_locked(ctx));
  // relaxed mode: the allocator may still call hipMalloc for sizes its pool does not hold
  HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
  ctx->capturing = new hc_graph();
  ctx->graphs.push_back(ctx->capturing);
  ctx->lazy = true;   // launches are listed, and enqueued on the capturing stream at hc_capture_end
  ctx->rewrite = !ctx->sw.no_fusion;
  ctx->pending.clear();
  ctx->dead.clear();
  return HC_OK;
}

static void fuse_recording(hc_ctx* ctx);
static int find_kernel_locked(hc_ctx* ctx, const std::string& name, hipFunction_t* out);
static int launch_fn(hc_ctx* ctx, hipFunction_t fn, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx,
                     uint32_t shared, const void* kernarg, size_t kernarg_bytes);

// Enqueues the (rewritten) list of a recording on the capturing stream. Caller holds the lock.
// `mark_at` / `mark_fn` / `mark_args` (batching): a one-lane marker kernel goes out behind the first `mark_at`
// entries that are enqueued.
static int emit_recording_locked(hc_ctx* ctx, std::vector<hc_pending>& list, size_t mark_at = (size_t)-1,
                                 hipFunction_t mark_fn = nullptr, const hck_map_args* mark_args = nullptr) {
  size_t sent = 0;
  for (hc_pending& e : list) {
    if (e.dropped || e.kind == hc_pending::FREE) continue;
    if (sent++ == mark_at && mark_fn) HC_TRY(launch_fn(ctx, mark_fn, 1, 1, 1, HCK_BLOCK, 0, mark_args, sizeof(*mark_args)));
    if (e.kind == hc_pending::KERNEL) {
      HC_TRY(launch_fn(ctx, e.fn, e.grid[0], e.grid[1], 1, HCK_BLOCK, 0, e.args.data(), e.args.size()));
    } else if (e.kind == hc_pending::RAW_KERNEL) {
      size_t n = e.args.size();
      void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, e.args.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &n,
                        HIP_LAUNCH_PARAM_END};
      HIP_TRY(hipModuleLaunchKernel(e.fn, e.grid[0], e.grid[1], e.grid[2], e.block[0], e.block[1], e.block[2],
                                    e.shared, ctx->stream, nullptr, config));
    } else if (e.kind == hc_pending::COPY_D2D) {
      HIP_TRY(hipMemcpyAsync(e.dst, e.src, e.bytes, hipMemcpyDeviceToDevice, ctx->stream));
    }
  }
  return HC_OK;
}

// HCHIP_RECORDING_LOG: the launches of a list as they will be enqueued, to stderr
static void log_launches_locked(const hc_ctx* ctx, const char* what) {
  size_t n = 0;
  for (const hc_pending& e : ctx->pending) {
    if (e.dropped || e.kind == hc_pending::FREE) continue;
    const char* name = e.kind == hc_pending::COPY_D2D ? "(copy)" : "(caller's kernel)";
    for (const auto& kv : ctx->functions)
      if (e.kind == hc_pending::KERNEL && kv.second == e.fn) name = kv.first.c_str();
    fprintf(stderr, "hchip %s %3zu: %s grid %u x %u\n", what, n++, name, e.grid[0], e.grid[1]);
  }
}

// Batching: rewrites the listed launches like a recording and enqueues them; the blocks released
// since the last batch go back to the pool (in stream order behind the launches that used them,
// which is what the pool assumes of every block it holds). Nothing to do outside batching, or
// during a capture (whose list is the capture's). Caller holds the lock.
static int flush_batch_locked(hc_ctx* ctx, BatchEnd why) {
  if (ctx->capturing || ctx->batch_limit == 0) return HC_OK;
  int status = HC_OK;
  // A batch that failed to go out inside a call whose status nobody looks at (hc_free from a
  // destructor) is reported again by the next call that would have enqueued it.
  if (ctx->batch_failed != HC_OK) {
    status = ctx->batch_failed;
    g_last_error = ctx->batch_failed_why;
    ctx->batch_failed = HC_OK;
  }
  if (!ctx->pending.empty()) {
    ctx->lazy = false;
    for (const hc_pending& e : ctx->pending) ctx->batch_listed += e.kind != hc_pending::FREE;
    if (!ctx->sw.no_fusion) fuse_recording(ctx);
    for (const hc_pending& e : ctx->pending) ctx->batch_enqueued += e.kind != hc_pending::FREE && !e.dropped;
    if (ctx->sw.recording_log) log_launches_locked(ctx, "batch");
    // A marker tells the host how far the device has got with this batch: a one-lane kernel behind the first half
    // of the launches that writes the batch's number into pinned host memory, which is what the idle rule of hc_free
    // looks at: the next batch is rewritten and enqueued while the second half still runs, instead of after the
    // device has run dry. (One marker, not a second one behind the batch: its store to host memory makes the
    // device write its caches back, about 17 us on the device per marker in a pass of config 5. And none once the
    // early batches have grown to the limit: a full list goes out whatever the device is doing. After a wait,
    // which starts the early batches over, the number in host memory is at most batch_seq and the device idle.)
    hipFunction_t mark_fn = nullptr;
    const bool marking = ctx->batch_idle_after > 0 && ctx->batch_idle_now < ctx->batch_limit && ctx->batch_done &&
                         find_kernel_locked(ctx, "hc_fill_b8", &mark_fn) == HC_OK;
    hck_map_args mark;
    memset(&mark, 0, sizeof(mark));
    mark.count = 1;
    size_t to_send = 0;
    for (const hc_pending& e : ctx->pending) to_send += e.kind != hc_pending::FREE && !e.dropped;
    if (marking) {
      mark.out = ctx->batch_done;
      mark.i0 = (int64_t)++ctx->batch_seq;
    }
    const int emitted = emit_recording_locked(ctx, ctx->pending, marking ? to_send / 2 : (size_t)-1, mark_fn, &mark);
    if (status == HC_OK) status = emitted;
    ctx->pending.clear();
    ctx->dead.clear();
    if (marking && (emitted != HC_OK || to_send == 0)) {
      // (the marker did not go out inside the list: the host must not wait for a number that no kernel will write)
      const int marked = launch_fn(ctx, mark_fn, 1, 1, 1, HCK_BLOCK, 0, &mark, sizeof(mark));
      if (status == HC_OK) status = marked;
    }
    ctx->lazy = true;
  }
  const bool full = ctx->batch_launches >= ctx->batch_limit;
  ctx->batch_launches = 0;
  ctx->batch_born.clear();
  // An early batch pays for itself when the device would otherwise sit idle until a wait (a program
  // that reads a result after every pass): the first one goes out after idle_after launches. Every
  // early batch doubles the length the next one needs, so that a program that never waits, and
  // whose device runs dry because the host is the slower side, ends up with full batches (fewer
  // rewrites and launches on the host, which is what it is short of); a wait starts over.
  if (status != HC_OK && why != BATCH_END_WAIT) {
    ctx->batch_failed = status;
    ctx->batch_failed_why = g_last_error;
  }
  // (a list that filled up while the device still had half a batch in front of it: the device is the slower side,
  // early batches have nothing to give until the next wait, and the markers they need can stay away)
  if (why == BATCH_END_IDLE) ctx->batch_idle_now = std::min(ctx->batch_idle_now * 2, ctx->batch_limit);
  else if (why == BATCH_END_WAIT) ctx->batch_idle_now = ctx->batch_idle_after;
  else if (full && ctx->batch_idle_after > 0) ctx->batch_idle_now = ctx->batch_limit;
  for (auto& kv : ctx->batch_parked) {
    auto& pool = ctx->free_blocks[kv.first];
    pool.insert(pool.end(), kv.second.begin(), kv.second.end());
    ctx->bytes_cached += kv.first * kv.second.size();
  }
  ctx->batch_parked.clear();
  ctx->batch_parked_bytes = 0;
  return status;
}

static int alloc_batch_flag_locked(hc_ctx* ctx) {
  (void)hipSetDevice(ctx->device);
  hipError_t e = hipHostMalloc((void**)&ctx->batch_done, 64, hipHostMallocDefault);
  if (e != hipSuccess) {
    ctx->batch_done = nullptr;
    return hip_fail(e, "hipHostMalloc (batching's completion flag)");
  }
  *ctx->batch_done = ctx->batch_seq;   // the number of the last batch whose first half the device has run
  return HC_OK;
}

extern "C" int hc_set_batching(hc_ctx* ctx, size_t max_launches, size_t idle_after) {
  REQUIRE(ctx, "hc_set_batching: null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  REQUIRE(!ctx->capturing, "hc_set_batching: not allowed while capturing");
  HC_TRY(flush_batch_locked(ctx));
  if (idle_after > 0 && !ctx->batch_done) HC_TRY(alloc_batch_flag_locked(ctx));
  ctx->batch_limit = max_launches;
  ctx->batch_idle_after = idle_after;
  ctx->batch_idle_now = idle_after;
  ctx->lazy = max_launches > 0;
  return HC_OK;
}

extern "C" int hc_batching_stats(hc_ctx* ctx, uint64_t* listed, uint64_t* enqueued) {
  REQUIRE(ctx, "hc_batching_stats: null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (listed) *listed = ctx->batch_listed;
  if (enqueued) *enqueued = ctx->batch_enqueued;
  return HC_OK;
}

extern "C" int hc_flush(hc_ctx* ctx) {
  REQUIRE(ctx, "hc_flush: null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  REQUIRE(!ctx->capturing, "hc_flush: not allowed while capturing");
  return flush_batch_locked(ctx);
}

// Gives a graph's parked blocks back to the general pool and forgets its ownership of
// blocks that are still live. Caller holds the lock.
static void release_graph_blocks_locked(hc_ctx* ctx, hc_graph* g) {
  for (auto& kv : g->parked)
    for (void* p : kv.second) {
      ctx->free_blocks[kv.first].push_back(p);
      ctx->bytes_cached += kv.first;
    }
  g->parked.clear();
  for (auto it = ctx->block_owner.begin(); it != ctx->block_owner.end();)
    it = it->second == g ? ctx->block_owner.erase(it) : std::next(it);
  for (size_t i = 0; i < ctx->graphs.size(); i++)
    if (ctx->graphs[i] == g) {
      ctx->graphs.erase(ctx->graphs.begin() + i);
      break;
    }
}

static int destroy_graph_locked(hc_ctx* ctx, hc_graph* graph);
static int end_capture_locked(hc_ctx* ctx, hc_graph** out);

static int end_capture(hc_ctx* ctx, hc_graph** out) {
  std::lock_guard<std::mutex> lock(ctx->mu);
  REQUIRE(ctx->capturing, "hc_capture_end: no capture in progress");
  const int status = end_capture_locked(ctx, out);
  std::vector<hc_graph*> doomed;
  doomed.swap(ctx->doomed);
  for (hc_graph* g : doomed) (void)destroy_graph_locked(ctx, g);
  return status;
}

static int end_capture_locked(hc_ctx* ctx, hc_graph** out) {
  hc_graph* g = ctx->capturing;
  int emitted = HC_OK;
  if (ctx->lazy) {
    ctx->lazy = false;
    if (out) {
      // HCHIP_NO_FUSION=1 when the capture began: the launches are enqueued as they were issued
      if (ctx->rewrite) fuse_recording(ctx);
      if (ctx->sw.recording_log) log_launches_locked(ctx, "recording");
      emitted = emit_recording_locked(ctx, ctx->pending);
      if (ctx->sw.graph_as_launches)
        for (hc_pending& e : ctx->pending)
          if (!e.dropped && e.kind != hc_pending::FREE) g->launches.push_back(e);
    }
    ctx->pending.clear();
  }
  ctx->rewrite = false;
  ctx->capturing = nullptr;
  ctx->lazy = ctx->batch_limit > 0;   // batching goes on where the capture interrupted it
  ctx->batch_launches = 0;
  hipError_t e = hipStreamEndCapture(ctx->stream, &g->graph);
  if (emitted != HC_OK) {
    (void)hipGetLastError();
    if (g->graph) (void)hipGraphDestroy(g->graph);
    release_graph_blocks_locked(ctx, g);
    delete g;
    return emitted;
  }
  if (e == hipSuccess && out) e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
  if (e != hipSuccess || !out) {
    (void)hipGetLastError();
    if (g->graph) (void)hipGraphDestroy(g->graph);
    // the recorded kernels never ran and never will: its blocks are ordinary again
    release_graph_blocks_locked(ctx, g);
    delete g;
    if (e != hipSuccess) return hip_fail(e, "hipStreamEndCapture / hipGraphInstantiate");
    return HC_OK;
  }
  // Blocks that only held merged-away intermediates go back to the general pool now instead of
  // staying reserved until hc_graph_destroy.
  for (const auto& d : ctx->dead) {
    auto parked = g->parked.find(d.second);
    if (parked == g->parked.end()) continue;
    auto& v = parked->second;
    auto it = std::find(v.begin(), v.end(), d.first);
    if (it == v.end()) continue;
    v.erase(it);
    ctx->block_owner.erase(d.first);
    ctx->free_blocks[d.second].push_back(d.first);
    ctx->bytes_cached += d.second;
  }
  ctx->dead.clear();
  *out = g;
  return HC_OK;
}

extern "C" int hc_capture_end(hc_ctx* ctx, hc_graph** out) {
  REQUIRE(ctx && out, "hc_capture_end: null argument");
  *out = nullptr;
  return end_capture(ctx, out);
}

extern "C" int hc_capture_abort(hc_ctx* ctx) {
  REQUIRE(ctx, "hc_capture_abort: null context");
  return end_capture(ctx, nullptr);
}

extern "C" int hc_graph_launch(hc_ctx* ctx, hc_graph* graph) {
  REQUIRE(ctx && graph && graph->exec, "hc_graph_launch: null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  REQUIRE(!ctx->capturing, "hc_graph_launch: not allowed while capturing");
  HC_TRY(flush_batch_locked(ctx));
  if (!graph->launches.empty()) return emit_recording_locked(ctx, graph->launches);
  HIP_TRY(hipGraphLaunch(graph->exec, ctx->stream));
  return HC_OK;
}

extern "C" int hc_graph_node_count(hc_graph* graph, size_t* out) {
  REQUIRE(graph && graph->graph && out, "hc_graph_node_count: null argument");
  HIP_TRY(hipGraphGetNodes(graph->graph, nullptr, out));
  return HC_OK;
}

// Caller holds the lock; no capture in progress.
static int destroy_graph_locked(hc_ctx* ctx, hc_graph* graph) {
  // listed launches may use blocks that are parked with this graph, and replays already enqueued
  // still use them: enqueue the former, let all of it finish
  HC_TRY(flush_batch_locked(ctx));
  HIP_TRY(hipStreamSynchronize(ctx->stream));
  if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
  if (graph->graph) (void)hipGraphDestroy(graph->graph);
  release_graph_blocks_locked(ctx, graph);
  delete graph;
  return HC_OK;
}

extern "C" int hc_graph_destroy(hc_ctx* ctx, hc_graph* graph) {
  REQUIRE(ctx, "hc_graph_destroy: null context");
  if (!graph) return HC_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  REQUIRE(graph != ctx->capturing, "hc_graph_destroy: this recording is still in progress");
  if (ctx->capturing) {
    // (waiting for the stream would invalidate the capture in progress: an owner that lets go of an
    // older graph in the middle of a recording gets its destruction when the recording ends)
    ctx->doomed.push_back(graph);
    return HC_OK;
  }
  return destroy_graph_locked(ctx, graph);
}

// ------------------------------------------------------------------ rewriting a recording
#include "hchip_rewrite.inc"

// ------------------------------------------------------------------ raw module API

extern "C" int hc_module_load(hc_ctx* ctx, const void* image, size_t bytes, hc_module** out) {
  REQUIRE(ctx && image && out && bytes > 0, "hc_module_load: bad argument");
  hipModule_t mod;
  hipError_t e = hipModuleLoadData(&mod, image);
  if (e != hipSuccess) return fail(HC_ERR_LOAD, "hipModuleLoadData: %s", hipGetErrorString(e));
  *out = new hc_module{mod};
  return HC_OK;
}

extern "C" int hc_module_unload(hc_ctx* ctx, hc_module* mod) {
  REQUIRE(ctx && mod, "hc_module_unload: null argument");
  hipError_t e = hipModuleUnload(mod->mod);
  delete mod;
  if (e != hipSuccess) return hip_fail(e, "hipModuleUnload");
  return HC_OK;
}

extern "C" int hc_module_get_function(hc_module* mod, const char* name, hc_function** out) {
  REQUIRE(mod && name && out, "hc_module_get_function: null argument");
  hipFunction_t fn;
  hipError_t e = hipModuleGetFunction(&fn, mod->mod, name);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(HC_ERR_LOAD, "kernel '%s' not found: %s", name, hipGetErrorString(e));
  }
  *out = new hc_function{fn};  // lives as long as the module; a few bytes, never freed
  return HC_OK;
}

// Declared by an entry point for the duration of its launches: the caller-visible buffers the
// operation reads and writes (scratch memory the entry point takes from the pool is its own
// business). Nests: an entry point that calls another one is covered by the inner declaration
// while that one runs.
struct OpNote {
  std::vector<const void*> reads, writes;
  hc_pending::Tag tag = hc_pending::NONE;
  hc_pending meta;    // tag fields for the next launch only (consumed by it)
  OpNote* outer;
  static thread_local OpNote* current;
  OpNote(std::initializer_list<const void*> r, std::initializer_list<const void*> w) : reads(r), writes(w), outer(current) {
    current = this;
  }
  ~OpNote() { current = outer; }
  OpNote(const OpNote&) = delete;
  OpNote& operator=(const OpNote&) = delete;
};
thread_local OpNote* OpNote::current = nullptr;

// Batching: one more launch is listed; a full batch is enqueued. Caller holds the mutex.
static int batch_grew_locked(hc_ctx* ctx) {
  if (ctx->capturing || ctx->batch_limit == 0) return HC_OK;
  // A full list goes out at the next place where no chain that the rewrite could merge is open (the caller
  // holds at most one result of the listed launches: hc_free looks), or a quarter of the limit later at the
  // latest: cut in the middle of a layer, the launches around the cut stay unmerged.
  if (++ctx->batch_launches < ctx->batch_limit) return HC_OK;
  if (ctx->batch_born.size() <= 1 || ctx->batch_launches >= ctx->batch_limit + ctx->batch_limit / 4)
    return flush_batch_locked(ctx);
  return HC_OK;
}

// Adds a launch to the list in progress (caller holds the mutex).
static void record_launch_locked(hc_ctx* ctx, const std::string& name, hipFunction_t fn, uint32_t gx, uint32_t gy,
                                 const void* args, size_t bytes) {
  hc_pending e;
  e.kind = hc_pending::KERNEL;
  e.fn = fn;
  e.name = name;
  e.grid[0] = gx;
  e.grid[1] = gy;
  e.args.assign((const char*)args, (const char*)args + bytes);
  if (OpNote* n = OpNote::current) {
    e.known = true;
    e.reads = n->reads;
    e.writes = n->writes;
    if (n->tag != hc_pending::NONE) {   // the tag describes exactly one launch: the next one
      e.tag = n->tag;
      e.dtype = n->meta.dtype;
      e.src_dtype = n->meta.src_dtype;
      e.rows = n->meta.rows;
      e.cols = n->meta.cols;
      e.in0 = n->meta.in0;
      e.in1 = n->meta.in1;
      e.add_form = n->meta.add_form;
      e.pn = n->meta.pn;
      memcpy(e.pext, n->meta.pext, sizeof(e.pext));
      memcpy(e.pstr, n->meta.pstr, sizeof(e.pstr));
      e.in2 = n->meta.in2;
      e.sf = n->meta.sf;
      e.op = n->meta.op;
      e.lanes = n->meta.lanes;
      e.out = n->meta.out;
      n->tag = hc_pending::NONE;
    }
  }
  ctx->pending.push_back(std::move(e));
}

static int launch_fn(hc_ctx* ctx, hipFunction_t fn, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx,
                     uint32_t shared, const void* kernarg, size_t kernarg_bytes) {
  // every built-in kernel takes one struct by value: pass it as the single kernel parameter,
  // which the runtime copies at enqueue (and into a graph node while capturing)
  (void)kernarg_bytes;
  void* params[] = {const_cast<void*>(kernarg)};
  HIP_TRY(hipModuleLaunchKernel(fn, gx, gy, gz, bx, 1, 1, shared, ctx->stream, params, nullptr));
  return HC_OK;
}

extern "C" int hc_launch(hc_ctx* ctx, hc_function* fn, const uint32_t grid[3], const uint32_t block[3],
                         uint32_t shared_bytes, const void* kernarg, size_t kernarg_bytes) {
  REQUIRE(ctx && fn && grid && block, "hc_launch: null argument");
  void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(kernarg),
                    HIP_LAUNCH_PARAM_BUFFER_SIZE, &kernarg_bytes, HIP_LAUNCH_PARAM_END};
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (ctx->lazy) {   // a caller's own kernel: listed as it is, and nothing is moved across it
    hc_pending e;
    e.kind = hc_pending::RAW_KERNEL;
    e.fn = fn->fn;
    for (int i = 0; i < 3; i++) e.grid[i] = grid[i], e.block[i] = block[i];
    e.shared = shared_bytes;
    e.args.assign((const char*)kernarg, (const char*)kernarg + kernarg_bytes);
    ctx->pending.push_back(std::move(e));
    return batch_grew_locked(ctx);
  }
  HIP_TRY(hipModuleLaunchKernel(fn->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                shared_bytes, ctx->stream, nullptr, config));
  return HC_OK;
}

// Look a kernel up by name in the embedded code objects (cached) and launch it with a
// 256-lane block.
// A built-in kernel by name (caller holds the mutex).
static int find_kernel_locked(hc_ctx* ctx, const std::string& name, hipFunction_t* out) {
  auto it = ctx->functions.find(name);
  if (it != ctx->functions.end()) {
    *out = it->second;
    return HC_OK;
  }
  hipFunction_t fn = nullptr;
  // (a name that was looked for in vain is remembered too: the rewrite of a recording asks for variants of a
  // kernel that need not exist, once per launch it considers)
  if (!ctx->functions_missing.count(name)) {
    for (hipModule_t m : ctx->modules) {
      if (hipModuleGetFunction(&fn, m, name.c_str()) == hipSuccess) break;
      (void)hipGetLastError();
      fn = nullptr;
    }
    if (!fn) ctx->functions_missing.insert(name);
  }
  if (!fn) return fail(HC_ERR_LOAD, "kernel '%s' is not in the embedded code objects", name.c_str());
  ctx->functions[name] = fn;
  *out = fn;
  return HC_OK;
}

static int launch(hc_ctx* ctx, const std::string& name, uint64_t blocks_x, uint32_t blocks_y,
                  const void* args, size_t bytes) {
  if (blocks_x == 0 || blocks_y == 0) return HC_OK;
  if (blocks_x > 0x7fffffffull)
    return fail(HC_ERR_TOO_LARGE, "%s: grid of %llu blocks exceeds the launch limit", name.c_str(),
                (unsigned long long)blocks_x);
  std::lock_guard<std::mutex> lock(ctx->mu);
  hipFunction_t fn = nullptr;
  HC_TRY(find_kernel_locked(ctx, name, &fn));
  if (ctx->lazy) {
    record_launch_locked(ctx, name, fn, (uint32_t)blocks_x, blocks_y, args, bytes);
    return batch_grew_locked(ctx);
  }
  return launch_fn(ctx, fn, (uint32_t)blocks_x, blocks_y, 1, HCK_BLOCK, 0, args, bytes);
}

static inline uint64_t ceil_div(uint64_t a, uint64_t b) { return (a + b - 1) / b; }

// ------------------------------------------------------------------ descriptors

static const char* dtype_name(int dtype) {
  switch (dtype) {
    case HC_I64: return "i64";
    case HC_BOOL: return "b8";
    case HC_F16: return "f16";
    case HC_F32: return "f32";
    default: return nullptr;
  }
}

static size_t dtype_size(int dtype) {
  switch (dtype) {
    case HC_I64: return 8;
    case HC_BOOL: return 1;
    case HC_F16: return 2;
    default: return 4;
  }
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// Build the joint broadcast descriptor for `nops` operands over one virtual shape:
// drop size-1 axes, merge axes that are jointly mergeable (stride[d] == stride[d+1] *
// shape[d+1] for every operand, which also merges runs of broadcast axes), split the
// innermost axis off and pick the vector width. `vec_max` is the widest vector allowed
// (elements); `ptrs` are checked for 16-byte alignment. *total receives the element count.
static int make_bcast(int nops, const hc_strides* const* ops, const void* const* ptrs, const void* out,
                      int vec_max, hck_bcast* d, int* vec, uint64_t* total) {
  const hc_strides* s0 = ops[0];
  REQUIRE(s0->ndim <= HC_MAX_DIMS, "strides: ndim %u exceeds %d", s0->ndim, HC_MAX_DIMS);
  for (int o = 1; o < nops; o++) {
    REQUIRE(ops[o]->ndim == s0->ndim, "strides: operand ranks differ (%u vs %u)", ops[o]->ndim, s0->ndim);
    for (uint32_t k = 0; k < s0->ndim; k++)
      REQUIRE(ops[o]->shape[k] == s0->shape[k], "strides: operand shapes differ on axis %u", k);
  }
  int64_t shape[HC_MAX_DIMS];
  int64_t stride[3][HC_MAX_DIMS];
  int n = 0;
  uint64_t count = 1;
  for (uint32_t k = 0; k < s0->ndim; k++) {
    REQUIRE(s0->shape[k] >= 0, "strides: negative extent on axis %u", k);
    count *= (uint64_t)s0->shape[k];
  }
  *total = count;
  memset(d, 0, sizeof(*d));
  *vec = 1;
  if (count == 0) return HC_OK;
  if (count > 0xffffffffull)
    return fail(HC_ERR_TOO_LARGE, "broadcast op over %llu elements exceeds the 32-bit index range",
                (unsigned long long)count);
  for (uint32_t k = 0; k < s0->ndim; k++) {
    if (s0->shape[k] == 1) continue;
    shape[n] = s0->shape[k];
    for (int o = 0; o < nops; o++) {
      REQUIRE(ops[o]->strides[k] >= 0 && ops[o]->strides[k] <= 0xffffffffll,
              "strides: stride %lld on axis %u is out of range", (long long)ops[o]->strides[k], k);
      stride[o][n] = ops[o]->strides[k];
    }
    n++;
  }
  // merge from the inside out
  int m = 0;
  int64_t mshape[HC_MAX_DIMS];
  int64_t mstride[3][HC_MAX_DIMS];
  for (int k = n - 1; k >= 0; k--) {
    bool merge = m > 0;
    if (merge)
      for (int o = 0; o < nops; o++)
        if (stride[o][k] != mstride[o][m - 1] * mshape[m - 1]) merge = false;
    if (merge) {
      mshape[m - 1] *= shape[k];  // strides of the inner axis stay
    } else {
      mshape[m] = shape[k];
      for (int o = 0; o < nops; o++) mstride[o][m] = stride[o][k];
      m++;
    }
  }
  // mshape[0] is now the innermost axis; it must have stride 0 or 1 for every operand to
  // be the vector axis, otherwise a unit inner axis is prepended.
  bool inner_ok = m > 0;
  if (inner_ok)
    for (int o = 0; o < nops; o++)
      if (mstride[o][0] != 0 && mstride[o][0] != 1) inner_ok = false;
  int first_outer = 0;
  if (inner_ok) {
    d->inner = (uint32_t)mshape[0];
    for (int o = 0; o < nops; o++) d->inner_stride[o] = (uint32_t)mstride[o][0];
    first_outer = 1;
  } else {
    d->inner = 1;
    for (int o = 0; o < nops; o++) d->inner_stride[o] = 0;
  }
  d->n_outer = (uint32_t)(m - first_outer);
  if (d->n_outer > HCK_MAX_DIMS - 1)
    return fail(HC_ERR_UNSUPPORTED, "strides: %d non-mergeable axes with a strided innermost axis", m);
  // outer axes are stored outermost-first (the kernel peels them from the back)
  for (int k = first_outer; k < m; k++) {
    const int dst = m - 1 - k;
    d->outer_shape[dst] = (uint32_t)mshape[k];
    for (int o = 0; o < nops; o++) d->outer_stride[o][dst] = (uint32_t)mstride[o][k];
  }
  int v = vec_max;
  if (d->inner % (uint32_t)v != 0 || !aligned16(out)) v = 1;
  for (int o = 0; o < nops && v > 1; o++) {
    if (!aligned16(ptrs[o])) v = 1;
    if (d->inner_stride[o] == 1)
      for (uint32_t k = 0; k < d->n_outer; k++)
        if (d->outer_stride[o][k] % (uint32_t)v != 0) v = 1;
  }
  *vec = v;
  d->inner_vecs = d->inner / (uint32_t)v;
  d->total_vecs = (uint32_t)(count / (uint64_t)v);
  hck_fast_div_setup(d->inner_vecs, &d->inner_magic, &d->inner_sh);
  for (uint32_t k = 0; k < d->n_outer; k++) hck_fast_div_setup(d->outer_shape[k], &d->outer_magic[k], &d->outer_sh[k]);
  return HC_OK;
}

static int vec_for_size(size_t el) { return (int)(16 / el); }

// ------------------------------------------------------------------ element-wise ops

static const char* const kBinaryNames[] = {"add", "mul", "sub", "div", "mod"};
static const char* const kCompareNames[] = {"eq", "ne", "lt", "le", "gt", "ge"};

extern "C" int hc_broadcast(hc_ctx* ctx, int dtype, const void* a, const hc_strides* as, void* out) {
  OpNote note({a}, {out});
  REQUIRE(ctx && a && as && out, "hc_broadcast: null argument");
  REQUIRE(dtype_name(dtype), "hc_broadcast: bad dtype %d", dtype);
  const size_t el = dtype_size(dtype);
  hck_binary_args k;
  memset(&k, 0, sizeof(k));
  int vec;
  uint64_t total;
  const hc_strides* ops[] = {as};
  const void* ptrs[] = {a};
  HC_TRY(make_bcast(1, ops, ptrs, out, vec_for_size(el), &k.d, &vec, &total));
  if (total == 0) return HC_OK;
  k.a = a;
  k.out = out;
  char name[64];
  snprintf(name, sizeof(name), "hc_broadcast_b%zu_v%d", el, vec);
  return launch(ctx, name, ceil_div(k.d.total_vecs, HCK_BLOCK), 1, &k, sizeof(k));
}

extern "C" int hc_binary_op(hc_ctx* ctx, int op, int dtype, const void* a, const hc_strides* as,
                            const void* b, const hc_strides* bs, void* out) {
  REQUIRE(ctx && a && as && b && bs && out, "hc_binary_op: null argument");
  REQUIRE(op >= HC_ADD && op <= HC_MOD, "hc_binary_op: bad op %d", op);
  if (dtype != HC_F32 && dtype != HC_F16 && dtype != HC_I64)
    return fail(HC_ERR_UNSUPPORTED, "hc_binary_op: dtype %d is not numeric", dtype);
  hck_binary_args k;
  memset(&k, 0, sizeof(k));
  int vec;
  uint64_t total;
  const hc_strides* ops[] = {as, bs};
  const void* ptrs[] = {a, b};
  HC_TRY(make_bcast(2, ops, ptrs, out, vec_for_size(dtype_size(dtype)), &k.d, &vec, &total));
  if (total == 0) return HC_OK;
  k.a = a;
  k.b = b;
  k.out = out;
  OpNote note({a, b}, {out});
  if (op == HC_ADD && dtype != HC_I64) {
    // the two forms a recording can merge into the product that made one operand: dense + dense,
    // and a dense [rows, cols] operand plus a row of `cols` elements repeated over the rows
    const hck_bcast& d = k.d;
    int form = 0;
    if (d.n_outer == 0 && d.inner_stride[0] == 1 && d.inner_stride[1] == 1) form = 3;
    if (d.n_outer == 1 && d.inner_stride[0] == 1 && d.inner_stride[1] == 1) {
      if (d.outer_stride[0][0] == d.inner && d.outer_stride[1][0] == 0) form = 1;
      if (d.outer_stride[0][0] == 0 && d.outer_stride[1][0] == d.inner) form = 2;
    }
    if (form != 0) {
      note.tag = hc_pending::ADD;
      note.meta.dtype = dtype;
      note.meta.rows = form == 3 ? 1 : d.outer_shape[0];
      note.meta.cols = d.inner;
      note.meta.in0 = a;
      note.meta.in1 = b;
      note.meta.add_form = form;
      note.meta.out = out;
    }
  }
  char name[64];
  snprintf(name, sizeof(name), "hc_binary_%s_%s_v%d", kBinaryNames[op], dtype_name(dtype), vec);
  return launch(ctx, name, ceil_div(k.d.total_vecs, HCK_BLOCK), 1, &k, sizeof(k));
}

extern "C" int hc_bitwise_op(hc_ctx* ctx, int op, int dtype, const void* a, const hc_strides* as,
                             const void* b, const hc_strides* bs, void* out) {
  OpNote note({a, b}, {out});
  REQUIRE(ctx && a && as && b && bs && out, "hc_bitwise_op: null argument");
  REQUIRE(op >= HC_BIT_OR && op <= HC_BIT_XOR, "hc_bitwise_op: bad op %d", op);
  REQUIRE(dtype_name(dtype), "hc_bitwise_op: bad dtype %d", dtype);
  static const char* const names[] = {"or", "and", "xor"};
  const size_t el = dtype_size(dtype);
  hck_binary_args k;
  memset(&k, 0, sizeof(k));
  int vec;
  uint64_t total;
  const hc_strides* ops[] = {as, bs};
  const void* ptrs[] = {a, b};
  HC_TRY(make_bcast(2, ops, ptrs, out, vec_for_size(el), &k.d, &vec, &total));
  if (total == 0) return HC_OK;
  k.a = a;
  k.b = b;
  k.out = out;
  char name[64];
  snprintf(name, sizeof(name), "hc_bitwise_%s_b%zu_v%d", names[op], el, vec);
  return launch(ctx, name, ceil_div(k.d.total_vecs, HCK_BLOCK), 1, &k, sizeof(k));
}

extern "C" int hc_compare(hc_ctx* ctx, int op, int dtype, const void* a, const hc_strides* as,
                          const void* b, const hc_strides* bs, void* out) {
  OpNote note({a, b}, {out});
  REQUIRE(ctx && a && as && b && bs && out, "hc_compare: null argument");
  REQUIRE(op >= HC_EQ && op <= HC_GE, "hc_compare: bad op %d", op);
  REQUIRE(dtype_name(dtype), "hc_compare: bad dtype %d", dtype);
  hck_binary_args k;
  memset(&k, 0, sizeof(k));
  int vec;
  uint64_t total;
  const hc_strides* ops[] = {as, bs};
  const void* ptrs[] = {a, b};
  HC_TRY(make_bcast(2, ops, ptrs, out, vec_for_size(dtype_size(dtype)), &k.d, &vec, &total));
  if (total == 0) return HC_OK;
  k.a = a;
  k.b = b;
  k.out = out;
  char name[64];
  snprintf(name, sizeof(name), "hc_compare_%s_%s_v%d", kCompareNames[op], dtype_name(dtype), vec);
  return launch(ctx, name, ceil_div(k.d.total_vecs, HCK_BLOCK), 1, &k, sizeof(k));
}

static int fused3(hc_ctx* ctx, const char* kernel, int dtype, const void* x, const hc_strides* xs,
                  const void* y, const hc_strides* ys, const void* z, const hc_strides* zs, void* out,
                  size_t el, const char* tname) {
  hck_ternary_args k;
  memset(&k, 0, sizeof(k));
  int vec;
  uint64_t total;
  const hc_strides* ops[] = {xs, ys, zs};
  const void* ptrs[] = {x, y, z};
  (void)dtype;
  HC_TRY(make_bcast(3, ops, ptrs, out, vec_for_size(el), &k.d, &vec, &total));
  if (total == 0) return HC_OK;
  k.x = x;
  k.y = y;
  k.z = z;
  k.out = out;
  OpNote note({x, y, z}, {out});
  if (strcmp(kernel, "hc_mul_add") == 0 && dtype != HC_I64 && k.d.n_outer == 1 && k.d.inner_stride[0] == 1 &&
      k.d.inner_stride[1] == 1 && k.d.inner_stride[2] == 1 && k.d.outer_stride[0][0] == k.d.inner &&
      k.d.outer_stride[1][0] == 0 && k.d.outer_stride[2][0] == 0) {
    note.tag = hc_pending::MUL_ADD;
    note.meta.dtype = dtype;
    note.meta.rows = k.d.outer_shape[0];
    note.meta.cols = k.d.inner;
    note.meta.in0 = x;
    note.meta.in1 = y;
    note.meta.in2 = z;
    note.meta.out = out;
  }
  char name[64];
  snprintf(name, sizeof(name), "%s_%s_v%d", kernel, tname, vec);
  return launch(ctx, name, ceil_div(k.d.total_vecs, HCK_BLOCK), 1, &k, sizeof(k));
}

extern "C" int hc_mul_add(hc_ctx* ctx, int dtype, const void* input, const hc_strides* is,
                          const void* coeff, const hc_strides* cs, const void* bias,
                          const hc_strides* bs, void* out) {
  REQUIRE(ctx && input && is && coeff && cs && bias && bs && out, "hc_mul_add: null argument");
  if (dtype != HC_F32 && dtype != HC_F16 && dtype != HC_I64)
    return fail(HC_ERR_UNSUPPORTED, "hc_mul_add: dtype %d is not numeric", dtype);
  return fused3(ctx, "hc_mul_add", dtype, input, is, coeff, cs, bias, bs, out, dtype_size(dtype),
                dtype_name(dtype));
}

extern "C" int hc_add_mul(hc_ctx* ctx, int dtype, const void* input, const hc_strides* is,
                          const void* bias, const hc_strides* bs, const void* coeff,
                          const hc_strides* cs, void* out) {
  REQUIRE(ctx && input && is && coeff && cs && bias && bs && out, "hc_add_mul: null argument");
  if (dtype != HC_F32 && dtype != HC_F16 && dtype != HC_I64)
    return fail(HC_ERR_UNSUPPORTED, "hc_add_mul: dtype %d is not numeric", dtype);
  return fused3(ctx, "hc_add_mul", dtype, input, is, coeff, cs, bias, bs, out, dtype_size(dtype),
                dtype_name(dtype));
}

extern "C" int hc_when(hc_ctx* ctx, int dtype, const void* mask, const hc_strides* ms, const void* a,
                       const hc_strides* as, const void* b, const hc_strides* bs, void* out) {
  OpNote note({mask, a, b}, {out});
  REQUIRE(ctx && mask && ms && a && as && b && bs && out, "hc_when: null argument");
  REQUIRE(dtype_name(dtype), "hc_when: bad dtype %d", dtype);
  const size_t el = dtype_size(dtype);
  char tname[8];
  snprintf(tname, sizeof(tname), "b%zu", el);
  return fused3(ctx, "hc_when", dtype, mask, ms, a, as, b, bs, out, el, tname);
}

extern "C" int hc_clamp(hc_ctx* ctx, int dtype, const void* a, const hc_strides* as, const void* lo,
                        const hc_strides* ls, const void* hi, const hc_strides* hs, void* out) {
  OpNote note({a, lo, hi}, {out});
  REQUIRE(ctx && a && as && out, "hc_clamp: null argument");
  REQUIRE((lo && ls) || (hi && hs), "hc_clamp: cannot clamp without bounds");
  if (dtype != HC_F32 && dtype != HC_F16 && dtype != HC_I64)
    return fail(HC_ERR_UNSUPPORTED, "hc_clamp: dtype %d is not numeric", dtype);
  const char* kernel = lo && hi ? "hc_clamp_both" : lo ? "hc_clamp_min" : "hc_clamp_max";
  // an absent bound aliases the input (the kernel does not look at it)
  return fused3(ctx, kernel, dtype, a, as, lo ? lo : a, lo ? ls : as, hi ? hi : a, hi ? hs : as, out,
                dtype_size(dtype), dtype_name(dtype));
}

static int launch_contiguous(hc_ctx* ctx, const char* name, size_t count, int vec, const void* args,
                             size_t bytes) {
  if (count == 0) return HC_OK;
  // one vector per lane; the ragged tail (< vec elements) rides on block 0
  const uint64_t lanes = count / (uint64_t)vec ? count / (uint64_t)vec : 1;
  return launch(ctx, name, ceil_div(lanes, HCK_BLOCK), 1, args, bytes);
}

extern "C" int hc_binary_op_scalar(hc_ctx* ctx, int op, int dtype, const void* a, float sf,
                                   int64_t si, int scalar_first, void* out, size_t count) {
  REQUIRE(ctx, "hc_binary_op_scalar: null context");
  REQUIRE(op >= HC_ADD && op <= HC_MOD, "hc_binary_op_scalar: bad op %d", op);
  if (dtype != HC_F32 && dtype != HC_F16 && dtype != HC_I64)
    return fail(HC_ERR_UNSUPPORTED, "hc_binary_op_scalar: dtype %d is not numeric", dtype);
  if (count == 0) return HC_OK;
  REQUIRE(a && out, "hc_binary_op_scalar: null pointer");
  REQUIRE(aligned16(a) && aligned16(out), "hc_binary_op_scalar: buffers must be 16-byte aligned");
  hck_scalar_args k;
  memset(&k, 0, sizeof(k));
  k.in = a;
  k.out = out;
  k.count = count;
  k.sf = sf;
  k.si = si;
  const char* kop = kBinaryNames[op];
  if (dtype == HC_F32) {
    // The CPU's vDSP forms (BackendCPU.swift:325-342, 366-389).
    if (!scalar_first) {
      if (op == HC_DIV) {
        k.sf = 1.0f / sf;
        kop = "mul";
      } else if (op == HC_SUB) {
        k.sf = -sf;
        kop = "add";
      }
    } else {
      if (op == HC_DIV) kop = "rdiv";
      else if (op == HC_SUB) kop = "rsubf";
      else if (op == HC_MOD) kop = "rmod";
    }
  } else if (scalar_first) {
    if (op == HC_DIV) kop = "rdiv";
    else if (op == HC_SUB) kop = "rsub";
    else if (op == HC_MOD) kop = "rmod";
  }
  OpNote note({a}, {out});
  if (dtype != HC_I64 && (strcmp(kop, "add") == 0 || strcmp(kop, "mul") == 0)) {
    note.tag = hc_pending::SCALAR;
    note.meta.dtype = dtype;
    note.meta.op = kop[0] == 'a' ? HC_ADD : HC_MUL;
    note.meta.sf = k.sf;
    note.meta.rows = 1;
    note.meta.cols = count;
    note.meta.in0 = a;
    note.meta.out = out;
  }
  char name[64];
  snprintf(name, sizeof(name), "hc_scalar_%s_%s", kop, dtype_name(dtype));
  return launch_contiguous(ctx, name, count, vec_for_size(dtype_size(dtype)), &k, sizeof(k));
}

extern "C" int hc_compare_scalar(hc_ctx* ctx, int op, int dtype, const void* a, float sf, int64_t si,
                                 int scalar_first, void* out, size_t count) {
  OpNote note({a}, {out});
  REQUIRE(ctx, "hc_compare_scalar: null context");
  REQUIRE(op >= HC_EQ && op <= HC_GE, "hc_compare_scalar: bad op %d", op);
  REQUIRE(dtype_name(dtype), "hc_compare_scalar: bad dtype %d", dtype);
  if (count == 0) return HC_OK;
  REQUIRE(a && out, "hc_compare_scalar: null pointer");
  REQUIRE(aligned16(a) && aligned16(out), "hc_compare_scalar: buffers must be 16-byte aligned");
  hck_scalar_args k;
  memset(&k, 0, sizeof(k));
  k.in = a;
  k.out = out;
  k.count = count;
  k.sf = sf;
  k.si = si;
  char name[64];
  snprintf(name, sizeof(name), "hc_cmps_%s%s_%s", scalar_first ? "r" : "", kCompareNames[op],
           dtype_name(dtype));
  const int vec = vec_for_size(dtype_size(dtype));
  return launch_contiguous(ctx, name, count, vec > 16 ? 16 : vec, &k, sizeof(k));
}

extern "C" int hc_cast(hc_ctx* ctx, const void* in, int in_type, void* out, int out_type, size_t count) {
  REQUIRE(ctx, "hc_cast: null context");
  REQUIRE(dtype_name(in_type) && dtype_name(out_type), "hc_cast: bad dtype %d -> %d", in_type, out_type);
  if (count == 0) return HC_OK;
  REQUIRE(in && out, "hc_cast: null pointer");
  if (in_type == out_type) return hc_memcpy_d2d(ctx, out, in, count * dtype_size(in_type));
  REQUIRE(aligned16(in) && aligned16(out), "hc_cast: buffers must be 16-byte aligned");
  hck_map_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.out = out;
  k.count = count;
  OpNote note({in}, {out});
  note.tag = hc_pending::CAST;
  note.meta.dtype = out_type;
  note.meta.src_dtype = in_type;
  note.meta.rows = 1;
  note.meta.cols = count;
  note.meta.in0 = in;
  note.meta.out = out;
  char name[64];
  snprintf(name, sizeof(name), "hc_cast_%s_%s", dtype_name(in_type), dtype_name(out_type));
  const int vi = vec_for_size(dtype_size(in_type)), vo = vec_for_size(dtype_size(out_type));
  return launch_contiguous(ctx, name, count, vi < vo ? vi : vo, &k, sizeof(k));
}

extern "C" int hc_pow(hc_ctx* ctx, int dtype, const void* in, float bf, float scalef, int64_t bi,
                      int64_t scalei, const void* scales, void* out, size_t count) {
  OpNote note({in, scales}, {out});
  REQUIRE(ctx, "hc_pow: null context");
  if (dtype != HC_F32 && dtype != HC_F16 && dtype != HC_I64)
    return fail(HC_ERR_UNSUPPORTED, "hc_pow: dtype %d is not numeric", dtype);
  if (count == 0) return HC_OK;
  REQUIRE(in && out, "hc_pow: null pointer");
  REQUIRE(aligned16(in) && aligned16(out), "hc_pow: buffers must be 16-byte aligned");
  hck_map_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.scales = scales;
  k.out = out;
  k.count = count;
  k.p0 = bf;
  k.p1 = scalef;
  k.i0 = bi;
  k.i1 = scalei;
  const char* mode = "generic";
  if (dtype == HC_F32) {
    if (bf == 2.0f) mode = "square";
    else if (bf == -1.0f) mode = "recip";
    else if (bf == 1.0f) mode = "linear";
  }
  char name[64];
  snprintf(name, sizeof(name), "hc_pow_%s_%s", mode, dtype_name(dtype));
  return launch_contiguous(ctx, name, count, vec_for_size(dtype_size(dtype)), &k, sizeof(k));
}

static const char* const kElemwiseNames[HC_ELEMWISE_COUNT] = {
    "sin", "cos", "minus_sin", "tan", "tan_grad", "atan", "atan_grad", "acos", "acos_grad", "asin",
    "asin_grad", "exp", "log", "recip", "sigmoid", "sigmoid_grad", "relu", "relu_grad", "abs",
    "abs_grad", "gelu_approx", "gelu_approx_grad", "gelu_exact", "gelu_exact_grad", "erf", "erf_grad",
    "floor", "ceil", "round"};

extern "C" int hc_elemwise(hc_ctx* ctx, int op, int dtype, const void* in, const void* scales,
                           void* out, size_t count) {
  REQUIRE(ctx, "hc_elemwise: null context");
  REQUIRE(op >= 0 && op < HC_ELEMWISE_COUNT, "hc_elemwise: bad op %d", op);
  if (dtype != HC_F32 && dtype != HC_F16)
    return fail(HC_ERR_UNSUPPORTED, "hc_elemwise: dtype %d is not a float type", dtype);
  if (count == 0) return HC_OK;
  REQUIRE(in && out, "hc_elemwise: null pointer");
  REQUIRE(aligned16(in) && aligned16(out), "hc_elemwise: buffers must be 16-byte aligned");
  hck_map_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.scales = scales;
  k.out = out;
  k.count = count;
  OpNote note({in, scales}, {out});
  if (op == HC_EXP && !scales) {
    note.tag = hc_pending::EXP;
    note.meta.dtype = dtype;
    note.meta.rows = 1;
    note.meta.cols = count;
    note.meta.in0 = in;
    note.meta.out = out;
  }
  if (op == HC_GELU_APPROX && !scales) {
    note.tag = hc_pending::GELU;
    note.meta.dtype = dtype;
    note.meta.rows = 1;
    note.meta.cols = count;
    note.meta.in0 = in;
    note.meta.out = out;
  }
  char name[64];
  snprintf(name, sizeof(name), "hc_elemwise_%s_%s", kElemwiseNames[op], dtype_name(dtype));
  return launch_contiguous(ctx, name, count, vec_for_size(dtype_size(dtype)), &k, sizeof(k));
}

static uint16_t f32_to_f16_bits(float f) {
  // IEEE binary32 -> binary16, round-to-nearest-even, overflow to inf (host-side, for fill).
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u, absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) return (uint16_t)(sign | (absx > 0x7f800000u ? 0x7e00u : 0x7c00u));
  if (absx >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
  if (absx < 0x38800000u) {
    if (absx < 0x33000000u) return (uint16_t)sign;
    const int shift = 126 - (int)(absx >> 23);
    const uint32_t mant = (absx & 0x7fffffu) | 0x800000u;
    uint32_t res = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (res & 1u))) res++;
    return (uint16_t)(sign | res);
  }
  uint32_t res = (((absx >> 23) - 112u) << 10) | ((absx & 0x7fffffu) >> 13);
  const uint32_t rem = absx & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (res & 1u))) res++;
  return (uint16_t)(sign | res);
}

extern "C" int hc_fill(hc_ctx* ctx, int dtype, float vf, int64_t vi, void* out, size_t count) {
  OpNote note({}, {out});
  REQUIRE(ctx, "hc_fill: null context");
  REQUIRE(dtype_name(dtype), "hc_fill: bad dtype %d", dtype);
  if (count == 0) return HC_OK;
  REQUIRE(out, "hc_fill: null pointer");
  REQUIRE(aligned16(out), "hc_fill: buffer must be 16-byte aligned");
  hck_map_args k;
  memset(&k, 0, sizeof(k));
  k.out = out;
  k.count = count;
  switch (dtype) {
    case HC_I64: k.i0 = vi; break;
    case HC_BOOL: k.i0 = vf == 0 ? 0 : 1; break;
    case HC_F16: k.i0 = f32_to_f16_bits(vf); break;
    default: {
      uint32_t bits;
      memcpy(&bits, &vf, 4);
      k.i0 = bits;
    }
  }
  const size_t el = dtype_size(dtype);
  char name[64];
  snprintf(name, sizeof(name), "hc_fill_b%zu", el);
  return launch_contiguous(ctx, name, count, vec_for_size(el), &k, sizeof(k));
}

// Temporaries of one entry point. Normally blocks of the context's pool, freed (stream-ordered)
// when the entry point returns. With an arena (a caller-provided device range) the pieces are cut
// from that range instead, 256-byte aligned, and nothing is allocated or freed.
struct Scratch {
  hc_ctx* ctx;
  std::vector<void*> ptrs;
  char* arena = nullptr;
  size_t arena_bytes = 0, arena_used = 0;
  explicit Scratch(hc_ctx* c) : ctx(c) {}
  Scratch(hc_ctx* c, void* base, size_t bytes) : ctx(c), arena((char*)base), arena_bytes(bytes) {}
  ~Scratch() {
    for (void* p : ptrs) (void)hc_free(ctx, p);
  }
  bool fixed() const { return arena != nullptr; }
  int get(size_t bytes, void** out) {
    if (arena) {
      const size_t need = (bytes + 255) / 256 * 256;
      if (need > arena_bytes - arena_used)
        return fail(HC_ERR_TOO_LARGE,
                    "this call needs %zu bytes of scratch memory, the fixed scratch buffer holds %zu (%zu in use)",
                    bytes, arena_bytes, arena_used);
      *out = arena + arena_used;
      arena_used += need;
      return HC_OK;
    }
    int s = hc_malloc(ctx, bytes, out);
    if (s == HC_OK) ptrs.push_back(*out);
    return s;
  }
};

// ------------------------------------------------------------------ reductions

static const char* const kReduceNames[] = {"sum", "prod", "argmax", "argmin"};

static int check_dims(const char* who, int64_t outer, int64_t reduce, int64_t inner) {
  REQUIRE(outer >= 0 && reduce >= 0 && inner >= 0, "%s: negative dimension", who);
  if ((uint64_t)outer > 0xffffffffull || (uint64_t)reduce > 0xffffffffull || (uint64_t)inner > 0xffffffffull ||
      (double)outer * (double)reduce * (double)inner > 4294967295.0)
    return fail(HC_ERR_TOO_LARGE, "%s: [%lld, %lld, %lld] exceeds the 32-bit index range", who,
                (long long)outer, (long long)reduce, (long long)inner);
  return HC_OK;
}

// Column reduction ([outer, reduce, inner], inner > 1): lanes (x 16-byte vectors when rows keep
// the alignment) along inner, the reduce axis split over blocks until the device is full,
// partials combined by a second launch of the same kernel over the [outer, splits, inner]
// partials. `opname` also covers the internal float-result reductions (maxf, expsumf, sumf).
static int reduce_cols(hc_ctx* ctx, Scratch& scratch, const char* opname, int dtype, const void* in, const float* aux,
                       void* out, int64_t outer, int64_t reduce, int64_t inner, bool arg) {
  const size_t el = dtype_size(dtype);
  const uint32_t vec = (aligned16(in) && ((uint64_t)inner * el) % 16 == 0) ? (uint32_t)(16 / el) : 1;
  // lanes of a wave along inner: a power of two that covers it, at most 64
  auto lanes_for = [](uint64_t jvecs) {
    uint32_t jl = 1;
    while (jl < 64 && jl < jvecs) jl <<= 1;
    return jl;
  };
  const uint32_t jl = lanes_for(ceil_div((uint64_t)inner, vec)), jl_final = lanes_for((uint64_t)inner);
  const uint64_t jblocks = ceil_div(ceil_div((uint64_t)inner, vec), jl);
  const uint64_t base_blocks = jblocks * (uint64_t)outer;
  const uint64_t want = (uint64_t)ctx->props.multiProcessorCount * 8;
  uint64_t splits = base_blocks >= want ? 1 : ceil_div(want, base_blocks);
  const uint64_t max_splits = reduce / 64 ? (uint64_t)reduce / 64 : 1;  // at least 64 rows per range
  if (splits > max_splits) splits = max_splits;
  if (splits > 256) splits = 256;
  hck_reduce_cols_args c;
  memset(&c, 0, sizeof(c));
  c.in = in;
  c.out = out;
  c.aux = aux;
  c.outer = (uint32_t)outer;
  c.reduce = (uint32_t)reduce;
  c.inner = (uint32_t)inner;
  c.jl = jl;
  c.jl_final = jl_final;
  c.chunk = (uint32_t)(ceil_div(ceil_div((uint64_t)reduce, splits), 4) * 4);
  if (c.chunk == 0) c.chunk = 4;
  splits = reduce ? ceil_div((uint64_t)reduce, c.chunk) : 1;
  c.splits = (uint32_t)splits;
  if (splits > 1) {
    const size_t n = (size_t)outer * splits * (size_t)inner;
    HC_TRY(scratch.get(n * (dtype == HC_I64 ? 8 : 4), &c.pvals));
    if (arg) {
      void* idx = nullptr;
      HC_TRY(scratch.get(n * 4, &idx));
      c.pidx = (uint32_t*)idx;
    }
  }
  char name[64];
  snprintf(name, sizeof(name), "hc_reduce_cols_%s_%s_%s", opname, dtype_name(dtype), vec > 1 ? "vN" : "v1");
  HC_TRY(launch(ctx, name, base_blocks * splits, 1, &c, sizeof(c)));
  if (splits > 1) {
    snprintf(name, sizeof(name), "hc_reduce_cols_final_%s_%s", opname, dtype_name(dtype));
    HC_TRY(launch(ctx, name, ceil_div((uint64_t)inner, jl_final) * (uint64_t)outer, 1, &c, sizeof(c)));
  }
  return HC_OK;
}

// logSoftmax / logSoftmaxGrad over a non-last axis: per-column maximum, exp-sum (and gradient
// sum) as float column reductions, then one element-wise pass.
static int softmax_cols(hc_ctx* ctx, int dtype, const void* in, const void* grad, void* out, int64_t outer,
                        int64_t reduce, int64_t inner) {
  Scratch scratch(ctx);
  const size_t cols = (size_t)outer * (size_t)inner;
  void *m = nullptr, *s = nullptr, *gs = nullptr;
  HC_TRY(scratch.get(cols * 4, &m));
  HC_TRY(scratch.get(cols * 4, &s));
  HC_TRY(reduce_cols(ctx, scratch, "maxf", dtype, in, nullptr, m, outer, reduce, inner, false));
  HC_TRY(reduce_cols(ctx, scratch, "expsumf", dtype, in, (const float*)m, s, outer, reduce, inner, false));
  if (grad) {
    HC_TRY(scratch.get(cols * 4, &gs));
    HC_TRY(reduce_cols(ctx, scratch, "sumf", dtype, grad, nullptr, gs, outer, reduce, inner, false));
  }
  hck_softmax_cols_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.grad = grad;
  k.out = out;
  k.col_max = (const float*)m;
  k.col_expsum = (const float*)s;
  k.col_gradsum = (const float*)gs;
  k.outer = (uint32_t)outer;
  k.reduce = (uint32_t)reduce;
  k.inner = (uint32_t)inner;
  HC_TRY(launch(ctx, "hc_log_softmax_cols_logsum", ceil_div((uint64_t)cols, HCK_BLOCK), 1, &k, sizeof(k)));
  const size_t el = dtype_size(dtype);
  const uint32_t vec = ((uint64_t)inner * el) % 16 == 0 ? (uint32_t)(16 / el) : 1;
  char name[64];
  snprintf(name, sizeof(name), "hc_log_softmax%s_cols_apply_%s_%s", grad ? "_grad" : "", dtype_name(dtype),
           vec > 1 ? "vN" : "v1");
  const uint64_t lanes = (uint64_t)outer * (uint64_t)reduce * ceil_div((uint64_t)inner, vec);
  return launch(ctx, name, ceil_div(lanes, HCK_BLOCK), 1, &k, sizeof(k));
}

// hc_reduce proper; `scratch` says where partial results live (the pool, or a fixed range).
static int reduce_impl(hc_ctx* ctx, Scratch& scratch, int op, int dtype, const void* in, void* out, int64_t outer,
                       int64_t reduce, int64_t inner, OpNote* note) {
  REQUIRE(ctx, "hc_reduce: null context");
  REQUIRE(op >= HC_SUM && op <= HC_ARGMIN, "hc_reduce: bad op %d", op);
  if (dtype != HC_F32 && dtype != HC_F16 && dtype != HC_I64 && dtype != HC_BOOL)
    return fail(HC_ERR_UNSUPPORTED, "hc_reduce: bad dtype %d", dtype);
  HC_TRY(check_dims("hc_reduce", outer, reduce, inner));
  if (outer * inner == 0) return HC_OK;
  REQUIRE(out, "hc_reduce: null output");
  REQUIRE(reduce > 0 || op == HC_SUM || op == HC_PROD, "hc_reduce: arg-reduction over an empty axis");
  REQUIRE(in || reduce == 0, "hc_reduce: null input");
  hck_reduce_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.out = out;
  k.outer = (uint32_t)outer;
  k.reduce = (uint32_t)reduce;
  k.inner = (uint32_t)inner;
  char name[64];
  if (inner == 1) {
    const bool vec_ok = aligned16(in);
    REQUIRE(vec_ok, "hc_reduce: input must be 16-byte aligned");
    auto tag_arg = [&](int lanes) {   // an arg-reduction in one launch: a gather of its indices can join it
      if (!note || (op != HC_ARGMAX && op != HC_ARGMIN)) return;
      note->tag = hc_pending::ARG_REDUCE;
      note->meta.dtype = dtype;
      note->meta.op = op;
      note->meta.rows = (uint64_t)outer;
      note->meta.cols = (uint64_t)reduce;
      note->meta.lanes = lanes;
      note->meta.in0 = in;
      note->meta.out = out;
    };
    // a team of 1, 8, 64 or 256 lanes per row, by row length
    if (reduce <= 1024) {
      const uint32_t lanes = reduce <= 8 ? 1 : reduce <= 128 ? 8 : 64;
      tag_arg((int)lanes);
      snprintf(name, sizeof(name), "hc_reduce_rows%u_%s_%s", lanes, kReduceNames[op], dtype_name(dtype));
      return launch(ctx, name, ceil_div((uint64_t)outer, HCK_BLOCK / lanes), 1, &k, sizeof(k));
    }
    // Few long rows (a sum or maximum over a whole tensor): a block per row would leave most of
    // the device idle, so the rows are cut into segments that leave partials, combined by the
    // final pass of the column reduction (partials laid out as [outer, segs, 1]).
    const uint64_t cus = (uint64_t)ctx->props.multiProcessorCount;
    if ((uint64_t)outer < 2 * cus && reduce >= 32768) {
      uint64_t segs = std::min<uint64_t>(ceil_div(4 * cus, (uint64_t)outer), (uint64_t)reduce / 8192);
      const uint64_t seg_len = ceil_div(ceil_div((uint64_t)reduce, segs), 8192) * 8192;
      segs = ceil_div((uint64_t)reduce, seg_len);
      if (segs > 1) {
        const bool arg = op == HC_ARGMAX || op == HC_ARGMIN;
        const size_t n = (size_t)outer * segs;
        HC_TRY(scratch.get(n * 8, &k.pvals));
        if (arg) {
          void* idx = nullptr;
          HC_TRY(scratch.get(n * 4, &idx));
          k.pidx = (uint32_t*)idx;
        }
        k.segs = (uint32_t)segs;
        k.seg_len = (uint32_t)seg_len;
        snprintf(name, sizeof(name), "hc_reduce_rowsplit_%s_%s", kReduceNames[op], dtype_name(dtype));
        HC_TRY(launch(ctx, name, n, 1, &k, sizeof(k)));
        hck_reduce_cols_args c;
        memset(&c, 0, sizeof(c));
        c.out = out;
        c.pvals = k.pvals;
        c.pidx = k.pidx;
        c.outer = (uint32_t)outer;
        c.reduce = (uint32_t)reduce;
        c.inner = 1;
        c.splits = (uint32_t)segs;
        c.chunk = (uint32_t)seg_len;
        c.jl_final = 1;  // one column: all 64 lanes of a wave along the partials
        snprintf(name, sizeof(name), "hc_reduce_cols_final_%s_%s", kReduceNames[op], dtype_name(dtype));
        return launch(ctx, name, (uint64_t)outer, 1, &c, sizeof(c));
      }
    }
    tag_arg(256);
    snprintf(name, sizeof(name), "hc_reduce_rows256_%s_%s", kReduceNames[op], dtype_name(dtype));
    return launch(ctx, name, (uint64_t)outer, 1, &k, sizeof(k));
  }
  return reduce_cols(ctx, scratch, kReduceNames[op], dtype, in, nullptr, out, outer, reduce, inner,
                     op == HC_ARGMAX || op == HC_ARGMIN);
}

extern "C" int hc_reduce(hc_ctx* ctx, int op, int dtype, const void* in, void* out, int64_t outer,
                         int64_t reduce, int64_t inner) {
  OpNote note({in}, {out});
  REQUIRE(ctx, "hc_reduce: null context");
  Scratch scratch(ctx);
  return reduce_impl(ctx, scratch, op, dtype, in, out, outer, reduce, inner, &note);
}

// hc_reduce with its partial results in the caller's device range [scratch, scratch + scratch_bytes)
// instead of pool blocks: the body of hc_reduce_noalloc (noalloc.hip), which owns that range.
__attribute__((visibility("hidden"))) int hc_reduce_in_scratch(hc_ctx* ctx, int op, int dtype, const void* in,
                                                               void* out, int64_t outer, int64_t reduce,
                                                               int64_t inner, void* scratch_base,
                                                               size_t scratch_bytes) {
  REQUIRE(ctx, "hc_reduce_noalloc: null context");
  REQUIRE(scratch_base, "hc_reduce_noalloc: the scratch buffer of device %d was not set up", ctx->device);
  OpNote note({in}, {out});   // (in a recording: the launches stay where they are, nothing is merged into them)
  Scratch scratch(ctx, scratch_base, scratch_bytes);
  return reduce_impl(ctx, scratch, op, dtype, in, out, outer, reduce, inner, nullptr);
}

__attribute__((visibility("hidden"))) int hc_ctx_device(const hc_ctx* ctx) { return ctx ? ctx->device : -1; }

__attribute__((visibility("hidden"))) int hc_set_error(int code, const char* message) {
  return fail(code, "%s", message);
}

extern "C" int hc_cumulative(hc_ctx* ctx, int op, int dtype, const void* in, void* out, int64_t outer,
                             int64_t reduce, int64_t inner, int exclusive, int reverse) {
  OpNote note({in}, {out});
  REQUIRE(ctx, "hc_cumulative: null context");
  REQUIRE(op == 0 || op == 1, "hc_cumulative: bad op %d", op);
  if (dtype != HC_F32 && dtype != HC_F16 && dtype != HC_I64)
    return fail(HC_ERR_UNSUPPORTED, "hc_cumulative: dtype %d is not numeric", dtype);
  HC_TRY(check_dims("hc_cumulative", outer, reduce, inner));
  if (outer * reduce * inner == 0) return HC_OK;
  REQUIRE(in && out, "hc_cumulative: null pointer");
  hck_scan_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.out = out;
  k.outer = (uint32_t)outer;
  k.reduce = (uint32_t)reduce;
  k.inner = (uint32_t)inner;
  k.exclusive = exclusive != 0;
  k.reverse = reverse != 0;
  const char* opn = op == 0 ? "sum" : "prod";
  // columns: a lane takes 16 bytes of adjacent columns when the layout allows and enough lanes remain
  const uint64_t vec = 16 / dtype_size(dtype);
  const bool colsv = inner > 1 && (uint64_t)inner % vec == 0 && aligned16(in) && aligned16(out) &&
                     (uint64_t)outer * (uint64_t)inner / vec >= 64;
  // (rows of a few elements: the column form with inner = 1 is a lane per row, adjacent lanes on
  // adjacent rows, instead of a wave per row)
  const bool lane_rows = inner == 1 && reduce <= 16;
  const char* form = lane_rows ? "cols" : inner == 1 ? "rows" : colsv ? "colsv" : "cols";
  const char* tn = dtype_name(dtype);
  // Few, long lines: cut the axis so that about eight waves per compute unit have work.
  const uint64_t cus = (uint64_t)ctx->props.multiProcessorCount;
  uint64_t segs = 1, seg_len = (uint64_t)reduce;
  if (lane_rows) {
    // one pass, no segments
  } else if (inner == 1) {
    const uint64_t want = cus * 8;  // waves
    if ((uint64_t)outer < want && reduce >= 4096) {
      segs = std::min<uint64_t>(ceil_div(want, (uint64_t)outer), (uint64_t)reduce / 1024);
      seg_len = ceil_div(ceil_div((uint64_t)reduce, segs), 256) * 256;  // whole 64 x 4 tiles
      segs = ceil_div((uint64_t)reduce, seg_len);
    }
  } else {
    const uint64_t want = cus * 8 * 64, lanes = (uint64_t)outer * (uint64_t)inner / (colsv ? vec : 1);
    if (lanes < want && reduce >= 128) {
      segs = std::min<uint64_t>(ceil_div(want, lanes), (uint64_t)reduce / 32);
      seg_len = ceil_div((uint64_t)reduce, segs);
      segs = ceil_div((uint64_t)reduce, seg_len);
    }
  }
  char name[64];
  const uint64_t units = (uint64_t)outer * segs * (uint64_t)inner;  // waves (rows) or columns (cols)
  const uint64_t blocks = inner == 1 && !lane_rows ? ceil_div(units, HCK_BLOCK / 64) : ceil_div(units / (colsv ? vec : 1), HCK_BLOCK);
  Scratch scratch(ctx);
  if (segs > 1) {
    k.segs = (uint32_t)segs;
    k.seg_len = (uint32_t)seg_len;
    HC_TRY(scratch.get(units * 8, &k.carry));
    snprintf(name, sizeof(name), "hc_cumulative_%s_%s_totals_%s", opn, form, tn);
    HC_TRY(launch(ctx, name, blocks, 1, &k, sizeof(k)));
    snprintf(name, sizeof(name), "hc_cumulative_%s_carry_%s", opn, dtype == HC_I64 ? "i64" : "f32");
    HC_TRY(launch(ctx, name, ceil_div((uint64_t)outer * (uint64_t)inner, HCK_BLOCK / 64), 1, &k, sizeof(k)));  // a wave per line
  }
  snprintf(name, sizeof(name), "hc_cumulative_%s_%s_%s", opn, form, tn);
  return launch(ctx, name, blocks, 1, &k, sizeof(k));
}

extern "C" int hc_argsort(hc_ctx* ctx, int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
                          int64_t inner, int descending) {
  OpNote note({in}, {out});
  REQUIRE(ctx, "hc_argsort: null context");
  if (dtype != HC_F32 && dtype != HC_F16 && dtype != HC_I64)
    return fail(HC_ERR_UNSUPPORTED, "hc_argsort: dtype %d is not numeric", dtype);
  HC_TRY(check_dims("hc_argsort", outer, reduce, inner));
  if (outer * reduce * inner == 0) return HC_OK;
  REQUIRE(in && out, "hc_argsort: null pointer");
  if (reduce > 4096) {
    // runs of 4096 sorted in LDS, then merged pairwise; two sets of (key, index) arrays alternate
    const uint64_t lines = (uint64_t)outer * (uint64_t)inner, total = lines * (uint64_t)reduce;
    Scratch scratch(ctx);
    void *keys[2], *idx[2];
    for (int b = 0; b < 2; b++) {
      HC_TRY(scratch.get(total * sizeof(uint64_t), &keys[b]));
      HC_TRY(scratch.get(total * sizeof(uint32_t), &idx[b]));
    }
    hck_sort_args s;
    memset(&s, 0, sizeof(s));
    s.in = in;
    s.out = out;
    s.outer = (uint32_t)outer;
    s.reduce = (uint32_t)reduce;
    s.inner = (uint32_t)inner;
    s.descending = descending != 0;
    s.keys_out = (uint64_t*)keys[0];
    s.idx_out = (uint32_t*)idx[0];
    char name[64];
    snprintf(name, sizeof(name), "hc_argsort_chunks_%s", dtype_name(dtype));
    HC_TRY(launch(ctx, name, lines * ceil_div((uint64_t)reduce, 4096), 1, &s, sizeof(s)));
    int cur = 0;
    for (uint64_t run = 4096; run < (uint64_t)reduce; run *= 2, cur ^= 1) {
      s.run = (uint32_t)run;
      s.keys_in = (const uint64_t*)keys[cur];
      s.idx_in = (const uint32_t*)idx[cur];
      s.keys_out = (uint64_t*)keys[cur ^ 1];
      s.idx_out = (uint32_t*)idx[cur ^ 1];
      HC_TRY(launch(ctx, "hc_argsort_merge", lines * ceil_div((uint64_t)reduce, 8 * HCK_BLOCK), 1, &s, sizeof(s)));
    }
    s.idx_in = (const uint32_t*)idx[cur];
    return launch(ctx, "hc_argsort_emit", ceil_div(total, HCK_BLOCK), 1, &s, sizeof(s));
  }
  hck_scan_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.out = out;
  k.outer = (uint32_t)outer;
  k.reduce = (uint32_t)reduce;
  k.inner = (uint32_t)inner;
  k.reverse = descending != 0;
  char name[64];
  snprintf(name, sizeof(name), "hc_argsort_%s", dtype_name(dtype));
  return launch(ctx, name, (uint64_t)outer * (uint64_t)inner, 1, &k, sizeof(k));
}

extern "C" int hc_log_softmax(hc_ctx* ctx, int dtype, const void* in, void* out, int64_t outer,
                              int64_t reduce, int64_t inner) {
  REQUIRE(ctx, "hc_log_softmax: null context");
  if (dtype != HC_F32 && dtype != HC_F16)
    return fail(HC_ERR_UNSUPPORTED, "hc_log_softmax: dtype %d is not a float type", dtype);
  HC_TRY(check_dims("hc_log_softmax", outer, reduce, inner));
  if (outer * reduce * inner == 0) return HC_OK;
  REQUIRE(in && out, "hc_log_softmax: null pointer");
  REQUIRE(aligned16(in) && aligned16(out), "hc_log_softmax: buffers must be 16-byte aligned");
  const size_t el_size = dtype_size(dtype);
  hck_reduce_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.out = out;
  k.outer = (uint32_t)outer;
  k.reduce = (uint32_t)reduce;
  k.inner = (uint32_t)inner;
  char name[64];
  // (few long rows: a block per row would leave most of the device idle; the column path cuts the
  // axis over many blocks)
  const bool few_long_rows = inner == 1 && (uint64_t)outer < 2 * (uint64_t)ctx->props.multiProcessorCount && reduce >= 32768;
  OpNote note({in}, {out});
  auto tag_rows = [&](int lanes) {   // rows held in the registers of a team of `lanes` lanes
    if (reduce % (int64_t)(16 / el_size) != 0) return;
    note.tag = hc_pending::LOG_SOFTMAX;
    note.meta.dtype = dtype;
    note.meta.rows = (uint64_t)outer;
    note.meta.cols = (uint64_t)reduce;
    note.meta.lanes = lanes;
    note.meta.in0 = in;
    note.meta.out = out;
  };
  if (inner == 1 && !few_long_rows) {
    // a lane or 8 lanes per row for short rows, a wave per row while the row fits its registers
    // (4 x 16 bytes per lane), else a block
    if ((uint64_t)reduce * el_size <= 512) {  // (8 lanes x 4 x 16 bytes: the row still fits the team's registers)
      const uint32_t lanes = reduce <= 8 ? 1 : 8;
      if (lanes == 8) tag_rows(8);
      snprintf(name, sizeof(name), "hc_log_softmax_rows%u_%s", lanes, dtype_name(dtype));
      return launch(ctx, name, ceil_div((uint64_t)outer, HCK_BLOCK / lanes), 1, &k, sizeof(k));
    }
    if ((uint64_t)reduce * el_size <= 64 * 16 * 4) {
      tag_rows(64);
      snprintf(name, sizeof(name), "hc_log_softmax_rows_%s", dtype_name(dtype));
      return launch(ctx, name, ceil_div((uint64_t)outer, HCK_BLOCK / 64), 1, &k, sizeof(k));
    }
    snprintf(name, sizeof(name), "hc_log_softmax_rows256_%s", dtype_name(dtype));
    return launch(ctx, name, (uint64_t)outer, 1, &k, sizeof(k));
  }
  return softmax_cols(ctx, dtype, in, nullptr, out, outer, reduce, inner);
}

extern "C" int hc_log_softmax_grad(hc_ctx* ctx, int dtype, const void* in, const void* out_grad, void* out,
                                   int64_t outer, int64_t reduce, int64_t inner) {
  OpNote note({in, out_grad}, {out});
  REQUIRE(ctx, "hc_log_softmax_grad: null context");
  if (dtype != HC_F32 && dtype != HC_F16)
    return fail(HC_ERR_UNSUPPORTED, "hc_log_softmax_grad: dtype %d is not a float type", dtype);
  HC_TRY(check_dims("hc_log_softmax_grad", outer, reduce, inner));
  if (outer * reduce * inner == 0) return HC_OK;
  REQUIRE(in && out_grad && out, "hc_log_softmax_grad: null pointer");
  REQUIRE(aligned16(in) && aligned16(out_grad) && aligned16(out), "hc_log_softmax_grad: buffers must be 16-byte aligned");
  const size_t el_size = dtype_size(dtype);
  hck_reduce_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.in2 = out_grad;
  k.out = out;
  k.outer = (uint32_t)outer;
  k.reduce = (uint32_t)reduce;
  k.inner = (uint32_t)inner;
  char name[64];
  // (few long rows: a block per row would leave most of the device idle; the column path cuts the
  // axis over many blocks)
  const bool few_long_rows = inner == 1 && (uint64_t)outer < 2 * (uint64_t)ctx->props.multiProcessorCount && reduce >= 32768;
  if (inner == 1 && !few_long_rows) {
    // a lane or 8 lanes per row for short rows, a wave per row while the row fits its registers
    // (4 x 16 bytes per lane), else a block
    if ((uint64_t)reduce * el_size <= 512) {  // (8 lanes x 4 x 16 bytes: the row still fits the team's registers)
      const uint32_t lanes = reduce <= 8 ? 1 : 8;
      snprintf(name, sizeof(name), "hc_log_softmax_grad_rows%u_%s", lanes, dtype_name(dtype));
      return launch(ctx, name, ceil_div((uint64_t)outer, HCK_BLOCK / lanes), 1, &k, sizeof(k));
    }
    if ((uint64_t)reduce * el_size <= 64 * 16 * 4) {
      snprintf(name, sizeof(name), "hc_log_softmax_grad_rows_%s", dtype_name(dtype));
      return launch(ctx, name, ceil_div((uint64_t)outer, HCK_BLOCK / 64), 1, &k, sizeof(k));
    }
    snprintf(name, sizeof(name), "hc_log_softmax_grad_rows256_%s", dtype_name(dtype));
    return launch(ctx, name, (uint64_t)outer, 1, &k, sizeof(k));
  }
  return softmax_cols(ctx, dtype, in, out_grad, out, outer, reduce, inner);
}


extern "C" int hc_normalize(hc_ctx* ctx, int dtype, const void* in, void* out, int64_t outer,
                            int64_t reduce, int64_t inner, float eps) {
  REQUIRE(ctx, "hc_normalize: null context");
  if (dtype != HC_F32 && dtype != HC_F16)
    return fail(HC_ERR_UNSUPPORTED, "hc_normalize: dtype %d is not a float type", dtype);
  HC_TRY(check_dims("hc_normalize", outer, reduce, inner));
  if (outer * reduce * inner == 0) return HC_OK;
  REQUIRE(in && out, "hc_normalize: null pointer");
  REQUIRE(aligned16(in) && aligned16(out), "hc_normalize: buffers must be 16-byte aligned");
  const size_t el_size = dtype_size(dtype);
  // (few long rows: a block per row would leave most of the device idle; the op-by-op composition
  // below runs every step over the whole device, at the price of nine launches)
  const bool few_long_rows = inner == 1 && (uint64_t)outer * 8 < (uint64_t)ctx->props.multiProcessorCount && reduce >= 32768;
  OpNote note({in}, {out});
  if (inner == 1 && !few_long_rows) {
    hck_reduce_args k;
    memset(&k, 0, sizeof(k));
    k.in = in;
    k.out = out;
    k.outer = (uint32_t)outer;
    k.reduce = (uint32_t)reduce;
    k.inner = 1;
    k.eps = eps;
    char name[64];
    // a lane or 8 lanes per row for short rows, a wave per row while the row fits its registers
    // (4 x 16 bytes per lane), else a block
    if ((uint64_t)reduce * el_size <= 512) {  // (8 lanes x 4 x 16 bytes: the row still fits the team's registers)
      const uint32_t lanes = reduce <= 8 ? 1 : 8;
      snprintf(name, sizeof(name), "hc_normalize_rows%u_%s", lanes, dtype_name(dtype));
      return launch(ctx, name, ceil_div((uint64_t)outer, HCK_BLOCK / lanes), 1, &k, sizeof(k));
    }
    if ((uint64_t)reduce * el_size <= 64 * 16 * 4) {
      if (dtype == HC_F32 && reduce % 4 == 0) {   // the form a recording can merge a LayerNorm's other steps into
        note.tag = hc_pending::NORMALIZE;
        note.meta.dtype = dtype;
        note.meta.rows = (uint64_t)outer;
        note.meta.cols = (uint64_t)reduce;
        note.meta.sf = eps;
        note.meta.in0 = in;
        note.meta.out = out;
      }
      snprintf(name, sizeof(name), "hc_normalize_rows_%s", dtype_name(dtype));
      return launch(ctx, name, ceil_div((uint64_t)outer, HCK_BLOCK / 64), 1, &k, sizeof(k));
    }
    snprintf(name, sizeof(name), "hc_normalize_rows256_%s", dtype_name(dtype));
    return launch(ctx, name, (uint64_t)outer, 1, &k, sizeof(k));
  }
  // inner > 1: the same composition the base class runs (Backend.swift:265-327), on device.
  const size_t el = dtype_size(dtype);
  const size_t full = (size_t)(outer * reduce * inner), red = (size_t)(outer * inner);
  hc_strides fs = {3, 0, {outer, reduce, inner}, {reduce * inner, inner, 1}};
  hc_strides rs = {3, 0, {outer, reduce, inner}, {inner, 0, 1}};
  Scratch scratch(ctx);
  void *t_red, *mean, *centered, *sq, *var, *norm;
  HC_TRY(scratch.get(red * el, &t_red));
  HC_TRY(scratch.get(red * el, &mean));
  HC_TRY(scratch.get(full * el, &centered));
  HC_TRY(scratch.get(full * el, &sq));
  HC_TRY(scratch.get(red * el, &var));
  HC_TRY(scratch.get(red * el, &norm));
  const float inv_n = 1.0f / (float)reduce;
  HC_TRY(hc_reduce(ctx, HC_SUM, dtype, in, t_red, outer, reduce, inner));
  HC_TRY(hc_binary_op_scalar(ctx, HC_MUL, dtype, t_red, inv_n, 0, 0, mean, red));
  HC_TRY(hc_binary_op(ctx, HC_SUB, dtype, in, &fs, mean, &rs, centered));
  HC_TRY(hc_pow(ctx, dtype, centered, 2.0f, 1.0f, 2, 1, nullptr, sq, full));
  HC_TRY(hc_reduce(ctx, HC_SUM, dtype, sq, t_red, outer, reduce, inner));
  HC_TRY(hc_binary_op_scalar(ctx, HC_MUL, dtype, t_red, inv_n, 0, 0, var, red));
  HC_TRY(hc_binary_op_scalar(ctx, HC_ADD, dtype, var, eps, 0, 0, t_red, red));
  HC_TRY(hc_pow(ctx, dtype, t_red, -0.5f, 1.0f, 0, 1, nullptr, norm, red));
  HC_TRY(hc_binary_op(ctx, HC_MUL, dtype, centered, &fs, norm, &rs, out));
  return HC_OK;
}

// ------------------------------------------------------------------ gather & friends

extern "C" int hc_gather(hc_ctx* ctx, int dtype, const void* in, const void* indices,
                         const hc_strides* idx_strides, void* out, int64_t outer, int64_t middle,
                         int64_t out_count, int64_t inner) {
  OpNote note({in, indices}, {out});
  REQUIRE(ctx && idx_strides, "hc_gather: null argument");
  REQUIRE(dtype_name(dtype), "hc_gather: bad dtype %d", dtype);
  REQUIRE(outer >= 0 && middle >= 0 && out_count >= 0 && inner >= 0, "hc_gather: negative dimension");
  const double out_total = (double)outer * (double)out_count * (double)inner;
  const double in_total = (double)outer * (double)middle * (double)inner;
  if (out_total == 0) return HC_OK;
  if (out_total > 4294967295.0 || in_total > 4294967295.0)
    return fail(HC_ERR_TOO_LARGE, "hc_gather: more than 2^32-1 elements");
  REQUIRE(in && indices && out, "hc_gather: null pointer");
  const uint64_t total = (uint64_t)outer * (uint64_t)out_count * (uint64_t)inner;
  {
    uint64_t n = 1;
    REQUIRE(idx_strides->ndim <= HC_MAX_DIMS, "hc_gather: ndim %u exceeds %d", idx_strides->ndim, HC_MAX_DIMS);
    for (uint32_t k = 0; k < idx_strides->ndim; k++) n *= (uint64_t)idx_strides->shape[k];
    REQUIRE(n == total, "hc_gather: index shape has %llu elements, expected %llu", (unsigned long long)n,
            (unsigned long long)total);
  }
  const size_t el = dtype_size(dtype);

  // Row form: trailing axes of the index map that cover exactly `inner` elements all have
  // stride 0, so the index depends on the row only.
  bool row_form = false;
  hc_strides row_strides;
  memset(&row_strides, 0, sizeof(row_strides));
  if (inner > 1) {
    uint64_t tail = 1;
    int k = (int)idx_strides->ndim;
    bool zero = true;
    while (k > 0 && tail < (uint64_t)inner) {
      k--;
      tail *= (uint64_t)idx_strides->shape[k];
      if (idx_strides->strides[k] != 0 && idx_strides->shape[k] != 1) zero = false;
    }
    if (zero && tail == (uint64_t)inner) {
      row_form = true;
      row_strides.ndim = (uint32_t)k;
      for (int d = 0; d < k; d++) {
        row_strides.shape[d] = idx_strides->shape[d];
        row_strides.strides[d] = idx_strides->strides[d];
      }
    }
  }
  if (row_form) {
    const size_t row_bytes = (size_t)inner * el;
    size_t vb = 16;
    while (vb > 1 && (row_bytes % vb != 0 || ((uintptr_t)in % vb) != 0 || ((uintptr_t)out % vb) != 0)) vb >>= 1;
    if (vb < el) vb = el;
    hck_gather_rows_args k;
    memset(&k, 0, sizeof(k));
    k.in = in;
    k.indices = (const int64_t*)indices;
    k.out = out;
    k.out_count = (uint32_t)out_count;
    k.middle = (uint32_t)middle;
    k.row_vecs = (uint32_t)(row_bytes / vb);
    k.total_rows = (uint32_t)(outer * out_count);
    int vec;
    uint64_t rows;
    const hc_strides* ops[] = {&row_strides};
    const void* ptrs[] = {indices};
    HC_TRY(make_bcast(1, ops, ptrs, out, 1, &k.idx, &vec, &rows));
    char name[64];
    if (vb == 16 && k.row_vecs % 64 == 0) {
      // long rows: one wave per 64 (or 256) vectors of a row
      const uint32_t t = k.row_vecs % 256 == 0 ? 4 : 1;
      snprintf(name, sizeof(name), "hc_gather_rows_wide%u", t);
      const uint64_t units = (uint64_t)k.total_rows * (k.row_vecs / (64 * t));
      return launch(ctx, name, ceil_div(units, HCK_BLOCK / 64), 1, &k, sizeof(k));
    }
    snprintf(name, sizeof(name), "hc_gather_rows_b%zu", vb);
    return launch(ctx, name, ceil_div((uint64_t)k.total_rows * k.row_vecs, HCK_BLOCK), 1, &k, sizeof(k));
  }
  hck_gather_elems_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.indices = (const int64_t*)indices;
  k.out = out;
  k.out_count = (uint32_t)out_count;
  k.middle = (uint32_t)middle;
  k.inner = (uint32_t)inner;
  k.total = (uint32_t)total;
  int vec;
  uint64_t n;
  const hc_strides* ops[] = {idx_strides};
  const void* ptrs[] = {indices};
  HC_TRY(make_bcast(1, ops, ptrs, out, 1, &k.idx, &vec, &n));
  if (out_count == 1 && inner == 1) {
    // one element per row, the rows' indices dense in memory: what follows an arg-reduction in
    // Tensor.max / min (ReduceRepeat.swift:201-209)
    bool dense = true;
    int64_t expect = 1;
    for (uint32_t d = idx_strides->ndim; d-- > 0;) {
      if (idx_strides->shape[d] == 1) continue;
      dense = dense && idx_strides->strides[d] == expect;
      expect *= idx_strides->shape[d];
    }
    if (dense) {
      note.tag = hc_pending::GATHER_ONE;
      note.meta.dtype = dtype;
      note.meta.rows = (uint64_t)outer;
      note.meta.cols = (uint64_t)middle;
      note.meta.in0 = in;
      note.meta.in1 = indices;
      note.meta.out = out;
    }
  }
  char name[64];
  snprintf(name, sizeof(name), "hc_gather_elems_b%zu", el);
  return launch(ctx, name, ceil_div(total, HCK_BLOCK), 1, &k, sizeof(k));
}

extern "C" int hc_scatter(hc_ctx* ctx, int dtype, const void* in, const void* indices,
                          const hc_strides* idx_strides, void* out, int64_t outer, int64_t middle,
                          int64_t out_count, int64_t inner, int indices_are_unique) {
  OpNote note({in, indices}, {out});
  REQUIRE(ctx && idx_strides, "hc_scatter: null argument");
  if (dtype != HC_F32 && dtype != HC_F16 && dtype != HC_I64)
    return fail(HC_ERR_UNSUPPORTED, "hc_scatter: dtype %d is not numeric", dtype);
  REQUIRE(outer >= 0 && middle >= 0 && out_count >= 0 && inner >= 0, "hc_scatter: negative dimension");
  const double in_total = (double)outer * (double)out_count * (double)inner;
  const double out_total = (double)outer * (double)middle * (double)inner;
  if (out_total == 0) return HC_OK;
  if (out_total > 4294967295.0 || in_total > 4294967295.0)
    return fail(HC_ERR_TOO_LARGE, "hc_scatter: more than 2^32-1 elements");
  REQUIRE(out, "hc_scatter: null pointer");
  const size_t n_out = (size_t)outer * (size_t)middle * (size_t)inner;
  const uint64_t total = (uint64_t)outer * (uint64_t)out_count * (uint64_t)inner;
  // Rows of at least 1 KiB in whole 16-byte vectors, index independent of the position inside
  // the row, repeated indices allowed: group the source rows by destination and add them in
  // source order, one workgroup per destination row. No atomics on the data, no zero fill, and
  // float sums come out in the CPU's order.
  if (!indices_are_unique && total != 0 && inner > 1 && idx_strides->ndim <= HC_MAX_DIMS) {
    REQUIRE(in && indices, "hc_scatter: null pointer");
    uint64_t tail = 1;
    int kd = (int)idx_strides->ndim;
    bool zero = true;
    while (kd > 0 && tail < (uint64_t)inner) {
      kd--;
      tail *= (uint64_t)idx_strides->shape[kd];
      if (idx_strides->strides[kd] != 0 && idx_strides->shape[kd] != 1) zero = false;
    }
    const size_t row_bytes = (size_t)inner * dtype_size(dtype);
    // (one workgroup per destination row: their number times the workgroup size must fit 32 bits)
    if (zero && tail == (uint64_t)inner && row_bytes % 16 == 0 && row_bytes >= 1024 && aligned16(in) &&
        aligned16(out) && (uint64_t)outer * (uint64_t)middle < (1ull << 24)) {
      uint64_t n = 1;
      for (uint32_t d = 0; d < idx_strides->ndim; d++) n *= (uint64_t)idx_strides->shape[d];
      REQUIRE(n == total, "hc_scatter: index shape has %llu elements, expected %llu", (unsigned long long)n,
              (unsigned long long)total);
      hc_strides row_strides;
      memset(&row_strides, 0, sizeof(row_strides));
      row_strides.ndim = (uint32_t)kd;
      for (int d = 0; d < kd; d++) {
        row_strides.shape[d] = idx_strides->shape[d];
        row_strides.strides[d] = idx_strides->strides[d];
      }
      const uint64_t n_buckets = (uint64_t)outer * (uint64_t)middle, n_rows = (uint64_t)outer * (uint64_t)out_count;
      Scratch scratch(ctx);
      void *counters = nullptr, *starts = nullptr, *list = nullptr;
      HC_TRY(scratch.get(2 * n_buckets * sizeof(int64_t), &counters));  // counts, then cursors
      HC_TRY(scratch.get(n_buckets * sizeof(int64_t), &starts));
      HC_TRY(scratch.get(n_rows * sizeof(uint32_t), &list));
      HC_TRY(hc_fill(ctx, HC_I64, 0.0f, 0, counters, 2 * n_buckets));
      hck_scatter_rows_args k;
      memset(&k, 0, sizeof(k));
      k.in = in;
      k.indices = (const int64_t*)indices;
      k.out = out;
      k.counts = (int64_t*)counters;
      k.cursor = (int64_t*)counters + n_buckets;
      k.starts = (const int64_t*)starts;
      k.list = (uint32_t*)list;
      k.n_src = (uint32_t)out_count;
      k.n_dst = (uint32_t)middle;
      k.row_vecs = (uint32_t)(row_bytes / 16);
      k.total_src = (uint32_t)n_rows;
      int vec;
      uint64_t rows;
      const hc_strides* ops[] = {&row_strides};
      const void* ptrs[] = {indices};
      HC_TRY(make_bcast(1, ops, ptrs, out, 1, &k.idx, &vec, &rows));
      HC_TRY(launch(ctx, "hc_scatter_rows_count", ceil_div(n_rows, HCK_BLOCK), 1, &k, sizeof(k)));
      HC_TRY(hc_cumulative(ctx, 0, HC_I64, counters, starts, 1, (int64_t)n_buckets, 1, 1, 0));
      HC_TRY(launch(ctx, "hc_scatter_rows_fill", ceil_div(n_rows, HCK_BLOCK), 1, &k, sizeof(k)));
      char name[64];
      snprintf(name, sizeof(name), "hc_scatter_rows_sum_%s", dtype_name(dtype));
      return launch(ctx, name, n_buckets, 1, &k, sizeof(k));
    }
  }
  // half values with repeated indices add up in a float buffer that is rounded once at the end
  const bool staged = dtype == HC_F16 && !indices_are_unique;
  Scratch scratch(ctx);
  void* acc = out;
  if (staged) HC_TRY(scratch.get(n_out * 4, &acc));
  HC_TRY(hc_fill(ctx, staged ? HC_F32 : dtype, 0.0f, 0, acc, n_out));
  if (total != 0) {
    REQUIRE(in && indices, "hc_scatter: null pointer");
    uint64_t n = 1;
    REQUIRE(idx_strides->ndim <= HC_MAX_DIMS, "hc_scatter: ndim %u exceeds %d", idx_strides->ndim, HC_MAX_DIMS);
    for (uint32_t k = 0; k < idx_strides->ndim; k++) n *= (uint64_t)idx_strides->shape[k];
    REQUIRE(n == total, "hc_scatter: index shape has %llu elements, expected %llu", (unsigned long long)n,
            (unsigned long long)total);
    hck_gather_elems_args k;
    memset(&k, 0, sizeof(k));
    k.in = in;
    k.indices = (const int64_t*)indices;
    k.out = acc;
    k.out_count = (uint32_t)out_count;
    k.middle = (uint32_t)middle;
    k.inner = (uint32_t)inner;
    k.total = (uint32_t)total;
    int vec;
    const hc_strides* ops[] = {idx_strides};
    const void* ptrs[] = {indices};
    HC_TRY(make_bcast(1, ops, ptrs, acc, 1, &k.idx, &vec, &n));
    char name[64];
    if (indices_are_unique) snprintf(name, sizeof(name), "hc_scatter_set_b%zu", dtype_size(dtype));
    else snprintf(name, sizeof(name), "hc_scatter_add_%s", dtype_name(dtype));
    HC_TRY(launch(ctx, name, ceil_div(total, HCK_BLOCK), 1, &k, sizeof(k)));
  }
  if (staged) HC_TRY(hc_cast(ctx, acc, HC_F32, out, HC_F16, n_out));
  return HC_OK;
}

extern "C" int hc_adamw(hc_ctx* ctx, int dtype, const void* param, const void* grad, const void* moment1,
                        const void* moment2, float beta1, float beta2, float eps, float weight_decay,
                        float lr, float step, size_t count, void* out_param, void* out_moment1,
                        void* out_moment2) {
  OpNote note({param, grad, moment1, moment2}, {out_param, out_moment1, out_moment2});
  REQUIRE(ctx, "hc_adamw: null context");
  if (dtype != HC_F32 && dtype != HC_F16)
    return fail(HC_ERR_UNSUPPORTED, "hc_adamw: dtype %d is not a float type", dtype);
  if (count == 0) return HC_OK;
  REQUIRE(param && grad && moment1 && moment2 && out_param && out_moment1 && out_moment2,
          "hc_adamw: null pointer");
  hck_adamw_args k;
  memset(&k, 0, sizeof(k));
  k.param = param;
  k.grad = grad;
  k.m1 = moment1;
  k.m2 = moment2;
  k.out_param = out_param;
  k.out_m1 = out_moment1;
  k.out_m2 = out_moment2;
  k.count = count;
  // the scalars of Backend.swift:818-892, all formed in Float
  k.beta1 = beta1;
  k.one_minus_beta1 = 1.0f - beta1;
  k.beta2 = beta2;
  k.one_minus_beta2 = 1.0f - beta2;
  k.bias1 = 1.0f / (1.0f - powf(beta1, step));
  k.bias2 = 1.0f / (1.0f - powf(beta2, step));
  k.eps = eps;
  k.lr = lr;
  k.decay = 1.0f - lr * weight_decay;
  k.exp_square = 2.0f;
  k.exp_root = 0.5f;
  char name[64];
  snprintf(name, sizeof(name), "hc_adamw_%s", dtype_name(dtype));
  REQUIRE(aligned16(param) && aligned16(grad) && aligned16(moment1) && aligned16(moment2) && aligned16(out_param) &&
              aligned16(out_moment1) && aligned16(out_moment2),
          "hc_adamw: buffers must be 16-byte aligned");
  // one 16-byte vector per lane (the kernel's loop only matters beyond 2^31 blocks)
  uint64_t blocks = ceil_div(ceil_div(count, 16 / dtype_size(dtype)), HCK_BLOCK);
  if (blocks > 0x7fffffffull) blocks = 0x7fffffffull;
  return launch(ctx, name, blocks, 1, &k, sizeof(k));
}

extern "C" int hc_axis_permutation(hc_ctx* ctx, const int64_t* perm, const int64_t* shape, int ndim,
                                   void* out) {
  OpNote note({}, {out});
  REQUIRE(ctx, "hc_axis_permutation: null context");
  REQUIRE(ndim >= 0 && ndim <= HC_MAX_DIMS, "hc_axis_permutation: ndim %d out of range", ndim);
  REQUIRE(ndim == 0 || (perm && shape), "hc_axis_permutation: null argument");
  hck_axis_perm_args k;
  memset(&k, 0, sizeof(k));
  uint64_t total = 1;
  int64_t old_strides[HC_MAX_DIMS];
  bool seen[HC_MAX_DIMS] = {false};
  for (int d = ndim - 1; d >= 0; d--) {
    REQUIRE(shape[d] >= 0, "hc_axis_permutation: negative extent");
    old_strides[d] = (int64_t)total;
    total *= (uint64_t)shape[d];
    if (total > 0xffffffffull) return fail(HC_ERR_TOO_LARGE, "hc_axis_permutation: more than 2^32-1 elements");
  }
  for (int d = 0; d < ndim; d++) {
    REQUIRE(perm[d] >= 0 && perm[d] < ndim && !seen[perm[d]], "hc_axis_permutation: invalid permutation");
    seen[perm[d]] = true;
  }
  if (total == 0) return HC_OK;
  REQUIRE(out, "hc_axis_permutation: null output");
  uint64_t acc = 1;
  for (int d = ndim - 1; d >= 0; d--) {
    k.new_shape[d] = (uint32_t)shape[perm[d]];
    k.permuted_strides[d] = (uint32_t)old_strides[perm[d]];
    k.new_strides[d] = (uint32_t)acc;
    acc *= (uint64_t)shape[perm[d]];
  }
  k.out = (int64_t*)out;
  k.total = (uint32_t)total;
  k.ndim = (uint32_t)ndim;
  return launch(ctx, "hc_axis_permutation", ceil_div(total, HCK_BLOCK), 1, &k, sizeof(k));
}

extern "C" int hc_permute(hc_ctx* ctx, int dtype, const void* in, const int64_t* perm, const int64_t* shape,
                          int ndim, int64_t inner, void* out) {
  OpNote note({in}, {out});
  REQUIRE(ctx, "hc_permute: null context");
  REQUIRE(dtype_name(dtype), "hc_permute: bad dtype %d", dtype);
  REQUIRE(ndim >= 0 && ndim <= HC_MAX_DIMS, "hc_permute: ndim %d out of range", ndim);
  REQUIRE(ndim == 0 || (perm && shape), "hc_permute: null argument");
  REQUIRE(inner >= 0, "hc_permute: negative inner count");
  const size_t el = dtype_size(dtype);
  bool seen[HC_MAX_DIMS] = {false};
  uint64_t total = (uint64_t)inner;
  for (int d = 0; d < ndim; d++) {
    REQUIRE(shape[d] >= 0, "hc_permute: negative extent");
    REQUIRE(perm[d] >= 0 && perm[d] < ndim && !seen[perm[d]], "hc_permute: invalid permutation");
    seen[perm[d]] = true;
    total *= (uint64_t)shape[d];
    if (total > 0xffffffffull) return fail(HC_ERR_TOO_LARGE, "hc_permute: more than 2^32-1 elements");
  }
  if (total == 0) return HC_OK;
  REQUIRE(in && out, "hc_permute: null pointer");
  // Axes in output order with their source strides (elements); the untouched trailing block is
  // one more innermost axis. Unit axes go, axes adjacent in both orders merge.
  struct Axis { uint64_t extent, stride; };
  Axis ax[HC_MAX_DIMS + 1];
  int n = 0;
  for (int d = 0; d < ndim; d++) {
    uint64_t stride = (uint64_t)inner;
    for (int e = (int)perm[d] + 1; e < ndim; e++) stride *= (uint64_t)shape[e];
    if (shape[perm[d]] == 1) continue;
    if (n > 0 && ax[n - 1].stride == stride * (uint64_t)shape[perm[d]]) {
      ax[n - 1].extent *= (uint64_t)shape[perm[d]];
      ax[n - 1].stride = stride;
    } else {
      ax[n].extent = (uint64_t)shape[perm[d]];
      ax[n].stride = stride;
      n++;
    }
  }
  if (inner > 1) {
    if (n > 0 && ax[n - 1].stride == (uint64_t)inner) {
      ax[n - 1].extent *= (uint64_t)inner;
      ax[n - 1].stride = 1;
    } else {
      ax[n].extent = (uint64_t)inner;
      ax[n].stride = 1;
      n++;
    }
  }
  hck_permute_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.out = out;
  char name[64];
  if (n == 0 || ax[n - 1].stride == 1) {
    // row form: the innermost axis is the same in source and output
    const uint64_t row_len = n == 0 ? 1 : ax[n - 1].extent;
    const int rows_n = n == 0 ? 0 : n - 1;
    uint32_t vec = (uint32_t)(16 / el);
    if (row_len % vec != 0 || !aligned16(in) || !aligned16(out)) vec = 1;
    for (int d = 0; d < rows_n && vec > 1; d++)
      if (ax[d].stride % vec != 0) vec = 1;
    k.ndim = (uint32_t)rows_n;
    k.inner = (uint32_t)row_len;
    k.inner_vecs = (uint32_t)(row_len / vec);
    k.total = (uint32_t)(total / vec);
    hck_fast_div_setup(k.inner_vecs, &k.inner_magic, &k.inner_sh);
    for (int d = 0; d < rows_n; d++) {
      k.shape[d] = (uint32_t)ax[d].extent;
      k.in_stride[d] = (uint32_t)ax[d].stride;
      hck_fast_div_setup(k.shape[d], &k.magic[d], &k.sh[d]);
    }
    if (n >= 2) {
      note.tag = hc_pending::PERMUTE;
      note.meta.dtype = dtype;
      note.meta.in0 = in;
      note.meta.out = out;
      note.meta.pn = n;
      for (int d = 0; d < n; d++) {
        note.meta.pext[d] = ax[d].extent;
        note.meta.pstr[d] = ax[d].stride;
      }
    }
    snprintf(name, sizeof(name), "hc_permute_rows_b%zu_%s", el, vec > 1 ? "vN" : "v1");
    return launch(ctx, name, ceil_div((uint64_t)k.total, HCK_BLOCK), 1, &k, sizeof(k));
  }
  // tile form: the output's innermost axis a is not the source's innermost axis c
  int c = -1;
  for (int d = 0; d < n; d++)
    if (ax[d].stride == 1) c = d;
  REQUIRE(c >= 0 && c != n - 1, "hc_permute: internal error (no contiguous source axis)");
  uint64_t out_stride[HC_MAX_DIMS + 1];
  uint64_t acc = 1;
  for (int d = n - 1; d >= 0; d--) {
    out_stride[d] = acc;
    acc *= ax[d].extent;
  }
  k.tile_a = (uint32_t)ax[n - 1].extent;
  k.a_stride = (uint32_t)ax[n - 1].stride;
  k.tile_c = (uint32_t)ax[c].extent;
  k.c_out_stride = (uint32_t)out_stride[c];
  // 64 x 64 tiles; when one of the two axes is shorter, the tile grows along the other (4096 elements)
  auto log2_ceil = [](uint64_t v) {
    uint32_t l = 0;
    while ((1ull << l) < v) l++;
    return l;
  };
  const uint32_t la = log2_ceil(ax[n - 1].extent), lc = log2_ceil(ax[c].extent);
  k.ta_log2 = std::min<uint32_t>(la, 6);
  k.tc_log2 = std::min<uint32_t>(lc, 6);
  if (k.tc_log2 < 6) k.ta_log2 = std::min<uint32_t>(la, std::min<uint32_t>(12 - k.tc_log2, 10));  // (LDS rows are padded)
  if (k.ta_log2 < 6) k.tc_log2 = std::min<uint32_t>(lc, 12 - k.ta_log2);
  k.tiles_a = (uint32_t)ceil_div(ax[n - 1].extent, 1ull << k.ta_log2);
  k.tiles_c = (uint32_t)ceil_div(ax[c].extent, 1ull << k.tc_log2);
  hck_fast_div_setup(k.tiles_a, &k.tiles_a_magic, &k.tiles_a_sh);
  hck_fast_div_setup(k.tiles_c, &k.tiles_c_magic, &k.tiles_c_sh);
  uint64_t batch = 1;
  for (int d = 0; d < n - 1; d++) {
    if (d == c) continue;
    k.shape[k.ndim] = (uint32_t)ax[d].extent;
    k.in_stride[k.ndim] = (uint32_t)ax[d].stride;
    k.out_stride[k.ndim] = (uint32_t)out_stride[d];
    hck_fast_div_setup(k.shape[k.ndim], &k.magic[k.ndim], &k.sh[k.ndim]);
    batch *= ax[d].extent;
    k.ndim++;
  }
  const uint64_t tiles = batch * k.tiles_a * k.tiles_c;
  if (tiles > 0x7fffffffull) return fail(HC_ERR_TOO_LARGE, "hc_permute: too many tiles");
  k.total = (uint32_t)tiles;
  snprintf(name, sizeof(name), "hc_permute_tile_b%zu", el);
  return launch(ctx, name, tiles, 1, &k, sizeof(k));
}

extern "C" int hc_triangular(hc_ctx* ctx, int dtype, const void* in, void* out, int64_t batch,
                             int64_t rows, int64_t cols, int upper, int64_t offset) {
  OpNote note({in}, {out});
  REQUIRE(ctx, "hc_triangular: null context");
  REQUIRE(dtype_name(dtype), "hc_triangular: bad dtype %d", dtype);
  REQUIRE(batch >= 0 && rows >= 0 && cols >= 0, "hc_triangular: negative dimension");
  const double total = (double)batch * (double)rows * (double)cols;
  if (total == 0) return HC_OK;
  if (total > 4294967295.0) return fail(HC_ERR_TOO_LARGE, "hc_triangular: more than 2^32-1 elements");
  REQUIRE(in && out, "hc_triangular: null pointer");
  hck_triangular_args k;
  memset(&k, 0, sizeof(k));
  k.in = in;
  k.out = out;
  k.total = (uint32_t)(batch * rows * cols);
  k.rows = (uint32_t)rows;
  k.cols = (uint32_t)cols;
  k.upper = upper ? 1 : 0;
  k.offset = offset;
  char name[64];
  const size_t el = dtype_size(dtype);
  if (((uint64_t)cols * el) % 16 == 0 && aligned16(in) && aligned16(out)) {  // 16 bytes of a row per lane
    k.total = (uint32_t)((uint64_t)k.total * el / 16);
    snprintf(name, sizeof(name), "hc_triangular_b%zu_vN", el);
    return launch(ctx, name, ceil_div(k.total, HCK_BLOCK), 1, &k, sizeof(k));
  }
  snprintf(name, sizeof(name), "hc_triangular_b%zu", el);
  return launch(ctx, name, ceil_div(k.total, HCK_BLOCK), 1, &k, sizeof(k));
}

extern "C" int hc_concat(hc_ctx* ctx, int dtype, const void* const* inputs, const int64_t* inner_counts,
                         int n_inputs, int64_t outer, void* out) {
  OpNote note({}, {out});
  if (inputs)
    for (int i = 0; i < n_inputs; i++) note.reads.push_back(inputs[i]);
  REQUIRE(ctx, "hc_concat: null context");
  REQUIRE(dtype_name(dtype), "hc_concat: bad dtype %d", dtype);
  REQUIRE(n_inputs >= 0 && outer >= 0, "hc_concat: negative count");
  REQUIRE(n_inputs == 0 || (inputs && inner_counts), "hc_concat: null argument");
  const size_t el = dtype_size(dtype);
  uint64_t total_inner = 0;
  for (int t = 0; t < n_inputs; t++) {
    REQUIRE(inner_counts[t] >= 0, "hc_concat: negative inner count");
    total_inner += (uint64_t)inner_counts[t] * el;
  }
  if (total_inner > 0xffffffffull || (uint64_t)outer > 0xffffffffull)
    return fail(HC_ERR_TOO_LARGE, "hc_concat: slice larger than 2^32-1 bytes");
  uint64_t off = 0;
  for (int t = 0; t < n_inputs; t++) {
    const uint64_t bytes = (uint64_t)inner_counts[t] * el;
    if (bytes != 0 && outer != 0) {
      REQUIRE(inputs[t] && out, "hc_concat: null pointer");
      hck_concat_args k;
      memset(&k, 0, sizeof(k));
      // the widest unit that every row piece and both addresses are multiples of
      uint64_t unit = 16;
      while (unit > 1 && ((bytes | total_inner | off | (uint64_t)(uintptr_t)inputs[t] | (uint64_t)(uintptr_t)out) & (unit - 1)) != 0)
        unit >>= 1;
      k.in = inputs[t];
      k.out = out;
      k.outer = (uint32_t)outer;
      k.inner = (uint32_t)(bytes / unit);
      k.total_inner = (uint32_t)(total_inner / unit);
      k.out_off = (uint32_t)(off / unit);
      char name[32];
      snprintf(name, sizeof(name), "hc_concat_b%u", (unsigned)unit);
      HC_TRY(launch(ctx, name, ceil_div((uint64_t)outer * (bytes / unit), HCK_BLOCK), 1, &k, sizeof(k)));
    }
    off += bytes;
  }
  return HC_OK;
}

// ------------------------------------------------------------------ matmul
#include "hchip_matmul.inc"
