// Measurement kernels: the fp16 MFMA pipe with nothing else going on. Every wave keeps four A
// and four B operand fragments in registers, taken from a buffer the caller supplies (so the
// bit patterns are those of the caller's matrices), and issues MFMAs on a 128 x 128 wave tile
// of accumulators, with no loads, LDS traffic or barriers in the loop. Timed with the caller's
// data this gives the rate the matrix cores sustain at the clock the board's power management
// settles on for those bit patterns: the ceiling a GEMM on that data can approach.
// Two instruction shapes: 32x32x16 (16 accumulator tiles of 16 registers) and 16x16x32 (64
// tiles of 4 registers; per multiply-accumulate it moves half as many accumulator registers and
// runs at a higher clock under the same power limit). The MFMAs are written as assembly so
// that the accumulators stay in the accumulation registers.
//
// Belongs to bench.py, not to the library: bench.py loads the code object built from this file
// (`hipcc --genco`, see __graft_entry__.build) through hc_module_load and launches it with
// hc_launch, one 256-lane workgroup per compute unit.
#include <hip/hip_runtime.h>

#include <stdint.h>
#include <type_traits>

#define HCK_BLOCK 256
#define HC_KERNEL extern "C" __global__ __launch_bounds__(HCK_BLOCK)

// `chunks` 16-byte pieces of operand bit patterns at `data`; one float per lane goes to `out`
// so that the arithmetic cannot be dropped. The kernel's only parameter (24 bytes of kernarg).
typedef struct {
  const void* data;
  void* out;
  uint32_t iters;
  uint32_t chunks;
} hck_probe_args;

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

template <int N, typename F> __device__ __forceinline__ void probe_static_for(F&& f) {
  if constexpr (N > 0) {
    probe_static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

__device__ __forceinline__ void probe_load(const hck_probe_args& p, uint32_t tid, half8 (&a)[4], half8 (&b)[4]) {
  const half8* data = (const half8*)p.data;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = data[((uint64_t)tid * 8 + i) % p.chunks];
    b[i] = data[((uint64_t)tid * 8 + 4 + i) % p.chunks];
  }
}

HC_KERNEL void hc_probe_mfma_f16_32x32x16(hck_probe_args p) {
  const uint32_t tid = blockIdx.x * HCK_BLOCK + threadIdx.x;
  half8 a[4], b[4];
  probe_load(p, tid, a, b);
  floatx16 acc[16];
  probe_static_for<16>([&](auto tc) {
#pragma unroll
    for (int e = 0; e < 16; e++) acc[decltype(tc)::value][e] = 0.0f;
  });
  // (a plain lambda: the assembly statement does not compile inside a generic one)
  auto mma = [&](int t) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[t]) : "v"(b[t / 4]), "v"(a[t % 4]));
  };
  for (uint32_t it = 0; it < p.iters; it++) probe_static_for<16>([&](auto tc) { mma(decltype(tc)::value); });
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // the compiler does not know the statements above are MFMAs
  float s = 0.0f;
  probe_static_for<16>([&](auto tc) {
#pragma unroll
    for (int e = 0; e < 16; e++) s += acc[decltype(tc)::value][e];
  });
  ((float*)p.out)[tid] = s;
}

HC_KERNEL void hc_probe_mfma_f16_16x16x32(hck_probe_args p) {
  const uint32_t tid = blockIdx.x * HCK_BLOCK + threadIdx.x;
  half8 a[4], b[4];
  probe_load(p, tid, a, b);
  floatx4 acc[64];
  probe_static_for<64>([&](auto tc) {
#pragma unroll
    for (int e = 0; e < 4; e++) acc[decltype(tc)::value][e] = 0.0f;
  });
  // 64 MFMAs of 16 x 16 x 32 = 32 k of the 128 x 128 wave tile: the work of 16 of the other shape
  // over two of these steps, so a launch with the same `iters` does the same work
  auto mma = [&](int t) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[t]) : "v"(b[(t / 8) % 4]), "v"(a[t % 4]));
  };
  for (uint32_t it = 0; it < p.iters / 2; it++) probe_static_for<64>([&](auto tc) { mma(decltype(tc)::value); });
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  float s = 0.0f;
  probe_static_for<64>([&](auto tc) {
#pragma unroll
    for (int e = 0; e < 4; e++) s += acc[decltype(tc)::value][e];
  });
  ((float*)p.out)[tid] = s;
}

// A kernel that does nothing: bench.py launches it in front of and behind each measured region,
// with a grid of `region number` workgroups of 64 lanes, so that a kernel trace of the run can be
// cut into those regions by name and grid size (launches of the untimed spin-up and warm-up
// steps must not count towards a region's averages).
extern "C" __global__ __launch_bounds__(64) void hc_bench_marker(hck_probe_args p) { (void)p; }
