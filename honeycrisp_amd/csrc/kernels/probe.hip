// Measurement kernel: the fp16 MFMA pipe with nothing else going on. Every wave keeps four A
// and four B operand fragments in registers, taken from a buffer the caller supplies (so the
// bit patterns are those of the caller's matrices), and issues the same 4 x 4 grid of
// 32x32x16 MFMAs per step as a wave of the 256x256 GEMM tile does, with no loads, LDS traffic
// or barriers in the loop. Timed with the caller's data it gives the rate the matrix cores
// sustain at the clock the board's power management settles on for those bit patterns: the
// ceiling a GEMM on that data can approach.
#include "common.hip.h"
#include "../kargs.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

HC_KERNEL void hc_probe_mfma_f16(hck_probe_args p) {
  const uint32_t tid = blockIdx.x * HCK_BLOCK + threadIdx.x;
  const half8* data = (const half8*)p.data;
  half8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = data[((uint64_t)tid * 8 + i) % p.chunks];
    b[i] = data[((uint64_t)tid * 8 + 4 + i) % p.chunks];
  }
  floatx16 acc[4][4] = {};
  for (uint32_t it = 0; it < p.iters; it++) {
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int i = 0; i < 4; i++)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[j], a[i], acc[i][j], 0, 0, 0);
    // rotate the A fragments: consecutive steps pair different operands, as fresh K-slices would
    const half8 t = a[0];
    a[0] = a[1];
    a[1] = a[2];
    a[2] = a[3];
    a[3] = t;
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) s += acc[i][j][e];
  ((float*)p.out)[tid] = s;
}
