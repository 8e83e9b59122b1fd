// Tuned fp16 GEMM for gfx950 (fp32 accumulate, v_mfma_f32_32x32x16_f16) for problems whose
// M, N are multiples of the block tile and K a multiple of 64; every transpose combination.
//
// Block tile BM x BN x 64, 256 lanes = 4 waves in a 2 x 2 grid, each wave (BM/2) x (BN/2)
// outputs held as (BM/64) x (BN/64) MFMA 32x32 accumulators (256 fp32 registers per lane
// for the 256 x 256 tile: the AGPR file, at one wave per SIMD).
//
// LDS: two stages of [BM + BN rows][64 halfs], K-contiguous, no padding. A row is eight
// 16-byte chunks; chunk c of row r is stored at slot c ^ f(r), f(r) = (r ^ (r >> 3)) & 7.
// With this XOR swizzle the three access patterns are bank-conflict free:
//   MFMA operand reads   32 consecutive rows, same chunk        -> 8 rows hit 8 slots
//   K-contiguous writes  8 lanes write the 8 chunks of one row  -> one full 128-byte row
//   transposed writes    32 lanes write rows 8 apart, same chunk -> f differs via r >> 3
//
// Pipeline per K-step: issue the global loads of step k+1 into registers, run the MFMAs
// of step k out of LDS stage k&1, then store the registers to stage (k+1)&1; one barrier
// per step. Operands contiguous along M/N are transposed in registers (an 8 x 8 or 4 x 8
// block of halfs per lane) on their way to LDS so that LDS is always K-contiguous.
//
// Workgroup ids are remapped so that the workgroups one XCD receives (ids equal mod 8)
// cover a contiguous band of tiles and share A / B panels in that XCD's L2.
#include "common.hip.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

enum { FAST_LOAD_K = 0, FAST_LOAD_MN = 1 };

typedef uint32_t Chunk __attribute__((ext_vector_type(4)));  // 16 bytes = 8 halfs

__device__ __forceinline__ uint32_t swz(uint32_t row) { return (row ^ (row >> 3)) & 7u; }

// Registers for one operand's share of a K-step: ROWS x 128 bytes / 256 lanes.
template <int ROWS> struct Stage {
  Chunk v[ROWS / 32];
};

// Global -> registers. The operand tile is rows [r0, r0 + ROWS) x k [k0, k0 + 64); logical
// element (r, k) is at base[r * rs + k * cs] with cs == 1 (FAST_LOAD_K) or rs == 1
// (FAST_LOAD_MN). Everything is in range and 16-byte aligned (checked by the host).
template <int ROWS, int MODE>
__device__ __forceinline__ void fetch(Stage<ROWS>& st, const half_t* base, uint32_t rs, uint32_t cs,
                                      uint32_t r0, uint32_t k0) {
  constexpr int N = ROWS / 32;
  const uint32_t t = threadIdx.x;
  if (MODE == FAST_LOAD_K) {
#pragma unroll
    for (int i = 0; i < N; i++) {
      const uint32_t id = t + 256 * i;
      st.v[i] = *reinterpret_cast<const Chunk*>(base + (size_t)(r0 + id / 8) * rs + k0 + (id % 8) * 8);
    }
  } else {
    constexpr int MB = ROWS / 8;  // 16-byte blocks along m/n; N k-rows per lane
    const uint32_t r = r0 + (t % MB) * 8, kb = k0 + (t / MB) * N;
#pragma unroll
    for (int i = 0; i < N; i++) st.v[i] = *reinterpret_cast<const Chunk*>(base + (size_t)(kb + i) * cs + r);
  }
}

// Registers -> LDS stage (K-contiguous, swizzled).
template <int ROWS, int MODE> __device__ __forceinline__ void stash(const Stage<ROWS>& st, char* lds) {
  constexpr int N = ROWS / 32;
  const uint32_t t = threadIdx.x;
  if (MODE == FAST_LOAD_K) {
#pragma unroll
    for (int i = 0; i < N; i++) {
      const uint32_t id = t + 256 * i;
      const uint32_t r = id / 8, c = id % 8;
      *reinterpret_cast<Chunk*>(lds + r * 128 + ((c ^ swz(r)) * 16)) = st.v[i];
    }
  } else {
    constexpr int MB = ROWS / 8;
    const uint32_t r = (t % MB) * 8, kb = (t / MB) * N;  // kb: first of N consecutive k
    half8 h[N];  // h[i][p] = element (k = kb + i, row r + p)
#pragma unroll
    for (int i = 0; i < N; i++) h[i] = __builtin_bit_cast(half8, st.v[i]);
    const uint32_t c = kb / 8, within = (kb % 8) * 2;
#pragma unroll
    for (int p = 0; p < 8; p++) {
      typedef _Float16 halfN __attribute__((ext_vector_type(N)));
      halfN col;
#pragma unroll
      for (int i = 0; i < N; i++) col[i] = h[i][p];
      const uint32_t row = r + p;
      *reinterpret_cast<halfN*>(lds + row * 128 + ((c ^ swz(row)) * 16) + within) = col;
    }
  }
}

template <int BM, int BN, int MODE_A, int MODE_B>
__device__ __forceinline__ void gemm_fast_impl(const hck_gemm_args& p, char* lds) {
  constexpr int MT = BM / 64, NT = BN / 64;       // MFMA tiles per wave along m, n
  constexpr int STAGE_BYTES = (BM + BN) * 128;

  // XCD-aware tile order: ids equal mod 8 land on one XCD; give that XCD a contiguous band.
  const uint32_t total = p.tiles_m * p.tiles_n;
  uint32_t tile = blockIdx.x;
  if ((total & 7u) == 0) tile = (blockIdx.x & 7u) * (total >> 3) + (blockIdx.x >> 3);
  const uint32_t tm = tile / p.tiles_n, tn = tile - tm * p.tiles_n;
  const uint32_t m0 = tm * BM, n0 = tn * BN;
  const uint32_t batch = blockIdx.y;
  const half_t* A = (const half_t*)p.a + batch * p.a_bs;
  const half_t* B = (const half_t*)p.b + batch * p.b_bs;
  half_t* C = (half_t*)p.c + batch * p.c_bs;

  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t wm = (wave >> 1) * (BM / 2), wn = (wave & 1) * (BN / 2);
  const uint32_t lrow = lane & 31, lgrp = lane >> 5;

  floatx16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

  Stage<BM> sa;
  Stage<BN> sb;
  fetch<BM, MODE_A>(sa, A, p.a_rs, p.a_cs, m0, 0);
  fetch<BN, MODE_B>(sb, B, p.b_cs, p.b_rs, n0, 0);
  stash<BM, MODE_A>(sa, lds);
  stash<BN, MODE_B>(sb, lds + BM * 128);
  __syncthreads();

  const uint32_t nk = p.K / 64;
  for (uint32_t ks = 0; ks < nk; ks++) {
    char* cur = lds + (ks & 1) * STAGE_BYTES;
    char* nxt = lds + ((ks + 1) & 1) * STAGE_BYTES;
    const bool more = ks + 1 < nk;
    if (more) {
      fetch<BM, MODE_A>(sa, A, p.a_rs, p.a_cs, m0, (ks + 1) * 64);
      fetch<BN, MODE_B>(sb, B, p.b_cs, p.b_rs, n0, (ks + 1) * 64);
    }
    const char* la = cur;
    const char* lb = cur + BM * 128;
#pragma unroll
    for (int s = 0; s < 4; s++) {
      Chunk fa[MT], fb[NT];
      const uint32_t c = 2 * s + lgrp;
#pragma unroll
      for (int i = 0; i < MT; i++) {
        const uint32_t r = wm + i * 32 + lrow;
        fa[i] = *reinterpret_cast<const Chunk*>(la + r * 128 + ((c ^ swz(r)) * 16));
      }
#pragma unroll
      for (int j = 0; j < NT; j++) {
        const uint32_t r = wn + j * 32 + lrow;
        fb[j] = *reinterpret_cast<const Chunk*>(lb + r * 128 + ((c ^ swz(r)) * 16));
      }
#pragma unroll
      for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, fa[i]),
                                                             __builtin_bit_cast(half8, fb[j]), acc[i][j], 0, 0, 0);
    }
    if (more) {
      stash<BM, MODE_A>(sa, nxt);
      stash<BN, MODE_B>(sb, nxt + BM * 128);
    }
    __syncthreads();
  }

  // Accumulator layout of the 32x32 MFMA: lane l, register v = row 8*(v/4) + 4*(l/32) + v%4,
  // column l%32. c_cs == 1 (row-major output).
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < NT; j++) {
      const uint32_t col = n0 + wn + j * 32 + lrow;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const uint32_t row = m0 + wm + i * 32 + 8 * (v / 4) + 4 * lgrp + (v % 4);
        C[(size_t)row * p.c_rs + col] = narrow<half_t>(acc[i][j][v]);
      }
    }
}

#define DEF_FAST(BM, BN, AN, AM, BNAME, BMODE)                                                        \
  extern "C" __global__ __launch_bounds__(256) void hc_gemm_f16_fast_##BM##x##BN##_##AN##BNAME(       \
      hck_gemm_args p) {                                                                              \
    __shared__ __attribute__((aligned(16))) char lds[2 * (BM + BN) * 128];                            \
    gemm_fast_impl<BM, BN, AM, BMODE>(p, lds);                                                        \
  }
#define DEF_FAST_TILE(BM, BN)                                                                         \
  DEF_FAST(BM, BN, k, FAST_LOAD_K, k, FAST_LOAD_K)                                                    \
  DEF_FAST(BM, BN, k, FAST_LOAD_K, n, FAST_LOAD_MN)                                                   \
  DEF_FAST(BM, BN, m, FAST_LOAD_MN, k, FAST_LOAD_K)                                                   \
  DEF_FAST(BM, BN, m, FAST_LOAD_MN, n, FAST_LOAD_MN)
DEF_FAST_TILE(256, 256)
DEF_FAST_TILE(256, 128)
DEF_FAST_TILE(128, 128)
