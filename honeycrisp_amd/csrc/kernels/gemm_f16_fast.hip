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
// Software pipeline, hand-scheduled at source level (sched_barrier pins the order), one
// workgroup barrier per K-step. A K-step is four 16-wide sub-steps; in each, the MFMA
// operands of the next sub-step are read from LDS while the current MFMAs run:
//   sub-step 0  + store the registers holding K-step k+1 to the other LDS stage
//   sub-step 1  + issue the global loads of K-step k+2 into those registers
//   sub-step 2
//   sub-step 3  first half, barrier, operands of K-step k+1 / sub-step 0, second half
// Operands contiguous along M/N are transposed in registers (an 8 x 8 or 4 x 8 block of
// halfs per lane) on their way to LDS so that LDS is always K-contiguous.
//
// Workgroup ids are remapped so that the workgroups one XCD receives (ids equal mod 8)
// cover a contiguous band of tiles and share A / B panels in that XCD's L2.
#include "common.hip.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t Chunk __attribute__((ext_vector_type(4)));  // 16 bytes = 8 halfs

enum { FAST_LOAD_K = 0, FAST_LOAD_MN = 1 };

__device__ __forceinline__ uint32_t swz(uint32_t row) { return (row ^ (row >> 3)) & 7u; }

// One operand's share of a K-step in registers: ROWS x 128 bytes / 256 lanes = ROWS/32 chunks.
// FAST_LOAD_K: chunk u is (row (t + 256u) / 8, k-chunk (t + 256u) % 8).
// FAST_LOAD_MN: chunk u is k-row kb + u, rows r .. r+7 (r = 8 * (t % (ROWS/8)),
// kb = (ROWS/32) * (t / (ROWS/8))).
template <int ROWS, int MODE> struct Operand {
  static constexpr int N = ROWS / 32;                         // global loads per lane and step
  static constexpr int STORES = MODE == FAST_LOAD_K ? N : 8;  // LDS stores per lane and step
  Chunk v[N];
  const half_t* src[N];  // this lane's global addresses at k = 0
  uint32_t kstride;      // elements between consecutive k
  uint32_t dst[STORES];  // byte offsets inside an LDS stage (operand-relative)

  __device__ __forceinline__ void init(const half_t* base, uint32_t rs, uint32_t cs, uint32_t r0) {
    const uint32_t t = threadIdx.x;
    if (MODE == FAST_LOAD_K) {
      kstride = 1;
#pragma unroll
      for (int u = 0; u < N; u++) {
        const uint32_t id = t + 256 * u, r = id / 8, c = id % 8;
        src[u] = base + (size_t)(r0 + r) * rs + c * 8;
        dst[u] = r * 128 + ((c ^ swz(r)) * 16);
      }
    } else {
      constexpr int MB = ROWS / 8;
      const uint32_t r = (t % MB) * 8, kb = (t / MB) * N;
      kstride = cs;
#pragma unroll
      for (int u = 0; u < N; u++) src[u] = base + (size_t)(kb + u) * cs + r0 + r;
      const uint32_t c = kb / 8, within = (kb % 8) * 2;
#pragma unroll
      for (int q = 0; q < 8; q++) {
        const uint32_t row = r + q;
        dst[q] = row * 128 + ((c ^ swz(row)) * 16) + within;
      }
    }
  }

  __device__ __forceinline__ void load(int u, uint32_t k0) {
    v[u] = *reinterpret_cast<const Chunk*>(src[u] + (size_t)k0 * kstride);
  }

  __device__ __forceinline__ void store(int u, char* lds) const {
    if (MODE == FAST_LOAD_K) {
      *reinterpret_cast<Chunk*>(lds + dst[u]) = v[u];
    } else {
      // column u of this lane's N x 8 block: N consecutive k for row r + u
      typedef _Float16 halfN __attribute__((ext_vector_type(N)));
      halfN col;
#pragma unroll
      for (int i = 0; i < N; i++) col[i] = __builtin_bit_cast(half8, v[i])[u];
      *reinterpret_cast<halfN*>(lds + dst[u]) = col;
    }
  }
};

// Workgroup barrier that orders LDS traffic only (no wait on outstanding global loads).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// MFMA operands of one 16-wide k sub-step for a wave: NT chunks of B rows, MT of A rows.
template <int MT, int NT> struct Frags {
  Chunk b[NT];
  Chunk a[MT];
};

template <int BM, int BN, int MODE_A, int MODE_B>
__device__ __forceinline__ void gemm_fast_impl(const hck_gemm_args& p, char* lds) {
  constexpr int MT = BM / 64, NT = BN / 64;  // MFMA tiles per wave along m, n
  constexpr int SLOTS = MT * NT;             // MFMAs per sub-step
  constexpr int READS = MT + NT;             // LDS operand reads per sub-step
  constexpr int STAGE_BYTES = (BM + BN) * 128;
  typedef Operand<BM, MODE_A> OpA;
  typedef Operand<BN, MODE_B> OpB;
  constexpr int NSTORE = OpA::STORES + OpB::STORES;
  constexpr int NLOAD = OpA::N + OpB::N;
  constexpr int STORES_PER_SLOT = (NSTORE + SLOTS - 1) / SLOTS;
  constexpr int LOADS_PER_SLOT = (NLOAD + SLOTS - 1) / SLOTS;

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

  // LDS byte offsets of this lane's operand rows; the chunk of sub-step s sits in slot
  // (2s + lgrp) ^ swz(row).
  uint32_t arow[MT], brow[NT], asw[MT], bsw[NT];
#pragma unroll
  for (int i = 0; i < MT; i++) {
    const uint32_t r = wm + i * 32 + lrow;
    arow[i] = r * 128;
    asw[i] = swz(r);
  }
#pragma unroll
  for (int j = 0; j < NT; j++) {
    const uint32_t r = wn + j * 32 + lrow;
    brow[j] = BM * 128 + r * 128;
    bsw[j] = swz(r);
  }
  // one operand read: index q < NT is B tile q, otherwise A tile q - NT
  auto read_one = [&](Frags<MT, NT>& f, const char* stage, int s, int q) {
    const uint32_t c = 2 * s + lgrp;
    if (q < NT)
      f.b[q] = *reinterpret_cast<const Chunk*>(stage + brow[q] + ((c ^ bsw[q]) * 16));
    else
      f.a[q - NT] = *reinterpret_cast<const Chunk*>(stage + arow[q - NT] + ((c ^ asw[q - NT]) * 16));
  };
  // MFMA number t of a sub-step. Operands swapped (B chunk first) so that a lane ends up
  // with four consecutive n for one m (see the epilogue).
  auto mma_one = [&](const Frags<MT, NT>& f, int t) {
    const int i = t / NT, j = t % NT;
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, f.b[j]),
                                                       __builtin_bit_cast(half8, f.a[i]), acc[i][j], 0, 0, 0);
  };

  OpA oa;
  OpB ob;
  oa.init(A, p.a_rs, p.a_cs, m0);
  ob.init(B, p.b_cs, p.b_rs, n0);
  auto load_unit = [&](int u, uint32_t k0) {
    if (u < OpA::N) oa.load(u, k0);
    else if (u < NLOAD) ob.load(u - OpA::N, k0);
  };
  auto store_unit = [&](int u, char* stage) {
    if (u < OpA::STORES) oa.store(u, stage);
    else if (u < NSTORE) ob.store(u - OpA::STORES, stage + BM * 128);
  };

  const uint32_t nk = p.K / 64;
  // prologue: K-step 0 into stage 0, K-step 1 into the registers
#pragma unroll
  for (int u = 0; u < NLOAD; u++) load_unit(u, 0);
#pragma unroll
  for (int u = 0; u < NSTORE; u++) store_unit(u, lds);
  {
    const uint32_t k1 = nk > 1 ? 64 : 0;
#pragma unroll
    for (int u = 0; u < NLOAD; u++) load_unit(u, k1);
  }
  lds_barrier();
  Frags<MT, NT> f0, f1;
#pragma unroll
  for (int q = 0; q < READS; q++) read_one(f0, lds, 0, q);

  // Steady state of step ks: the registers hold the global data of step ks+1 and f0 the
  // first sub-step's operands. LDS stage `nxt` was last read in step ks-1, before the
  // barrier every wave passed in that step's last sub-step, so it may be overwritten now.
  // The body is branch-free (the last steps re-load the final K-slice and store it to a
  // stage nobody reads).
  for (uint32_t ks = 0; ks < nk; ks++) {
    const char* cur = lds + (ks & 1) * STAGE_BYTES;
    char* nxt = lds + ((ks + 1) & 1) * STAGE_BYTES;
    const uint32_t k2 = (ks + 2 < nk ? ks + 2 : nk - 1) * 64;
    __builtin_amdgcn_sched_barrier(0);
    // sub-step 0: MFMAs on f0; operands of sub-step 1; registers -> LDS stage nxt
#pragma unroll
    for (int t = 0; t < SLOTS; t++) {
      if (t < READS) read_one(f1, cur, 1, t);
      mma_one(f0, t);
#pragma unroll
      for (int e = 0; e < STORES_PER_SLOT; e++) store_unit(t * STORES_PER_SLOT + e, nxt);
      __builtin_amdgcn_sched_barrier(0);
    }
    // sub-step 1: MFMAs on f1; operands of sub-step 2; global loads of step ks+2
#pragma unroll
    for (int t = 0; t < SLOTS; t++) {
      if (t < READS) read_one(f0, cur, 2, t);
      mma_one(f1, t);
#pragma unroll
      for (int e = 0; e < LOADS_PER_SLOT; e++) load_unit(t * LOADS_PER_SLOT + e, k2);
      __builtin_amdgcn_sched_barrier(0);
    }
    // sub-step 2: MFMAs on f0; operands of sub-step 3
#pragma unroll
    for (int t = 0; t < SLOTS; t++) {
      if (t < READS) read_one(f1, cur, 3, t);
      mma_one(f0, t);
      __builtin_amdgcn_sched_barrier(0);
    }
    // sub-step 3: half of the MFMAs, then the step's only barrier (every read of `cur` by
    // this wave has been issued and is waited for by the barrier's LDS fence), then the
    // next step's first operands from `nxt` under cover of the other half.
#pragma unroll
    for (int t = 0; t < SLOTS / 2; t++) mma_one(f1, t);
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = SLOTS / 2; t < SLOTS; t++) {
      if (t - SLOTS / 2 < READS) read_one(f0, nxt, 0, t - SLOTS / 2);
      if (SLOTS / 2 < READS && t == SLOTS - 1) {
#pragma unroll
        for (int q = SLOTS / 2; q < READS; q++) read_one(f0, nxt, 0, q);
      }
      mma_one(f1, t);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // Epilogue. With the operands swapped, the MFMA tile is C^T: lane l holds m = l % 32 and,
  // in registers 4g..4g+3, the four consecutive columns n = 8g + 4*(l/32) + (0..3).
  // Four halfs = one 8-byte store; c_cs == 1 (row-major output).
#pragma unroll
  for (int i = 0; i < MT; i++) {
    const uint32_t row = m0 + wm + i * 32 + lrow;
#pragma unroll
    for (int j = 0; j < NT; j++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        typedef _Float16 half4v __attribute__((ext_vector_type(4)));
        half4v h;
#pragma unroll
        for (int e = 0; e < 4; e++) h[e] = narrow<half_t>(acc[i][j][4 * g + e]);
        const uint32_t col = n0 + wn + j * 32 + 8 * g + 4 * lgrp;
        *reinterpret_cast<half4v*>(C + (size_t)row * p.c_rs + col) = h;
      }
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
