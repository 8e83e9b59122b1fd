// fp16 and fp32 GEMM for gfx950 with direct global->LDS loads (buffer_load_dwordx4 ... lds) and,
// for fp16 operands that are contiguous along M/N, transposing LDS reads
// (ds_read_b64_tr_b16). Block tile BM x BN, 4 waves 2 x 2, fp32 accumulate with
// v_mfma_f32_32x32x16_f16 / v_mfma_f32_32x32x2_f32, whole tiles only. No operand passes
// through VGPRs on its way to LDS: that removes the register->LDS stores, which cost about
// 20 % of the MFMA rate when issued from the same waves.
//
// LDS: a ring of four stages, each one K-slice of 64 bytes (32 halfs, 16 floats):
// [A region: BM*64 bytes][B region: BN*64 bytes].
//   K-contiguous operand (A of NN/NT, B of NT/TT): rows of 64 bytes = four 16-byte slots,
//     chunk c of row r in slot c ^ f(r), f(r) = ((r>>1)&3) ^ ((r>>3)&1); MFMA operand = one
//     ds_read_b128. For fp32 the four floats of a chunk feed four consecutive MFMAs; lanes
//     0..31 take chunk 2s and lanes 32..63 chunk 2s+1 in sub-step s, a permutation of k that
//     both operands share.
//   M/N-contiguous fp16 operand (A of TN/TT, B of NN/TN): natural [k][m] layout, 32 k-rows of
//     ROWS halfs, 16-byte slot x of k-row k stored at slot x ^ g(k),
//     g(k) = ((k&7) ^ ((k>>3&1)<<2)) << 1. MFMA operand = two ds_read_b64_tr_b16: in a group
//     of 16 lanes, lane r points at k-row k0 + r/4, columns 4*(r%4)..+3 (8 bytes); the
//     instruction returns to lane i the four k-values of column i. Two reads (k0, k0+4) give
//     a lane its 8 consecutive k for one m, in the same order as the K-contiguous operand.
//   M/N-contiguous fp32 operand: [16 k][ROWS floats], MFMA operands are single ds_read_b32
//     (32 consecutive floats of k-row k for lanes 0..31, of k-row k+4 for lanes 32..63).
// A wave-level DMA instruction fills 1 KiB of LDS in lane order (lane l -> byte 16*l), so
// any permutation of 16-byte pieces inside a 1 KiB block is free: the lane simply fetches
// the global piece that belongs in its slot. Both swizzles stay inside such blocks.
//
// Pipeline. The texture-address path of a CU accepts one 1 KiB DMA instruction per 16
// cycles, i.e. a K-slice of 32 for a 256 x 256 tile keeps it busy for 512 of the 1024 cycles
// its MFMAs take: DMA instructions issued in a burst stall the issuing waves (and their
// MFMAs) behind that queue, so they are spread evenly, one every few MFMAs. That needs a
// target stage that is free during the whole K-step, hence four stages: K-step j computes
// out of stage j%4 in two sub-steps (half a stage each),
//   sub-step 0: MFMAs on operands read earlier; read the operands of sub-step 1; issue the
//               second half of the DMA of K-step j+3 into stage (j-1)%4
//   wait until this wave's DMA of K-step j+1 has landed (vmcnt = DMA instructions issued
//               since), one LDS barrier: stage j%4 is now free, stage (j+1)%4 visible
//   sub-step 1: MFMAs; read the first operands of K-step j+1; issue the first half of the
//               DMA of K-step j+4 into stage j%4.
// The stages are distinct __shared__ arrays and the loop is unrolled by four so that every
// LDS access names its stage statically.
#include "common.hip.h"
#include <type_traits>

#ifndef HC_READS_PER_SLOT
#define HC_READS_PER_SLOT 0
#endif

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t Chunk __attribute__((ext_vector_type(4)));  // 16 bytes = 8 halfs

enum { DMA_K = 0, DMA_MN = 1 };

#define LDS_AS __attribute__((address_space(3)))

__device__ __forceinline__ uint32_t swz_k(uint32_t row) { return ((row >> 1) & 3u) ^ ((row >> 3) & 1u); }
__device__ __forceinline__ uint32_t swz_mn(uint32_t k) { return (((k & 7u) ^ (((k >> 3) & 1u) << 2)) << 1); }

// Workgroup barrier for LDS traffic only: this wave's LDS reads have returned (lgkmcnt), its
// DMA is waited for separately (wait_dma), and nothing is said about global memory. A fence
// builtin would do the same but also waits for every DMA instruction in flight, including
// those that fill stages nobody is about to read. The "memory" clobber keeps the compiler
// from moving LDS accesses across it.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// s_waitcnt vmcnt(N) with the other counters untouched (gfx9 encoding: vmcnt in bits 3:0 and
// 15:14, expcnt 6:4, lgkmcnt 11:8): at most N of this wave's DMA instructions still in flight.
template <int N> __device__ __forceinline__ void wait_dma() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// One operand of the block tile: where its DMA lanes fetch from and where a wave's MFMA
// operand reads land.
template <typename T, int ROWS, int MODE> struct DmaOperand {
  static constexpr int ES = sizeof(T);
  static constexpr bool F32 = ES == 4;
  static constexpr int NI = ROWS / 64;                        // DMA instructions per wave and K-step
  static constexpr int TILES = ROWS / 64;                     // MFMA tiles per wave along this operand
  // LDS reads per sub-step
  static constexpr int READS = MODE == DMA_K ? TILES : (F32 ? 4 * TILES : 2 * TILES);
  static constexpr int NADDR = TILES * 2;
  static constexpr int ROWB = ROWS * ES;                      // bytes per k-row (DMA_MN layout)
  static constexpr int BYTES = ROWS * 64;                     // per stage

  uint32_t goff[NI];     // byte offset of this lane's 16-byte piece for DMA instruction i (k = 0)
  uint32_t kstride;      // bytes per unit of k
  uint32_t raddr[NADDR]; // byte offsets (inside the operand's LDS region) of the MFMA operand reads

  // `limit` (edge kernels): extent of this operand along M / N. Rows or 16-byte pieces past it
  // are fetched from the last valid row / piece instead: they only feed outputs that are
  // never stored. 0 = no clamping.
  __device__ __forceinline__ void init(uint32_t rs, uint32_t cs, uint32_t r0, uint32_t woff, uint32_t limit) {
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (MODE == DMA_K) {
      kstride = ES;
#pragma unroll
      for (int i = 0; i < NI; i++) {
        const uint32_t row = (wave * NI + i) * 16 + lane / 4;
        const uint32_t c = (lane % 4) ^ swz_k(row);
        uint32_t grow = r0 + row;
        if (limit && grow >= limit) grow = limit - 1;
        goff[i] = grow * rs * ES + c * 16;
      }
      const uint32_t lrow = lane & 31, lgrp = lane >> 5;
#pragma unroll
      for (int q = 0; q < TILES; q++) {
        const uint32_t r = woff + q * 32 + lrow;
#pragma unroll
        for (int s = 0; s < 2; s++) raddr[q * 2 + s] = r * 64 + (((2 * s + lgrp) ^ swz_k(r)) * 16);
      }
    } else if (F32) {
      // [16 k][ROWS floats]; the 128-byte halves of every 256 bytes swap places in k-rows
      // with bit 2 set: an MFMA operand read touches rows k and k + 4, 32 floats of each
      constexpr uint32_t KPI = 1024 / ROWB;   // k-rows per DMA instruction
      constexpr uint32_t PIECES = ROWB / 16;  // 16-byte pieces per k-row
      kstride = cs * ES;
#pragma unroll
      for (int i = 0; i < NI; i++) {
        const uint32_t krow = (wave * NI + i) * KPI + lane / PIECES;
        const uint32_t piece = (lane % PIECES) ^ (((krow >> 2) & 1u) << 3);
        uint32_t col = r0 + piece * 4;
        if (limit && col + 4 > limit) col = limit - 4;
        goff[i] = (krow * cs + col) * ES;
      }
      const uint32_t lrow = lane & 31, lgrp = lane >> 5;
#pragma unroll
      for (int q = 0; q < TILES; q++) {
        const uint32_t n = woff + q * 32 + lrow;  // k = 4 * lgrp + e + 8 * s, e and s as immediates
        raddr[q] = 4 * lgrp * ROWB + ((n ^ (lgrp << 5)) * 4);
      }
    } else {
      constexpr int KPI = 512 / ROWS;       // k-rows per DMA instruction
      constexpr uint32_t SLOTS_PER_ROW = ROWS / 8;
      kstride = cs * 2;
#pragma unroll
      for (int i = 0; i < NI; i++) {
        const uint32_t krow = (wave * NI + i) * KPI + lane / SLOTS_PER_ROW;
        const uint32_t slot = (lane % SLOTS_PER_ROW) ^ (swz_mn(krow) & (SLOTS_PER_ROW - 1));
        uint32_t col = r0 + slot * 8;
        if (limit && col + 8 > limit) col = limit - 8;
        goff[i] = (krow * cs + col) * 2;
      }
      const uint32_t j = lane >> 4, r16 = lane & 15;
#pragma unroll
      for (int q = 0; q < TILES; q++) {
        const uint32_t m = woff + q * 32 + 16 * (j & 1) + 4 * (r16 & 3);
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const uint32_t k = 8 * (j >> 1) + 4 * h + (r16 >> 2);  // + 16 * s as an immediate offset
          raddr[q * 2 + h] = k * ROWB + (((m >> 3) ^ (swz_mn(k) & (ROWS / 8 - 1))) * 16) + (m & 7) * 2;
        }
      }
    }
  }

  // k offset, inside a K-slice, of the piece this lane fetches with DMA instruction i
  __device__ __forceinline__ uint32_t klocal(int i) const {
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (MODE == DMA_K) {
      const uint32_t row = (wave * NI + i) * 16 + lane / 4;
      return ((lane % 4) ^ swz_k(row)) * (16 / ES);
    }
    constexpr uint32_t PER_ROW = ROWB / 16, KPI = 1024 / ROWB;
    return (wave * NI + i) * KPI + lane / PER_ROW;
  }

  // DMA instruction i of this wave for the K-slice starting at k0: 1 KiB into `region`.
  // A buffer load: the descriptor (base of the operand, no stride, range 2^32 - 16 bytes) lives
  // in scalar registers, the lane offset goes in as it is and the K offset as the scalar
  // offset, so no vector or scalar address arithmetic stands in front of the load. The host
  // keeps operands of this kernel below 4 GiB.
  // Edge kernels (kend != 0): lanes whose piece lies at k >= kend pass an offset beyond the
  // descriptor's range, which reads as zero, so the ragged last slice contributes nothing.
  __device__ __forceinline__ void dma(int i, const T* base, uint32_t k0, char* region, uint32_t kend = 0) const {
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0xfffffff0u, 0x00020000);
    uint32_t off = goff[i];
    if (kend != 0 && k0 + 64 / ES > kend) {  // wave-uniform
      if (k0 + klocal(i) >= kend) off = 0xfffffff0u;
    }
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (LDS_AS void*)(region + (wave * NI + i) * 1024), 16, off,
                                             k0 * kstride, 0, 0);
  }

  // Edge kernels: clears what the piece straddling `kend` holds beyond it (gemm_zero_piece_tail),
  // after this wave's DMA of the K-slice starting at k0 has landed in `region`.
  __device__ __forceinline__ void zero_k_tail(char* region, uint32_t k0, uint32_t kend) const {
    if (MODE != DMA_K) return;
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
    for (int i = 0; i < NI; i++)
      gemm_zero_piece_tail<T>(region + (wave * NI + i) * 1024 + lane * 16, k0 + klocal(i), kend);
  }

  // Read number u of sub-step s into the operand registers of tile u (DMA_K), half u%2 of
  // tile u/2 (DMA_MN, fp16) or element u%4 of tile u/4 (DMA_MN, fp32).
  __device__ __forceinline__ void read(int u, int s, const char* region, Chunk* frag) const {
    if (MODE == DMA_K) {
      frag[u] = *reinterpret_cast<const Chunk*>(region + raddr[u * 2 + s]);
    } else if (F32) {
      const int q = u / 4, e = u % 4;
      frag[q][e] = *reinterpret_cast<const uint32_t*>(region + raddr[q] + (8 * s + e) * ROWB);
    } else {
      const int q = u / 2, h = u % 2;
      typedef short short4v __attribute__((ext_vector_type(4)));
      const short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (LDS_AS short4v*)(region + raddr[q * 2 + h] + s * 16 * ROWB));
      typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
      const u32x2 w = __builtin_bit_cast(u32x2, v);
      frag[q][2 * h] = w[0];
      frag[q][2 * h + 1] = w[1];
    }
  }
};

template <typename T, int BM, int BN, int MODE_A, int MODE_B, bool EDGE>
__device__ __forceinline__ void gemm_dma_impl(const hck_gemm_args& p, char* lds0, char* lds1, char* lds2, char* lds3) {
  constexpr int MT = BM / 64, NT = BN / 64;
  constexpr int SLOTS = MT * NT;
  typedef DmaOperand<T, BM, MODE_A> OpA;
  typedef DmaOperand<T, BN, MODE_B> OpB;
  constexpr bool F32 = sizeof(T) == 4;
  constexpr uint32_t BK = 64 / sizeof(T);  // K-slice of one stage
  constexpr int READS = OpA::READS + OpB::READS;
  constexpr int NDMA = OpA::NI + OpB::NI;  // per wave and K-step
  constexpr int HALF = NDMA / 2;
  constexpr int A_BYTES = OpA::BYTES;

  uint32_t tm, tn;
  uint32_t block_in_product, batch_of_block;
  gemm_block_and_batch(block_in_product, batch_of_block);
  gemm_tile_of_block(p, block_in_product, tm, tn);
  const uint32_t m0 = tm * BM, n0 = tn * BN;
  const uint32_t batch = batch_of_block;
#ifdef HC_GEMM_MERGED
  // (the second build of this file, kernels *_m: what a recording's rewrite needs)
  uint32_t batch_hi = batch, batch_lo = 0;
  if (p.bdiv != 0) {
    batch_hi = batch / p.bdiv;
    batch_lo = batch - batch_hi * p.bdiv;
  }
  const T* A = (const T*)p.a + batch_hi * p.a_bs + batch_lo * p.a_bs2;
  const T* B = (const T*)p.b + batch_hi * p.b_bs + batch_lo * p.b_bs2;
  T* C = (T*)p.c + batch_hi * p.c_bs + batch_lo * p.c_bs2;
  if (p.group != 0) {  // a member of a group of products over the same A
    A = (const T*)p.a;
    B = (const T*)gemm_table_entry(p.g_b, batch);
    C = (T*)gemm_table_entry(p.g_c, batch);
  }
  const void* const ep_p0 = gemm_epilogue_operand(p, 0, batch);
  const void* const ep_p1 = gemm_epilogue_operand(p, 1, batch);
  const void* const ep_p2 = gemm_epilogue_operand(p, 2, batch);
#else
  const T* A = (const T*)p.a + batch * p.a_bs;
  const T* B = (const T*)p.b + batch * p.b_bs;
  T* C = (T*)p.c + batch * p.c_bs;
#endif

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

  OpA oa;
  OpB ob;
  oa.init(p.a_rs, p.a_cs, m0, wm, EDGE ? p.a_lim : 0);
  ob.init(p.b_cs, p.b_rs, n0, wn, EDGE ? p.b_lim : 0);
  const uint32_t kend = EDGE ? p.K : 0;

  struct Frags {
    Chunk a[MT];
    Chunk b[NT];
  };
  // unit u of the operand reads of a sub-step: B's reads first, then A's
  auto read_unit = [&](Frags& f, const char* stage, int s, int u) {
    if (u < OpB::READS) ob.read(u, s, stage + A_BYTES, f.b);
    else if (u < READS) oa.read(u - OpB::READS, s, stage, f.a);
  };
  // unit u of the DMA of the K-slice starting at k0
  // `tail`: a compile-time flag. Only the last K-slice can be ragged, so only the DMA that may
  // fetch it carries the range check of the edge kernels (a scalar compare and a branch in
  // front of every DMA instruction otherwise, in the middle of the MFMA stream).
  auto dma_unit = [&](auto tail, int u, uint32_t k0, char* stage) {
    const uint32_t ke = decltype(tail)::value ? kend : 0;
    if (u < OpA::NI) oa.dma(u, A, k0, stage, ke);
    else if (u < NDMA) ob.dma(u - OpA::NI, B, k0, stage + A_BYTES, ke);
  };
  typedef std::integral_constant<bool, EDGE> Tail;     // checks where the kernel has them at all
  typedef std::integral_constant<bool, false> NoTail;
  // MFMA t of a sub-step; operands swapped (B first) so that a lane holds four consecutive
  // n for one m (see the epilogue).
  auto mma_one = [&](const Frags& f, int t) {
    const int i = t / NT, j = t % NT;
    if constexpr (F32) {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        // (copies first: a bit_cast applied directly to a vector element reads element 0)
        const uint32_t wb = f.b[j][e], wa = f.a[i][e];
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, wb),
                                                         __builtin_bit_cast(float, wa), acc[i][j], 0, 0, 0);
      }
    } else {
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, f.b[j]),
                                                         __builtin_bit_cast(half8, f.a[i]), acc[i][j], 0, 0, 0);
    }
  };
  // reads per MFMA slot
  constexpr int RPS = HC_READS_PER_SLOT ? HC_READS_PER_SLOT : (READS + SLOTS - 1) / SLOTS;
  // one DMA instruction every DSTRIDE MFMAs
  constexpr int DSTRIDE = SLOTS / (NDMA - HALF) > 0 ? SLOTS / (NDMA - HALF) : 1;
  static_assert(DSTRIDE * (NDMA - HALF) <= SLOTS, "more DMA instructions than MFMA slots");

  const uint32_t nk = (p.K + BK - 1) / BK;
  // (edge kernels) K is not a whole number of 16-byte pieces: the last slice of a K-contiguous
  // operand is cleaned up after it has landed
  const bool ktail = EDGE && p.K % (16 / sizeof(T)) != 0;
  auto zero_tail = [&](char* stage, uint32_t k0) {
    oa.zero_k_tail(stage, k0, kend);
    ob.zero_k_tail(stage + A_BYTES, k0, kend);
  };
  Frags f0, f1;

  // K-step j out of `cur`; `nxt` holds K-step j+1, `prev` held K-step j-1.
  auto step = [&](auto tail, char* cur, char* nxt, char* prev, uint32_t j) {
    const uint32_t k3 = (j + 3 < nk ? j + 3 : nk - 1) * BK, k4 = (j + 4 < nk ? j + 4 : nk - 1) * BK;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < SLOTS; t++) {  // sub-step 0
      if (t % DSTRIDE == 0 && HALF + t / DSTRIDE < NDMA) dma_unit(tail, HALF + t / DSTRIDE, k3, prev);
#pragma unroll
      for (int e = 0; e < RPS; e++) read_unit(f1, cur, 1, t * RPS + e);
      mma_one(f0, t);
      __builtin_amdgcn_sched_barrier(0);
    }
    wait_dma<2 * NDMA>();  // K-step j+1 of this wave has landed ...
    if constexpr (decltype(tail)::value) {
      if (ktail && j + 2 == nk) zero_tail(nxt, (j + 1) * BK);
    }
    lds_barrier();         // ... and everybody's; nobody reads cur any more
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < SLOTS; t++) {  // sub-step 1
      if (t % DSTRIDE == 0 && t / DSTRIDE < HALF) dma_unit(tail, t / DSTRIDE, k4, cur);
#pragma unroll
      for (int e = 0; e < RPS; e++) read_unit(f0, nxt, 0, t * RPS + e);
      mma_one(f1, t);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // prologue: K-steps 0..2 and the first half of K-step 3 (slices past the end repeat the
  // last one; nobody reads them)
  auto kclamp = [&](uint32_t j) { return (j < nk ? j : nk - 1) * BK; };
#pragma unroll
  for (int u = 0; u < NDMA; u++) dma_unit(Tail{}, u, 0, lds0);
#pragma unroll
  for (int u = 0; u < NDMA; u++) dma_unit(Tail{}, u, kclamp(1), lds1);
#pragma unroll
  for (int u = 0; u < NDMA; u++) dma_unit(Tail{}, u, kclamp(2), lds2);
#pragma unroll
  for (int u = 0; u < HALF; u++) dma_unit(Tail{}, u, kclamp(3), lds3);
  wait_dma<2 * NDMA + HALF>();
  if constexpr (EDGE) {
    if (ktail && nk == 1) zero_tail(lds0, 0);
  }
  lds_barrier();
#pragma unroll
  for (int u = 0; u < READS; u++) read_unit(f0, lds0, 0, u);

  uint32_t j = 0;
  if constexpr (EDGE) {  // K-step j fetches slices j+3 and j+4: up to j = nk-6 the last slice is not among them
    for (; j + 9 <= nk; j += 4) {
      step(NoTail{}, lds0, lds1, lds3, j);
      step(NoTail{}, lds1, lds2, lds0, j + 1);
      step(NoTail{}, lds2, lds3, lds1, j + 2);
      step(NoTail{}, lds3, lds0, lds2, j + 3);
    }
  }
  for (; j + 3 < nk; j += 4) {
    step(Tail{}, lds0, lds1, lds3, j);
    step(Tail{}, lds1, lds2, lds0, j + 1);
    step(Tail{}, lds2, lds3, lds1, j + 2);
    step(Tail{}, lds3, lds0, lds2, j + 3);
  }
  if (j < nk) step(Tail{}, lds0, lds1, lds3, j);
  if (j + 1 < nk) step(Tail{}, lds1, lds2, lds0, j + 1);
  if (j + 2 < nk) step(Tail{}, lds2, lds3, lds1, j + 2);
  wait_dma<0>();  // no LDS write of this workgroup may be in flight when it ends

  // Epilogue. With the operands swapped, the MFMA tile is C^T: lane l holds m = l % 32 and,
  // in registers 4g..4g+3, the four consecutive columns n = 8g + 4*(l/32) + (0..3). Stored
  // directly that would be short pieces of 32 different rows per instruction, so the wave's
  // part of C goes through LDS in slabs of 32 rows (every stage is free now; wave w uses
  // stage w) and leaves as 16-byte pieces, whole rows of the slab contiguous. 16-byte unit u
  // of row r sits at unit u ^ s(r) to spread the column-wise writes over the banks. A wave's
  // LDS instructions execute in order, so a slab may be overwritten right after its reads.
  lds_barrier();
  char* mine = wave == 0 ? lds0 : wave == 1 ? lds1 : wave == 2 ? lds2 : lds3;
  constexpr uint32_t ES = sizeof(T), WN = BN / 2, RB = WN * ES, UNITS = RB / 16, RPI = 64 / UNITS;
  constexpr uint32_t SLAB = 32 * RB, NSLAB = (BM + BN) * 64 / SLAB;
  static_assert(NSLAB >= 1 && UNITS <= 64, "a slab must fit one stage");
  auto unit_swz = [&](uint32_t r) { return (RB >= 256 ? r : r * RB / 256) & (UNITS - 1); };
#ifdef HC_GEMM_MERGED
  // (operations merged into this product: the lane's columns are the same for all its pieces)
  const uint32_t ep_col = n0 + wn + (lane % UNITS) * (16 / ES);
  Chunk ep_r0 = Chunk{}, ep_r1 = Chunk{}, ep_r2 = Chunk{};
  if (p.ep_kind[0] != HCK_EP_NONE) {
    const bool ok = !EDGE || ep_col < p.N;
    ep_r0 = gemm_epilogue_row_piece<T, Chunk>(p.ep_kind[0], ep_p0, ep_col, ok);
    ep_r1 = gemm_epilogue_row_piece<T, Chunk>(p.ep_kind[1], ep_p1, ep_col, ok);
    ep_r2 = gemm_epilogue_row_piece<T, Chunk>(p.ep_kind[2], ep_p2, ep_col, ok);
  }
#endif
  // One copy of the write-out per kind of epilogue (MODE 0: plain stores; 1: merged additions; 2:
  // with a matrix operand; 3: additions and GELU). The plain one is all that the kernels of the
  // ordinary build contain; the kernels a recording's rewrite uses are a second build of this file
  // (HC_GEMM_MERGED, names ending in _m) that picks the mode per launch and also knows two-level
  // batches and groups of products. Kept apart on purpose: with the merged code in the same kernel
  // the plain fp16 4096^3 product ran 7 % slower (1216 against 1313 TFLOP/s on the same device, same
  // main loop instruction for instruction), and where the plain path shared blocks with code that
  // loads, the compiler guarded those loads' registers with waits that, at run time, wait for the
  // plain path's own stores (one in-order counter for loads and stores).
#ifdef HC_GEMM_MERGED
  auto write_out = [&](auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
#else
  {
    constexpr int MODE = 0;
#endif
#pragma unroll
    for (int i = 0; i < MT; i++) {
      char* slab = mine + (i % NSLAB) * SLAB;
#pragma unroll
      for (int j = 0; j < NT; j++) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
          if constexpr (F32) {
            floatx4 h;
#pragma unroll
            for (int e = 0; e < 4; e++) h[e] = acc[i][j][4 * g + e];
            *reinterpret_cast<floatx4*>(slab + lrow * RB + (((j * 8 + 2 * g + lgrp) ^ unit_swz(lrow)) * 16)) = h;
          } else {
            half4v h;
#pragma unroll
            for (int e = 0; e < 4; e++) h[e] = narrow<half_t>(acc[i][j][4 * g + e]);
            *reinterpret_cast<half4v*>(slab + lrow * RB + (((j * 4 + g) ^ unit_swz(lrow)) * 16) + lgrp * 8) = h;
          }
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // wave-private region: no barrier needed
      if constexpr (MODE == 0) {
#pragma unroll
        for (uint32_t it = 0; it < 32 / RPI; it++) {
          const uint32_t r = it * RPI + lane / UNITS, u = lane % UNITS;
          const Chunk v = *reinterpret_cast<const Chunk*>(slab + r * RB + ((u ^ unit_swz(r)) * 16));
          const uint32_t row = m0 + wm + i * 32 + r, col = n0 + wn + u * (16 / ES);
          gemm_store_piece<T, Chunk, EDGE, EDGE && !HC_GEMM_IS_MERGED>(C + (size_t)row * p.c_rs + col, row, col, p.M, p.N, v, slab + r * RB + ((u ^ unit_swz(r)) * 16));
        }
      }
#ifdef HC_GEMM_MERGED
      if constexpr (MODE != 0) {
        gemm_store_slab_merged_as<T, Chunk, EDGE, 32 / RPI, true, (MODE == 3 ? 1 : 4), MODE == 2, MODE == 3>(
            p, ep_p0, ep_p1, ep_p2, ep_r0, ep_r1, ep_r2, C,
            [=](uint32_t it) {
              const uint32_t r = it * RPI + lane / UNITS, u = lane % UNITS;
              return *reinterpret_cast<const Chunk*>(slab + r * RB + ((u ^ unit_swz(r)) * 16));
            },
            [=](uint32_t it) { return m0 + wm + i * 32 + it * RPI + lane / UNITS; }, [=](uint32_t) { return ep_col; });
      }
#endif
      asm volatile("" ::: "memory");
    }
#ifdef HC_GEMM_MERGED
  };
  const bool ep_matrix = p.ep_kind[0] == HCK_EP_ADD_MATRIX || p.ep_kind[1] == HCK_EP_ADD_MATRIX || p.ep_kind[2] == HCK_EP_ADD_MATRIX;
  const bool ep_gelu = p.ep_kind[0] == HCK_EP_GELU || p.ep_kind[1] == HCK_EP_GELU || p.ep_kind[2] == HCK_EP_GELU;
  if (p.ep_kind[0] == HCK_EP_NONE) write_out(std::integral_constant<int, 0>{});
  else if (ep_gelu) write_out(std::integral_constant<int, 3>{});
  else if (ep_matrix) write_out(std::integral_constant<int, 2>{});
  else write_out(std::integral_constant<int, 1>{});
#else
  }
#endif
}

// Two variants per kernel: whole tiles only, and "_e" (edge) for M, N that are not multiples of
// the tile and K that is not a multiple of the K-slice.
#ifdef HC_GEMM_MERGED
#define HC_GEMM_NAME(base) base##_m
#else
#define HC_GEMM_NAME(base) base
#endif
// (Every stage is a __shared__ array of its own on purpose: the compiler then knows that a DMA into
// one stage does not touch the stage a read comes from. As parts of one array it guards every LDS
// read with a wait for all DMA in flight, and the kernels run three times slower.)
#define DEF_DMA(T, TN, BM, BN, AN, AM, BNAME, BMODE)                                                  \
  extern "C" __global__ __launch_bounds__(256) void HC_GEMM_NAME(hc_gemm_##TN##_dma_##BM##x##BN##_##AN##BNAME)( \
      hck_gemm_args p) {                                                                              \
    __shared__ __attribute__((aligned(1024))) char lds0[(BM + BN) * 64];                              \
    __shared__ __attribute__((aligned(1024))) char lds1[(BM + BN) * 64];                              \
    __shared__ __attribute__((aligned(1024))) char lds2[(BM + BN) * 64];                              \
    __shared__ __attribute__((aligned(1024))) char lds3[(BM + BN) * 64];                              \
    gemm_dma_impl<T, BM, BN, AM, BMODE, false>(p, lds0, lds1, lds2, lds3);                            \
  }                                                                                                   \
  extern "C" __global__ __launch_bounds__(256) void HC_GEMM_NAME(hc_gemm_##TN##_dma_##BM##x##BN##_##AN##BNAME##_e)( \
      hck_gemm_args p) {                                                                              \
    __shared__ __attribute__((aligned(1024))) char lds0[(BM + BN) * 64];                              \
    __shared__ __attribute__((aligned(1024))) char lds1[(BM + BN) * 64];                              \
    __shared__ __attribute__((aligned(1024))) char lds2[(BM + BN) * 64];                              \
    __shared__ __attribute__((aligned(1024))) char lds3[(BM + BN) * 64];                              \
    gemm_dma_impl<T, BM, BN, AM, BMODE, true>(p, lds0, lds1, lds2, lds3);                             \
  }
#define DEF_DMA_TILE(T, TN, BM, BN)                                                                   \
  DEF_DMA(T, TN, BM, BN, k, DMA_K, k, DMA_K)                                                          \
  DEF_DMA(T, TN, BM, BN, k, DMA_K, n, DMA_MN)                                                         \
  DEF_DMA(T, TN, BM, BN, m, DMA_MN, k, DMA_K)                                                         \
  DEF_DMA(T, TN, BM, BN, m, DMA_MN, n, DMA_MN)
#define DEF_DMA_TYPE(T, TN)                                                                           \
  DEF_DMA_TILE(T, TN, 256, 256)                                                                       \
  DEF_DMA_TILE(T, TN, 256, 128)                                                                       \
  DEF_DMA_TILE(T, TN, 128, 128)                                                                       \
  DEF_DMA_TILE(T, TN, 256, 64)                                                                        \
  DEF_DMA_TILE(T, TN, 128, 64)                                                                        \
  DEF_DMA_TILE(T, TN, 64, 64)
DEF_DMA_TYPE(half_t, f16)
DEF_DMA_TYPE(float, f32)
