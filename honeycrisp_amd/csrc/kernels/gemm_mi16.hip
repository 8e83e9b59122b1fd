// fp16 GEMM for gfx950 on v_mfma_f32_16x16x32_f16, the power-efficient shape of the fp16 matrix
// instruction: per multiply-accumulate it moves half as many accumulator registers as the
// 32x32x16 shape, and on random operands a loop of nothing but these instructions sustains
// about 1.9 PFLOP/s against 1.7 for 32x32x16 (the board lowers its clock to stay within its
// power limit). Global->LDS traffic, LDS layouts and swizzles are those of the two-stage
// pipeline with 128-byte K-slices (gemm_dma2.hip: whole cache lines for K-contiguous operands,
// 16-byte loads straight into LDS, ds_read_b64_tr_b16 for M/N-contiguous operands); what differs
// is the form of the load (buffer_load_dwordx4 ... lds, see DmaOperand::dma) and how a wave reads
// its operands and lays out its accumulators:
//   wave tile (BM/2) x (BN/2) = MT x NT tiles of 16 x 16, one MFMA per tile and 32 k;
//   operand of a tile: lane l holds row l%16, k = 8*(l/16) .. +7 (one 16-byte chunk);
//   accumulator of a tile (operands swapped, so it is C^T): lane l holds m = l%16 and the four
//   consecutive columns n = 4*(l/16) .. +3.
// A K-step (one stage, 64 halfs) is two sub-steps of MT*NT MFMAs, with the barrier between them:
//   sub-step 0: MFMAs on k 0..31; read the operands of k 32..63; the rest of the DMA of K-step j+1
//   wait for this wave's DMA, barrier
//   sub-step 1: MFMAs on k 32..63; read the first operands of K-step j+1; DMA of K-step j+2 into
//     this stage, spread over the MFMAs.
#include <type_traits>

#include "common.hip.h"

// length of the DMA window in quarter sub-steps (see the K loop)
#ifndef HC_MI16_WINDOW_X4
#define HC_MI16_WINDOW_X4 5
#endif
// 1: the operand reads of a sub-step are spread over its MFMAs, 0: issued under the first ones
#ifndef HC_MI16_READ_SPREAD
#define HC_MI16_READ_SPREAD 0
#endif

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

typedef uint32_t Chunk __attribute__((ext_vector_type(4)));  // 16 bytes = 8 halfs

enum { DMA_K = 0, DMA_MN = 1 };

#define LDS_AS __attribute__((address_space(3)))

__device__ __forceinline__ uint32_t swz_k(uint32_t row) { return row & 7u; }
__device__ __forceinline__ uint32_t swz_mn(uint32_t k) { return (((k & 7u) ^ (((k >> 3) & 1u) << 2)) << 1); }

// Workgroup barrier for LDS traffic only: this wave's LDS reads have returned (lgkmcnt), its
// DMA is waited for separately (wait_dma), and nothing is said about global memory. A fence
// builtin would do the same but also waits for every DMA instruction in flight, including
// those that fill stages nobody is about to read. The "memory" clobber keeps the compiler
// from moving LDS accesses across it.
// (builtins, not an assembly statement: the compiler's wait-count pass then knows that no LDS read is
// outstanding behind the barrier and does not guard the first MFMAs of the next sub-step with waits
// of its own, each of which would take one of the three issue slots between two MFMAs. The empty
// assembly statements keep the compiler from moving memory accesses across the pair.)
__device__ __forceinline__ void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0); vmcnt and expcnt untouched
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
// s_waitcnt vmcnt(N) with the other counters untouched (gfx9 encoding: vmcnt in bits 3:0 and
// 15:14, expcnt 6:4, lgkmcnt 11:8): at most N of this wave's DMA instructions still in flight.
template <int N> __device__ __forceinline__ void wait_dma() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// DMA side of one operand of the block tile: which 16-byte piece of global memory each lane
// fetches and where it lands. ROWS (the tile's extent along M or N) is a multiple of 64.
//   DMA_K : LDS rows of 128 bytes (64 k of one row), chunk c of row r in slot c ^ (r & 7);
//           one instruction covers 8 rows.
//   DMA_MN: LDS [64 k-rows][ROWS halfs], 16-byte slot u of k-row k holds columns
//           8 (u ^ swz(k)) .. +7; the instructions of a K-slice cover its 8 ROWS pieces in
//           order, 64 each (a k-row need not be a whole number of instructions).
template <int ROWS, int MODE> struct DmaOperand {
  static constexpr int NI = ROWS / 32;           // DMA instructions per wave and K-step
  static constexpr int ROWB = ROWS * 2;          // bytes per k-row (DMA_MN layout)
  static constexpr int BYTES = ROWS * 128;       // per stage
  static constexpr uint32_t SLOTS = ROWS / 8;    // 16-byte slots per k-row (DMA_MN layout)
  // the swizzle permutes slots inside aligned groups of SWZ_MASK + 1 (a divisor of SLOTS)
  static constexpr uint32_t SWZ_MASK = (SLOTS & (SLOTS - 1)) == 0 ? SLOTS - 1 : 7;
  static_assert(ROWS % 64 == 0 && SLOTS % (SWZ_MASK + 1) == 0, "unsupported tile extent");

  // Four consecutive DMA instructions of a wave share one LDS base (the M0 register) and differ in the
  // instruction's immediate offset, which the hardware adds to the LDS address and to the memory
  // address alike: instruction i targets base + (i % 4) KiB. The lane offsets take the immediate out
  // again, and the buffer descriptor starts IMM_SPAN bytes in front of the operand so that they stay
  // non-negative. (One M0 write and its wait state per four loads instead of per load: between two
  // MFMAs a wave has three issue slots.)
  static constexpr uint32_t IMM_SPAN = 3 * 1024;
  // The descriptor's range, and the lane offset that reads as zero: lane offset + immediate is a 32-bit
  // sum, so the offset of a lane that must not fetch stays out of range with any immediate added.
  static constexpr uint32_t RANGE = 0xffffe000u;
  uint32_t goff[NI];     // byte offset of this lane's 16-byte piece for DMA instruction i (k = 0), see above
  uint32_t kstride;      // bytes per unit of k

  __device__ __forceinline__ static uint32_t mn_swz(uint32_t k) { return swz_mn(k) & SWZ_MASK; }

  // `limit` (edge kernels): extent of this operand along M / N. Rows or 16-byte pieces past it
  // are fetched from the last valid row / piece instead: they only feed outputs that are
  // never stored. 0 = no clamping.
  __device__ __forceinline__ void init(uint32_t rs, uint32_t cs, uint32_t r0, uint32_t limit) {
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (MODE == DMA_K) {
      kstride = 2;
#pragma unroll
      for (int i = 0; i < NI; i++) {
        const uint32_t row = (wave * NI + i) * 8 + lane / 8;
        const uint32_t c = (lane % 8) ^ swz_k(row);
        uint32_t grow = r0 + row;
        if (limit && grow >= limit) grow = limit - 1;
        goff[i] = grow * rs * 2 + c * 16 + IMM_SPAN - (i & 3) * 1024;
      }
    } else {
      kstride = cs * 2;
#pragma unroll
      for (int i = 0; i < NI; i++) {
        const uint32_t piece = (wave * NI + i) * 64 + lane;
        const uint32_t krow = piece / SLOTS;
        const uint32_t slot = (piece % SLOTS) ^ mn_swz(krow);
        uint32_t col = r0 + slot * 8;
        if (limit && col + 8 > limit) col = limit - 8;
        goff[i] = (krow * cs + col) * 2 + IMM_SPAN - (i & 3) * 1024;
      }
    }
  }

  // k offset, inside a K-slice, of the piece this lane fetches with DMA instruction i
  __device__ __forceinline__ uint32_t klocal(int i) const {
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (MODE == DMA_K) {
      const uint32_t row = (wave * NI + i) * 8 + lane / 8;
      return ((lane % 8) ^ swz_k(row)) * 8;
    }
    return ((wave * NI + i) * 64 + lane) / SLOTS;
  }

  // DMA instruction I of this wave for the K-slice starting at k0: 1 KiB into `region`.
  // A buffer load: the descriptor (base of the operand less IMM_SPAN, no stride, range RANGE
  // bytes) lives in scalar registers, the lane offset goes in as it is and the K offset as the scalar
  // offset, so no vector or scalar address arithmetic stands in front of the load. The host
  // keeps operands of this kernel 16 KiB below 4 GiB.
  // Edge kernels (kend != 0): lanes whose piece lies at k >= kend pass an offset beyond the
  // descriptor's range, which reads as zero, so the ragged last slice contributes nothing.
  template <int I> __device__ __forceinline__ void dma(const half_t* base, uint32_t k0, char* region, uint32_t kend = 0) const {
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)base - IMM_SPAN), 0, RANGE, 0x00020000);
    uint32_t off = goff[I];
    if (kend != 0 && k0 + 64 > kend) {  // wave-uniform
      if (k0 + klocal(I) >= kend) off = RANGE;
    }
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (LDS_AS void*)(region + (wave * NI + (I & ~3)) * 1024), 16, off,
                                             k0 * kstride, (I & 3) * 1024, 0);
  }

  // Edge kernels: clears what the piece straddling `kend` holds beyond it (gemm_zero_piece_tail),
  // after this wave's DMA of the K-slice starting at k0 has landed in `region`.
  __device__ __forceinline__ void zero_k_tail(char* region, uint32_t k0, uint32_t kend) const {
    if (MODE != DMA_K) return;
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
    for (int i = 0; i < NI; i++)
      gemm_zero_piece_tail<half_t>(region + (wave * NI + i) * 1024 + lane * 16, k0 + klocal(i), kend);
  }
};

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>)
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// Where a wave's operand reads land, for the 16 x 16 x 32 instruction. The DMA side (which
// global piece goes to which LDS slot) is DmaOperand's.
template <int ROWS, int MODE> struct Mi16Reads {
  static constexpr int TILES = ROWS / 32;  // 16-row tiles per wave along this operand
  static constexpr int READS = MODE == DMA_K ? TILES : 2 * TILES;  // LDS reads per sub-step
  static constexpr int ROWB = ROWS * 2;
  uint32_t raddr[TILES * 2];

  __device__ __forceinline__ void init(uint32_t woff) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t r16 = lane & 15, grp = lane >> 4;
    if (MODE == DMA_K) {
      // rows of 128 bytes, chunk c of row r in slot c ^ (r & 7); sub-step s reads chunk 4 s + grp
#pragma unroll
      for (int q = 0; q < TILES; q++) {
        const uint32_t r = woff + q * 16 + r16;
#pragma unroll
        for (int s = 0; s < 2; s++) raddr[q * 2 + s] = r * 128 + (((4 * s + grp) ^ swz_k(r)) * 16);
      }
    } else {
      // [k][m] layout; a transposing read hands lane i of a 16-lane group column i of four
      // k-rows: the group points at k-rows 8 grp + 4 h + (0..3), lane r16 at k-row + r16 / 4,
      // columns 4 (r16 % 4) .. +3. Sub-step s adds 32 k-rows as an immediate offset.
#pragma unroll
      for (int q = 0; q < TILES; q++) {
        const uint32_t m = woff + q * 16 + 4 * (r16 & 3);
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const uint32_t k = 8 * grp + 4 * h + (r16 >> 2);
          raddr[q * 2 + h] = k * ROWB + (((m >> 3) ^ DmaOperand<ROWS, MODE>::mn_swz(k)) * 16) + (m & 7) * 2;
        }
      }
    }
  }
  // read number u of sub-step s
  __device__ __forceinline__ void read(int u, int s, const char* region, Chunk* frag) const {
    if (MODE == DMA_K) {
      frag[u] = *reinterpret_cast<const Chunk*>(region + raddr[u * 2 + s]);
    } else {
      const int q = u / 2, h = u % 2;
      typedef short short4v __attribute__((ext_vector_type(4)));
      const short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (LDS_AS short4v*)(region + raddr[q * 2 + h] + s * 32 * ROWB));
      typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
      const u32x2 w = __builtin_bit_cast(u32x2, v);
      frag[q][2 * h] = w[0];
      frag[q][2 * h + 1] = w[1];
    }
  }
};

template <int BM, int BN, int MODE_A, int MODE_B, bool EDGE>
__device__ __forceinline__ void gemm_mi16_impl(const hck_gemm_args& p, char* lds0, char* lds1) {
  typedef half_t T;
  constexpr int MT = BM / 32, NT = BN / 32;  // 16 x 16 tiles per wave
  constexpr int SLOTS = MT * NT;             // MFMAs per sub-step
  typedef DmaOperand<BM, MODE_A> OpA;
  typedef DmaOperand<BN, MODE_B> OpB;
  typedef Mi16Reads<BM, MODE_A> RdA;
  typedef Mi16Reads<BN, MODE_B> RdB;
  constexpr uint32_t BK = 64;  // halfs per stage
  constexpr int READS = RdA::READS + RdB::READS;
  constexpr int NDMA = OpA::NI + OpB::NI;  // per wave and K-step
  constexpr int A_BYTES = OpA::BYTES;

  uint32_t tm, tn;
  gemm_tile_of_block(p, blockIdx.x, tm, tn);
  const uint32_t m0 = tm * BM, n0 = tn * BN;
  const uint32_t batch = blockIdx.y;
#ifdef HC_MI16_TIMESTAMPS
  // (measurement build: when a workgroup starts, leaves its K loop and ends, on the 100 MHz clock)
  const uint64_t ts_start = __builtin_amdgcn_s_memrealtime();
  const uint64_t tc_start = __builtin_amdgcn_s_memtime();
#endif
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

  floatx4 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
      for (int v = 0; v < 4; v++) acc[i][j][v] = 0.0f;

  OpA oa;
  OpB ob;
  oa.init(p.a_rs, p.a_cs, m0, EDGE ? p.a_lim : 0);
  ob.init(p.b_cs, p.b_rs, n0, EDGE ? p.b_lim : 0);
  RdA ra;
  RdB rb;
  ra.init(wm);
  rb.init(wn);
  const uint32_t kend = EDGE ? p.K : 0;

  struct Frags {
    Chunk a[MT];
    Chunk b[NT];
  };
  // unit u of the operand reads of a sub-step: B's reads first, then A's
  auto read_unit = [&](Frags& f, const char* stage, int s, int u) {
    if (u < RdB::READS) rb.read(u, s, stage + A_BYTES, f.b);
    else if (u < READS) ra.read(u - RdB::READS, s, stage, f.a);
  };
  // `tail`: a compile-time flag. Only the last K-slice can be ragged, so only the DMA that may
  // fetch it carries the range check of the edge kernels (a scalar compare and a branch in
  // front of every DMA instruction otherwise, in the middle of the MFMA stream).
  auto dma_unit = [&](auto tail, auto uc, uint32_t k0, char* stage) {
    constexpr int u = decltype(uc)::value;
    const uint32_t ke = decltype(tail)::value ? kend : 0;
    if constexpr (u < OpA::NI) oa.template dma<u>(A, k0, stage, ke);
    else if constexpr (u < NDMA) ob.template dma<u - OpA::NI>(B, k0, stage + A_BYTES, ke);
  };
  typedef std::integral_constant<bool, EDGE> Tail;     // checks where the kernel has them at all
  typedef std::integral_constant<bool, false> NoTail;
  // MFMA t of a sub-step; operands swapped (B first) so that a lane holds four consecutive n
  auto mma_one = [&](const Frags& f, int t) {
    const int j = t / MT, i = t % MT;
    // Written as assembly to pin the accumulators to the accumulation registers: left to itself
    // the register allocator keeps part of them in ordinary registers and copies them back and
    // forth around every instruction. An accumulator is touched again 63 MFMAs later at the
    // earliest and read by the epilogue only after a barrier, so no wait states are missing.
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(f.b[j]), "v"(f.a[i]));
  };
  // The DMA of a K-slice is spread evenly over a window of W MFMA slots that starts right after
  // the barrier that frees its stage (sub-step 1, then sub-step 0 of the next step): unit u
  // goes out in window slot u * W / NDMA; the rest of sub-step 0 is the time the last loads
  // get to land (needed: about 600 cycles = 40 MFMAs of this shape).
  constexpr int W = SLOTS * HC_MI16_WINDOW_X4 / 4 > 0 ? SLOTS * HC_MI16_WINDOW_X4 / 4 : 1;
  static_assert(W <= 2 * SLOTS, "the DMA window ends with sub-step 0");
  constexpr int U0 = (SLOTS * NDMA + W - 1) / W < NDMA ? (SLOTS * NDMA + W - 1) / W : NDMA;  // units of sub-step 1

  constexpr int RSTRIDE = HC_MI16_READ_SPREAD && SLOTS / READS > 1 ? SLOTS / READS : 1;

  const uint32_t nk = (p.K + BK - 1) / BK;
  auto kclamp = [&](uint32_t j) { return (j < nk ? j : nk - 1) * BK; };  // steps past the end repeat the last one
  // (edge kernels) K is not a whole number of 16-byte pieces: the last slice of a K-contiguous
  // operand is cleaned up after it has landed
  const bool ktail = EDGE && p.K % (16 / sizeof(half_t)) != 0;
  auto zero_tail = [&](char* stage, uint32_t k0) {
    oa.zero_k_tail(stage, k0, kend);
    ob.zero_k_tail(stage + A_BYTES, k0, kend);
  };
  Frags f0, f1;

  // (compile-time loop indices throughout: every register array is indexed statically)
  auto substep = [&](auto tail, const Frags& use, Frags& fill, const char* from, auto s_next_c, auto part_c,
                     char* to, uint32_t k0) {
    constexpr int s_next = decltype(s_next_c)::value, part = decltype(part_c)::value;
    static_for<SLOTS>([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      // units u with u * W / NDMA == this window slot
      constexpr int w = part * SLOTS + t;
      constexpr int lo = (w * NDMA + W - 1) / W < NDMA ? (w * NDMA + W - 1) / W : NDMA;
      constexpr int hi = ((w + 1) * NDMA + W - 1) / W < NDMA ? ((w + 1) * NDMA + W - 1) / W : NDMA;
      static_for<hi - lo>([&](auto uc) { dma_unit(tail, std::integral_constant<int, lo + decltype(uc)::value>{}, k0, to); });
      // operand reads of the following sub-step: one every RSTRIDE slots
      if constexpr (t % RSTRIDE == 0 && t / RSTRIDE < READS) read_unit(fill, from, s_next, t / RSTRIDE);
      mma_one(use, t);
      __builtin_amdgcn_sched_barrier(0);
    });
    static_for<(READS > SLOTS / RSTRIDE ? READS - SLOTS / RSTRIDE : 0)>(  // (tiles with more reads than slots)
        [&](auto uc) { read_unit(fill, from, s_next, SLOTS / RSTRIDE + decltype(uc)::value); });
  };

  // K-step j out of `cur`; `nxt` receives the rest of K-step j+1, then `cur` K-step j+2
  auto step = [&](auto tail, char* cur, char* nxt, uint32_t j) {
    __builtin_amdgcn_sched_barrier(0);
    substep(tail, f0, f1, cur, std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{}, nxt, kclamp(j + 1));
    wait_dma<0>();  // K-step j+1 of this wave has landed ...
    if constexpr (decltype(tail)::value) {
      if (ktail && j + 2 == nk) zero_tail(nxt, (j + 1) * BK);
    }
    lds_barrier();  // ... and everybody's; nobody reads cur any more
    __builtin_amdgcn_sched_barrier(0);
    substep(tail, f1, f0, nxt, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, cur, kclamp(j + 2));
  };

  // prologue: K-step 0 and the first window part of K-step 1
  static_for<NDMA>([&](auto uc) { dma_unit(Tail{}, uc, 0, lds0); });
  static_for<U0>([&](auto uc) { dma_unit(Tail{}, uc, kclamp(1), lds1); });
  // The accumulators are cleared here, while the first loads are on their way: left to the
  // compiler the 256 register writes sit after the barrier, in front of the first MFMA.
  __builtin_amdgcn_sched_barrier(0);
  // (a plain lambda: the assembly statement does not compile inside a generic one)
  auto pin_acc = [&](int t) { asm volatile("" : "+a"(acc[t % MT][t / MT])); };
  static_for<SLOTS>([&](auto tc) { pin_acc(decltype(tc)::value); });
  __builtin_amdgcn_sched_barrier(0);
  wait_dma<U0>();
  if constexpr (EDGE) {
    if (ktail && nk == 1) zero_tail(lds0, 0);
  }
  lds_barrier();
  static_for<READS>([&](auto uc) { read_unit(f0, lds0, 0, decltype(uc)::value); });

  uint32_t j = 0;
  if constexpr (EDGE) {  // K-step j fetches slices j+1 and j+2: up to j = nk-4 the last slice is not among them
    for (; j + 5 <= nk; j += 2) {
      step(NoTail{}, lds0, lds1, j);
      step(NoTail{}, lds1, lds0, j + 1);
    }
  }
  for (; j + 1 < nk; j += 2) {
    step(Tail{}, lds0, lds1, j);
    step(Tail{}, lds1, lds0, j + 1);
  }
  if (j < nk) step(Tail{}, lds0, lds1, j);
  wait_dma<0>();  // no LDS write of this workgroup may be in flight when it ends
#ifdef HC_MI16_TIMESTAMPS
  const uint64_t ts_loop = __builtin_amdgcn_s_memrealtime();
#endif
  // The compiler does not know that the assembly statements are MFMAs, so it would not keep the
  // epilogue's accumulator reads the required distance from the last of them: do it by hand.
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

  // Epilogue. Lane l of tile (i, j) holds m = l % 16 and the four consecutive columns
  // n = 4 * (l / 16) .. +3 (8 bytes of halfs). The wave's part of C goes through LDS in slabs
  // of 32 rows = two rows of tiles (both stages are free now; wave w uses half of a stage) and
  // leaves as 16-byte pieces, whole rows of the slab contiguous. 16-byte unit u of row r sits
  // at unit u ^ s(r) to spread the writes over the banks. A wave's LDS instructions execute in
  // order, so a slab may be overwritten right after its reads.
  lds_barrier();
  char* mine = (wave < 2 ? lds0 : lds1) + (wave & 1) * ((BM + BN) * 64);
  constexpr uint32_t WN = BN / 2, RB = WN * 2, UNITS = RB / 16;
  constexpr uint32_t SLAB = 32 * RB, NSLAB = (BM + BN) * 64 / SLAB;
  static_assert(NSLAB >= 1 && (32 * UNITS) % 64 == 0 && MT % 2 == 0, "a slab is two rows of tiles and must fit half a stage");
  // (the swizzle stays inside aligned groups of USWZ + 1 units, a divisor of UNITS)
  constexpr uint32_t USWZ = (UNITS & (UNITS - 1)) == 0 ? UNITS - 1 : 3;
  static_assert(UNITS % (USWZ + 1) == 0, "unsupported tile width");
  auto unit_swz = [&](uint32_t r) { return (RB >= 256 ? r : r * RB / 256) & USWZ; };
#ifdef HC_GEMM_MERGED
  // (operations merged into this product: if 64 lanes are whole rows of units, a lane's columns
  // are the same for all its pieces and the row operands are fetched once)
  constexpr bool EP_COL_FIXED = 64 % UNITS == 0;
  const uint32_t ep_col = n0 + wn + (lane % UNITS) * 8;
  Chunk ep_r0 = Chunk{}, ep_r1 = Chunk{}, ep_r2 = Chunk{};
  if (EP_COL_FIXED && p.ep_kind[0] != HCK_EP_NONE) {
    const bool ok = !EDGE || ep_col < p.N;
    ep_r0 = gemm_epilogue_row_piece<T, Chunk>(p.ep_kind[0], ep_p0, ep_col, ok);
    ep_r1 = gemm_epilogue_row_piece<T, Chunk>(p.ep_kind[1], ep_p1, ep_col, ok);
    ep_r2 = gemm_epilogue_row_piece<T, Chunk>(p.ep_kind[2], ep_p2, ep_col, ok);
  }
#endif
  const uint32_t r16 = lane & 15, grp = lane >> 4;
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
    for (int ii = 0; ii < MT / 2; ii++) {
      char* slab = mine + (ii % NSLAB) * SLAB;
#pragma unroll
      for (int half = 0; half < 2; half++) {
        const uint32_t row = half * 16 + r16;
#pragma unroll
        for (int jj = 0; jj < NT; jj++) {
          half4v h;
#pragma unroll
          for (int e = 0; e < 4; e++) h[e] = narrow<half_t>(acc[2 * ii + half][jj][e]);
          // columns jj * 16 + 4 grp .. +3: unit 2 jj + grp / 2, second half of the unit if grp is odd
          *reinterpret_cast<half4v*>(slab + row * RB + (((2 * jj + (grp >> 1)) ^ unit_swz(row)) * 16) + (grp & 1) * 8) = h;
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // wave-private region: no barrier needed
      if constexpr (MODE == 0) {
#pragma unroll
        for (uint32_t it = 0; it < 32 * UNITS / 64; it++) {
          const uint32_t piece = it * 64 + lane, r = piece / UNITS, u = piece % UNITS;
          const Chunk v = *reinterpret_cast<const Chunk*>(slab + r * RB + ((u ^ unit_swz(r)) * 16));
          const uint32_t row = m0 + wm + ii * 32 + r, col = n0 + wn + u * 8;
          gemm_store_piece<half_t, Chunk, EDGE, EDGE && !HC_GEMM_IS_MERGED>(C + (size_t)row * p.c_rs + col, row, col, p.M, p.N, v, slab + r * RB + ((u ^ unit_swz(r)) * 16));
        }
      }
#ifdef HC_GEMM_MERGED
      if constexpr (MODE != 0) {
        gemm_store_slab_merged_as<T, Chunk, EDGE, 32 * UNITS / 64, EP_COL_FIXED, (MODE == 3 ? 1 : 2), MODE == 2, MODE == 3>(
            p, ep_p0, ep_p1, ep_p2, ep_r0, ep_r1, ep_r2, C,
            [=](uint32_t it) {
              const uint32_t piece = it * 64 + lane, r = piece / UNITS, u = piece % UNITS;
              return *reinterpret_cast<const Chunk*>(slab + r * RB + ((u ^ unit_swz(r)) * 16));
            },
            [=](uint32_t it) { return m0 + wm + ii * 32 + (it * 64 + lane) / UNITS; },
            [=](uint32_t it) { return n0 + wn + ((it * 64 + lane) % UNITS) * 8; });
      }
#endif
      asm volatile("" ::: "memory");
    }
#ifdef HC_MI16_TIMESTAMPS
  if (threadIdx.x == 0) {  // over the first 32 bytes of the tile's first row (the result is not used)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    uint64_t* t = (uint64_t*)(C + (size_t)m0 * p.c_rs + n0);
    uint32_t hw_id, xcc_id;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw_id));
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc_id));
    t[0] = ts_start;
    t[1] = ts_loop;
    t[2] = __builtin_amdgcn_s_memrealtime();
    t[3] = ((__builtin_amdgcn_s_memtime() - tc_start) << 16) | ((uint64_t)(xcc_id & 0xf) << 12) | (hw_id & 0xfff);
  }
#endif
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

#ifdef HC_GEMM_MERGED
#define HC_GEMM_NAME(base) base##_m
#else
#define HC_GEMM_NAME(base) base
#endif
#define DEF_MI16(BM, BN, AN, AM, BNAME, BMODE)                                                        \
  extern "C" __global__ __launch_bounds__(256) void HC_GEMM_NAME(hc_gemm_f16_mi16_##BM##x##BN##_##AN##BNAME)( \
      hck_gemm_args p) {                                                                              \
    __shared__ __attribute__((aligned(1024))) char lds0[(BM + BN) * 128];                             \
    __shared__ __attribute__((aligned(1024))) char lds1[(BM + BN) * 128];                             \
    gemm_mi16_impl<BM, BN, AM, BMODE, false>(p, lds0, lds1);                                          \
  }                                                                                                   \
  extern "C" __global__ __launch_bounds__(256) void HC_GEMM_NAME(hc_gemm_f16_mi16_##BM##x##BN##_##AN##BNAME##_e)( \
      hck_gemm_args p) {                                                                              \
    __shared__ __attribute__((aligned(1024))) char lds0[(BM + BN) * 128];                             \
    __shared__ __attribute__((aligned(1024))) char lds1[(BM + BN) * 128];                             \
    gemm_mi16_impl<BM, BN, AM, BMODE, true>(p, lds0, lds1);                                           \
  }
#define DEF_MI16_TILE(BM, BN)                                                                         \
  DEF_MI16(BM, BN, k, DMA_K, k, DMA_K)                                                                \
  DEF_MI16(BM, BN, k, DMA_K, n, DMA_MN)                                                               \
  DEF_MI16(BM, BN, m, DMA_MN, k, DMA_K)                                                               \
  DEF_MI16(BM, BN, m, DMA_MN, n, DMA_MN)
DEF_MI16_TILE(256, 256)
#ifndef HC_MI16_ONLY_256  // (a quick build with the largest tile only, for kernel experiments)
DEF_MI16_TILE(256, 192)
DEF_MI16_TILE(192, 256)
DEF_MI16_TILE(192, 192)
DEF_MI16_TILE(256, 128)
DEF_MI16_TILE(128, 128)
DEF_MI16_TILE(256, 64)
DEF_MI16_TILE(128, 64)
DEF_MI16_TILE(64, 64)
#endif
