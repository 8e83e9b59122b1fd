// One kernel for the attention of a head: scores = q k^T, the softmax chain over every row of
// scores ([* scale] [+ mask] logSoftmax [exp]), out = probabilities x v; fp16, 64-wide heads. It
// exists for recordings: the rewrite of a recording replaces the three launches (batched product,
// row kernel, batched product) by this one when the scores and the probabilities have no other
// reader, and a replay must return the bits of the three launches. So this kernel does their
// arithmetic, not a rearranged one:
//   * both products accumulate in fp32 with v_mfma_f32_32x32x16_f16, the second operand of the
//     product first, k ascending in steps of 16, as every tiled 32x32x16 kernel of the library does
//     (gemm_dma.hip, gemm_dma2.hip), and round once to fp16;
//   * the scores are rounded to fp16 and laid out in LDS as a [64, T] tile; a team of LANES lanes
//     then takes a row exactly as the row kernel takes it from memory (RowRegs: lane l owns the
//     16-byte vectors l, l + LANES, ...; the same order of partial sums, the same shuffles, the same
//     exponential), writes the probabilities back in fp16, and the second product reads them.
// The softmax is over the whole row (true maximum and sum, as the reference computes it,
// BackendCPU.swift:1000-1038), not a running one, so the score tile must hold whole rows: T <= TMAX.
// The fp32 form (attention_f32_impl, further down) is built the same way around v_mfma_f32_32x32x2_f32.
//
// A workgroup (4 waves) owns 64 query rows of one head. grid.x = T / 64, grid.y = heads.
//   phase 0: q tile and all keys into LDS (rows of 128 bytes, 16-byte chunk c of row r in slot
//            c ^ (r & 7), so that the MFMA operand reads of 32 rows hit different banks); the
//            values are fetched into registers meanwhile
//   phase 1: wave w multiplies the q tile with keys 128 p + 32 w .. + 31 (p = 0, 1, ...): two
//            32 x 32 accumulators, four MFMAs each; scores to LDS
//   phase 2: row teams run the chain in place; the values go to LDS over the keys
//   phase 3: wave w owns a 32 x 32 tile of the [64, 64] output, k over the T keys; the values are
//            stored [key][64] and read with the transposing LDS read, like an operand that is
//            contiguous along n in the tiled GEMM kernels
#include "row_teams.hip.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t Chunk __attribute__((ext_vector_type(4)));
#define LDS_AS __attribute__((address_space(3)))

// Workgroup barrier for LDS traffic only: this wave's LDS accesses are done (lgkmcnt), nothing is said
// about loads from memory that are still on their way into registers.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// Which head (z) and which block of 64 query rows (qb) a workgroup takes; grid.x = blocks per head, grid.y = heads.
// Workgroups go to the eight XCDs round robin in launch order and every XCD has an L2 of its own: the blocks
// of one head, which all read that head's keys and values, are given to workgroups 8 apart, so they run on
// one XCD and the keys and values come from memory once. (Heads beyond the last whole group of 8: launch order.)
__device__ __forceinline__ void attention_block(uint32_t& z, uint32_t& qb) {
  const uint32_t nq = gridDim.x, heads = gridDim.y;
  const uint32_t l = blockIdx.y * nq + blockIdx.x;
  const uint32_t grouped = heads / 8 * 8 * nq;
  if (l < grouped) {
    const uint32_t g = l / (8 * nq), r = l - g * 8 * nq;
    z = 8 * g + (r & 7);
    qb = r >> 3;
  } else {
    z = l / nq;
    qb = l - z * nq;
  }
}

// Phase 2 of the kernel below: the softmax chain over the BQ rows of the score tile in LDS, in place.
// NCH = 16-byte vectors of scores (eight fp16, four fp32) a lane holds per row. `n` is the row length the lanes test
// their vectors against: the caller passes a constant (the full NCH * LANES * VEC) when T fills the vectors
// exactly, and the tests fold away: straight-line code, where the tested form has an exec-mask
// branch around every vector of every step.
template <typename T, int LANES, int NCH, uint32_t BQ, uint32_t SP>
__device__ __forceinline__ void attention_softmax_rows(const hck_attention_args& p, char* s_lds, const uint32_t n, const uint32_t TT,
                                                       const uint32_t z, const uint32_t m0) {
  const uint32_t tid = threadIdx.x;
  typedef RowRegs<T, LANES, NCH> Row;
  constexpr bool HALF = sizeof(T) == 2;
  constexpr int VEC = Row::VEC, CHUNKS = Row::CHUNKS;
  constexpr uint32_t TEAMS = HCK_BLOCK / LANES;       // rows the workgroup's teams take in one go
  constexpr int R = TEAMS * 8 <= BQ ? 8 : BQ / TEAMS;  // 8 rows per team at a time (2 with 32 teams)
  static_assert(BQ % (TEAMS * R) == 0, "the teams' passes cover the tile exactly");
  const uint32_t tl = tid % LANES, team = tid / LANES;
  const bool then_exp = (p.flags & HCK_SM_EXP) != 0;
  for (uint32_t first = team * R; first < BQ; first += TEAMS * R) {
    Row r[R];
#pragma unroll
    for (int j = 0; j < R; j++) r[j].load((const T*)(s_lds + (first + j) * SP), n, tl);
    // Two of the chain's steps are fp16 in, fp16 out with one operation in between, formed in fp32 by
    // the separate kernels: x * s and x + mask. With both operands fp16 values the fp32 result is exact
    // (product: 22 significant bits) or rounds innocuously twice (sum: fp32 has 2 * 11 + 2 bits), so the
    // packed fp16 instruction returns the same bits at an eighth of the instructions (no conversions,
    // two elements each). The scale qualifies when it is an fp16 value itself (1 / 8 is), which is
    // wave-uniform; otherwise the fp32 form stays.
    if (p.flags & HCK_SM_SCALE) {
      const float s = p.scale;
      const half_t s16 = (half_t)s;
      if (HALF && (float)s16 == s) {
        const half2_t s2 = {s16, s16};
#pragma unroll
        for (int j = 0; j < R; j++)
#pragma unroll
          for (int c = 0; c < CHUNKS; c++)
#pragma unroll
            for (int i = 0; i < VEC; i += 2) {
              const half2_t x = {(half_t)r[j].v[c][i], (half_t)r[j].v[c][i + 1]};
              const half2_t y = x * s2;
              r[j].v[c][i] = y[0], r[j].v[c][i + 1] = y[1];
            }
      } else {
#pragma unroll
        for (int j = 0; j < R; j++)
#pragma unroll
          for (int c = 0; c < CHUNKS; c++)
#pragma unroll
            for (int i = 0; i < VEC; i++) r[j].v[c][i] = narrow<T>((float)r[j].v[c][i] * s);
      }
    }
    if (p.flags & HCK_SM_MASK) {
      Row m[R];
#pragma unroll
      for (int j = 0; j < R; j++) {
        const uint64_t grow = (uint64_t)z * TT + m0 + first + j;  // this row among all score rows
        m[j].load((const T*)p.mask + (size_t)(grow % p.mask_rows) * TT, n, tl);
      }
#pragma unroll
      for (int j = 0; j < R; j++)
#pragma unroll
        for (int c = 0; c < CHUNKS; c++)
          if ((tl + LANES * c) * VEC < n) {
            if constexpr (HALF) {
#pragma unroll
              for (int i = 0; i < VEC; i += 2) {
                const half2_t x = {(half_t)r[j].v[c][i], (half_t)r[j].v[c][i + 1]}, y = {(half_t)m[j].v[c][i], (half_t)m[j].v[c][i + 1]};
                const half2_t w = x + y;
                r[j].v[c][i] = w[0], r[j].v[c][i + 1] = w[1];
              }
            } else {
#pragma unroll
              for (int i = 0; i < VEC; i++) r[j].v[c][i] = narrow<T>((float)r[j].v[c][i] + (float)m[j].v[c][i]);
            }
          }
    }
    float mx[R], sum[R];
#pragma unroll
    for (int j = 0; j < R; j++) {
      mx[j] = -INFINITY;
      r[j].each(n, tl, [&](float x) { if (x > mx[j]) mx[j] = x; });
    }
    team_reduce_each<LANES, R>(mx, MaxOp());
#pragma unroll
    for (int j = 0; j < R; j++) {
      sum[j] = 0.0f;
      r[j].each(n, tl, [&](float x) { sum[j] += exp_in<T>(x - mx[j]); });
    }
    team_reduce_each<LANES, R>(sum, SumOp());
#pragma unroll
    for (int j = 0; j < R; j++) {
      const float log_sum = logf(sum[j]) + mx[j];
      r[j].store((T*)(s_lds + (first + j) * SP), n, tl, [&](float x) {
        const float ls = x - log_sum;
        if (!then_exp) return ls;
        const float stored = (float)narrow<T>(ls);
        return (HALF ? exp_hw(stored) : expf(stored)) * 1.0f;
      });
    }
  }
}

template <int TMAX, int LANES> __device__ __forceinline__ void attention_impl(const hck_attention_args& p) {
  constexpr uint32_t BQ = 64;
  constexpr uint32_t SP = TMAX * 2 + 16;  // bytes per row of the score tile (rows stay 16-byte aligned)
  constexpr uint32_t VP = 144;            // bytes per key row of the values (128 + a shift of the banks)
  constexpr int KV_CHUNKS = TMAX * 8 / HCK_BLOCK;  // 16-byte chunks of k (or v) per lane
  __shared__ __attribute__((aligned(16))) char q_lds[BQ * 128];
  __shared__ __attribute__((aligned(16))) char kv_lds[TMAX * VP];
  __shared__ __attribute__((aligned(16))) char s_lds[BQ * SP];

  const uint32_t T = p.T, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t z, qb;
  attention_block(z, qb);
  const uint32_t m0 = qb * BQ;
  uint32_t zh = z, zl = 0;
  if (p.bdiv != 0) {
    zh = z / p.bdiv;
    zl = z - zh * p.bdiv;
  }
  const half_t* Q = (const half_t*)p.q + zh * p.q_bs + zl * p.q_bs2 + (size_t)m0 * p.q_rs;
  const half_t* K = (const half_t*)p.k + zh * p.k_bs + zl * p.k_bs2;
  const half_t* V = (const half_t*)p.v + zh * p.v_bs + zl * p.v_bs2;
  half_t* O = (half_t*)p.out + zh * p.o_bs + zl * p.o_bs2 + (size_t)m0 * p.o_rs;

#ifdef HC_ATTENTION_TIMESTAMPS
  uint64_t ts[6];
  ts[0] = __builtin_amdgcn_s_memrealtime();
#define HC_TS(i) ts[i] = __builtin_amdgcn_s_memrealtime()
#else
#define HC_TS(i)
#endif
  // ---- phase 0: q and k first, v behind them: v is not needed before phase 3, so its loads stay in flight
  // through the scores (the barrier below waits for LDS only, not for them)
#pragma unroll
  for (int i = 0; i < (int)(BQ * 8 / HCK_BLOCK); i++) {
    const uint32_t piece = i * HCK_BLOCK + tid, r = piece >> 3, c = piece & 7;
    *reinterpret_cast<Chunk*>(q_lds + r * 128 + ((c ^ (r & 7)) * 16)) = *reinterpret_cast<const Chunk*>(Q + (size_t)r * p.q_rs + c * 8);
  }
  Chunk kreg[KV_CHUNKS], vreg[KV_CHUNKS];
#pragma unroll
  for (int i = 0; i < KV_CHUNKS; i++) {
    const uint32_t piece = i * HCK_BLOCK + tid, r = piece >> 3, c = piece & 7;
    if (r < T) kreg[i] = *reinterpret_cast<const Chunk*>(K + (size_t)r * p.k_rs + c * 8);
  }
#pragma unroll
  for (int i = 0; i < KV_CHUNKS; i++) {
    const uint32_t piece = i * HCK_BLOCK + tid, r = piece >> 3, c = piece & 7;
    if (r < T) vreg[i] = *reinterpret_cast<const Chunk*>(V + (size_t)r * p.v_rs + c * 8);
  }
#pragma unroll
  for (int i = 0; i < KV_CHUNKS; i++) {
    const uint32_t piece = i * HCK_BLOCK + tid, r = piece >> 3, c = piece & 7;
    if (r < T) *reinterpret_cast<Chunk*>(kv_lds + r * 128 + ((c ^ (r & 7)) * 16)) = kreg[i];
  }
  lds_barrier();
  HC_TS(1);

  // ---- phase 1: scores
  const uint32_t l32 = lane & 31, lgrp = lane >> 5;
  Chunk qf[2][4];  // the q tile's operands: rows 32 mt + l32, k = 16 s + 8 lgrp .. + 7
#pragma unroll
  for (int mt = 0; mt < 2; mt++)
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const uint32_t r = mt * 32 + l32;
      qf[mt][s] = *reinterpret_cast<const Chunk*>(q_lds + r * 128 + (((2 * s + lgrp) ^ (r & 7)) * 16));
    }
  for (uint32_t nb = wave * 32; nb < T; nb += 128) {
    floatx16 acc[2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[mt][e] = 0.0f;
    const uint32_t r = nb + l32;
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const Chunk kf = *reinterpret_cast<const Chunk*>(kv_lds + r * 128 + (((2 * s + lgrp) ^ (r & 7)) * 16));
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
        acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, kf), __builtin_bit_cast(half8, qf[mt][s]), acc[mt], 0, 0, 0);
    }
    // lane: query row 32 mt + l32, keys nb + 8 g + 4 lgrp .. + 3 in registers 4 g .. 4 g + 3
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        half4v h;
#pragma unroll
        for (int e = 0; e < 4; e++) h[e] = narrow<half_t>(acc[mt][4 * g + e]);
        *reinterpret_cast<half4v*>(s_lds + (mt * 32 + l32) * SP + (nb + 8 * g + 4 * lgrp) * 2) = h;
      }
  }
  __syncthreads();  // scores complete; nobody reads the keys any more
  HC_TS(2);

  // the values over the keys: [key][64 halfs], rows of VP bytes
#pragma unroll
  for (int i = 0; i < KV_CHUNKS; i++) {
    const uint32_t piece = i * HCK_BLOCK + tid, r = piece >> 3, c = piece & 7;
    if (r < T) *reinterpret_cast<Chunk*>(kv_lds + r * VP + c * 16) = vreg[i];
  }

  // ---- phase 2: the chain over the rows of the score tile, in place (softmax_chain_rows_impl of
  // the row kernels, with the row in LDS instead of memory). A team works on R rows at a time (8, or all it has), stage
  // by stage, so that the latencies of one row's shuffles and exponentials hide behind the others'
  // (there is one wave per SIMD here, not the many of the row kernel); per row the arithmetic and its
  // order are the row kernel's.
  {
    // (vectors per lane: what rows of TMAX elements need, at most the row kernel's four)
    constexpr int NCH = (TMAX + LANES * 8 - 1) / (LANES * 8);
    static_assert(NCH <= 4, "rows of TMAX elements fit the team's registers");
    constexpr uint32_t FULL = LANES * 8;   // scores per vector round of a team
    // T is a multiple of 64 (the host's condition): with teams of 8 lanes it fills T / 64 rounds exactly
    if (T == NCH * FULL) attention_softmax_rows<half_t, LANES, NCH, BQ, SP>(p, s_lds, NCH * FULL, T, z, m0);
    else if (NCH > 1 && T == (NCH - 1) * FULL) attention_softmax_rows<half_t, LANES, (NCH > 1 ? NCH - 1 : 1), BQ, SP>(p, s_lds, (NCH - 1) * FULL, T, z, m0);
    else if (NCH > 2 && T == (NCH - 2) * FULL) attention_softmax_rows<half_t, LANES, (NCH > 2 ? NCH - 2 : 1), BQ, SP>(p, s_lds, (NCH - 2) * FULL, T, z, m0);
    else if (NCH > 3 && T == (NCH - 3) * FULL) attention_softmax_rows<half_t, LANES, (NCH > 3 ? NCH - 3 : 1), BQ, SP>(p, s_lds, (NCH - 3) * FULL, T, z, m0);
    else attention_softmax_rows<half_t, LANES, NCH, BQ, SP>(p, s_lds, T, T, z, m0);
  }
  __syncthreads();
  HC_TS(3);

  // ---- phase 3: out tile (mt, nt) of wave w; operands: probabilities rows 32 mt + l32 (k-contiguous),
  // values columns 32 nt + l32 through the transposing read (a group of 16 lanes: k-rows
  // 8 (grp / 2) + 4 h + r / 4, columns 16 (grp % 2) + 4 (r % 4) .. + 3; lane i receives column i)
  {
    const uint32_t mt = wave >> 1, nt = wave & 1;
    const uint32_t r16 = lane & 15, grp = lane >> 4;
    floatx16 acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.0f;
    const char* prow = s_lds + (mt * 32 + l32) * SP + lgrp * 16;
    const char* vcol = kv_lds + (8 * (grp >> 1) + (r16 >> 2)) * VP + (nt * 32 + 16 * (grp & 1) + 4 * (r16 & 3)) * 2;
    for (uint32_t k0 = 0; k0 < T; k0 += 16) {
      const Chunk pf = *reinterpret_cast<const Chunk*>(prow + k0 * 2);
      typedef short short4v __attribute__((ext_vector_type(4)));
      typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
      const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS short4v*)(vcol + k0 * VP)));
      const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS short4v*)(vcol + (k0 + 4) * VP)));
      const Chunk vf = {lo[0], lo[1], hi[0], hi[1]};
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, vf), __builtin_bit_cast(half8, pf), acc, 0, 0, 0);
    }
    // lane: query row 32 mt + l32, columns 32 nt + 8 g + 4 lgrp .. + 3
#pragma unroll
    for (int g = 0; g < 4; g++) {
      half4v h;
#pragma unroll
      for (int e = 0; e < 4; e++) h[e] = narrow<half_t>(acc[4 * g + e]);
      *reinterpret_cast<half4v*>(O + (size_t)(mt * 32 + l32) * p.o_rs + nt * 32 + 8 * g + 4 * lgrp) = h;
    }
  }
#ifdef HC_ATTENTION_TIMESTAMPS
  HC_TS(4);
  if (tid == 0) {   // (measurement build: over the first bytes of the tile's first row)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    ts[5] = __builtin_amdgcn_s_memrealtime();
    for (int i = 0; i < 6; i++) ((uint64_t*)O)[i] = ts[i];
  }
#endif
}

// The same kernel for fp32 tensors, T <= 256. Both products run on v_mfma_f32_32x32x2_f32 as the tiled
// fp32 kernels of the library run them (gemm_dma.hip, gemm_dma2.hip): the second operand of the product
// first, and inside every 16 k the instructions take the pairs k = {0, 4}, {1, 5}, {2, 6}, {3, 7},
// {8, 12}, ... in this order (a lane of the upper half of the wave holds the second k of a pair), so a
// score or an output element is the same chain of fused additions here and there. Rows of fp32 are 256
// bytes per 64 k: 16 chunks of 16 bytes, chunk c of row r in slot c ^ (r & 15).
//   phase 0: q tile and keys to LDS, values into registers
//   phase 1: wave w multiplies the q tile with keys 128 p + 32 w .. + 31; fp32 scores to LDS as a [64, T] tile
//   phase 2: the row teams' chain in place (a wave per row for T > 128, 8 lanes below: what hc_log_softmax
//            picks for fp32 rows of these lengths); the values go to LDS over the keys, [key][64 floats], the
//            128-byte halves of key rows with bit 2 set swapped (an operand read takes 32 floats of key k from
//            one half of the wave and 32 of key k + 4 from the other)
//   phase 3: wave w owns a 32 x 32 tile of the output, k over the T keys
template <int TMAX> __device__ __forceinline__ void attention_f32_impl(const hck_attention_args& p) {
  constexpr uint32_t BQ = 64;
  constexpr uint32_t SP = TMAX * 4 + 16;  // bytes per row of the score tile
  constexpr int Q_CHUNKS = BQ * 16 / HCK_BLOCK, KV_CHUNKS = TMAX * 16 / HCK_BLOCK;  // 16-byte chunks per lane
  __shared__ __attribute__((aligned(16))) char q_lds[BQ * 256];
  __shared__ __attribute__((aligned(16))) char kv_lds[TMAX * 256];
  __shared__ __attribute__((aligned(16))) char s_lds[BQ * SP];

  const uint32_t T = p.T, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t z, qb;
  attention_block(z, qb);
  const uint32_t m0 = qb * BQ;
  uint32_t zh = z, zl = 0;
  if (p.bdiv != 0) {
    zh = z / p.bdiv;
    zl = z - zh * p.bdiv;
  }
  const float* Q = (const float*)p.q + zh * p.q_bs + zl * p.q_bs2 + (size_t)m0 * p.q_rs;
  const float* K = (const float*)p.k + zh * p.k_bs + zl * p.k_bs2;
  const float* V = (const float*)p.v + zh * p.v_bs + zl * p.v_bs2;
  float* O = (float*)p.out + zh * p.o_bs + zl * p.o_bs2 + (size_t)m0 * p.o_rs;

#ifdef HC_ATTENTION_TIMESTAMPS
  uint64_t ts[6];
  ts[0] = __builtin_amdgcn_s_memrealtime();
#endif
  // ---- phase 0
#pragma unroll
  for (int i = 0; i < Q_CHUNKS; i++) {
    const uint32_t piece = i * HCK_BLOCK + tid, r = piece >> 4, c = piece & 15;
    *reinterpret_cast<Chunk*>(q_lds + r * 256 + ((c ^ (r & 15)) * 16)) = *reinterpret_cast<const Chunk*>(Q + (size_t)r * p.q_rs + c * 4);
  }
  Chunk kreg[KV_CHUNKS], vreg[KV_CHUNKS];
#pragma unroll
  for (int i = 0; i < KV_CHUNKS; i++) {
    const uint32_t piece = i * HCK_BLOCK + tid, r = piece >> 4, c = piece & 15;
    if (r < T) kreg[i] = *reinterpret_cast<const Chunk*>(K + (size_t)r * p.k_rs + c * 4);
  }
#pragma unroll
  for (int i = 0; i < KV_CHUNKS; i++) {
    const uint32_t piece = i * HCK_BLOCK + tid, r = piece >> 4, c = piece & 15;
    if (r < T) vreg[i] = *reinterpret_cast<const Chunk*>(V + (size_t)r * p.v_rs + c * 4);
  }
#pragma unroll
  for (int i = 0; i < KV_CHUNKS; i++) {
    const uint32_t piece = i * HCK_BLOCK + tid, r = piece >> 4, c = piece & 15;
    if (r < T) *reinterpret_cast<Chunk*>(kv_lds + r * 256 + ((c ^ (r & 15)) * 16)) = kreg[i];
  }
  lds_barrier();
  HC_TS(1);

  // ---- phase 1: scores
  const uint32_t l32 = lane & 31, lgrp = lane >> 5;
  {
    Chunk qf[2][8];  // the q tile's operands: rows 32 mt + l32, chunk 2 u + lgrp = k 8 u + 4 lgrp .. + 3
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const uint32_t r = mt * 32 + l32;
        qf[mt][u] = *reinterpret_cast<const Chunk*>(q_lds + r * 256 + (((2 * u + lgrp) ^ (r & 15)) * 16));
      }
    for (uint32_t nb = wave * 32; nb < T; nb += 128) {
      floatx16 acc[2];
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[mt][e] = 0.0f;
      const uint32_t r = nb + l32;
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const Chunk kf = *reinterpret_cast<const Chunk*>(kv_lds + r * 256 + (((2 * u + lgrp) ^ (r & 15)) * 16));
#pragma unroll
        for (int e = 0; e < 4; e++) {
          // (copies first: a bit_cast applied directly to a vector element reads element 0)
          const uint32_t wk = kf[e];
#pragma unroll
          for (int mt = 0; mt < 2; mt++) {
            const uint32_t wq = qf[mt][u][e];
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, wk), __builtin_bit_cast(float, wq), acc[mt], 0, 0, 0);
          }
        }
      }
      // lane: query row 32 mt + l32, keys nb + 8 g + 4 lgrp .. + 3 in registers 4 g .. 4 g + 3
#pragma unroll
      for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          floatx4 h;
#pragma unroll
          for (int e = 0; e < 4; e++) h[e] = acc[mt][4 * g + e];
          *reinterpret_cast<floatx4*>(s_lds + (mt * 32 + l32) * SP + (nb + 8 * g + 4 * lgrp) * 4) = h;
        }
    }
  }
  __syncthreads();  // scores complete; nobody reads the keys any more
  HC_TS(2);

  // the values over the keys
#pragma unroll
  for (int i = 0; i < KV_CHUNKS; i++) {
    const uint32_t piece = i * HCK_BLOCK + tid, r = piece >> 4, c = piece & 15;
    if (r < T) *reinterpret_cast<Chunk*>(kv_lds + r * 256 + ((c ^ (((r >> 2) & 1u) << 3)) * 16)) = vreg[i];
  }

  // ---- phase 2
  if (T > 128) {
    constexpr int NCH = (TMAX + 255) / 256;   // a wave per row: 256 scores per round of vectors
    static_assert(NCH == 1, "rows of TMAX fp32 scores are one vector per lane of a wave");
    if (T == 256) attention_softmax_rows<float, 64, 1, BQ, SP>(p, s_lds, 256, T, z, m0);
    else attention_softmax_rows<float, 64, 1, BQ, SP>(p, s_lds, T, T, z, m0);
  } else {
    // teams of 8 lanes: 32 scores per round, T a multiple of 64
    if (T == 128) attention_softmax_rows<float, 8, 4, BQ, SP>(p, s_lds, 128, T, z, m0);
    else attention_softmax_rows<float, 8, 2, BQ, SP>(p, s_lds, T, T, z, m0);
  }
  __syncthreads();
  HC_TS(3);

  // ---- phase 3: out tile (mt, nt) of wave w; operands: values column 32 nt + l32 (one float per key), probabilities
  // row 32 mt + l32 (k-contiguous)
  {
    const uint32_t mt = wave >> 1, nt = wave & 1;
    floatx16 acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.0f;
    const char* prow = s_lds + (mt * 32 + l32) * SP + lgrp * 16;
    // key k0 + 8 s + 4 lgrp + e: bit 2 of the key is lgrp (k0 + 8 s is a multiple of 8), which picks the half
    const char* vcol = kv_lds + 4 * lgrp * 256 + (((nt * 32 + l32) ^ (lgrp << 5)) * 4);
    for (uint32_t k0 = 0; k0 < T; k0 += 8) {
      const Chunk pf = *reinterpret_cast<const Chunk*>(prow + k0 * 4);
      uint32_t vf[4];
#pragma unroll
      for (int e = 0; e < 4; e++) vf[e] = *reinterpret_cast<const uint32_t*>(vcol + (k0 + e) * 256);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const uint32_t wp = pf[e];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, vf[e]), __builtin_bit_cast(float, wp), acc, 0, 0, 0);
      }
    }
    // lane: query row 32 mt + l32, columns 32 nt + 8 g + 4 lgrp .. + 3
#pragma unroll
    for (int g = 0; g < 4; g++) {
      floatx4 h;
#pragma unroll
      for (int e = 0; e < 4; e++) h[e] = acc[4 * g + e];
      *reinterpret_cast<floatx4*>(O + (size_t)(mt * 32 + l32) * p.o_rs + nt * 32 + 8 * g + 4 * lgrp) = h;
    }
  }
#ifdef HC_ATTENTION_TIMESTAMPS
  HC_TS(4);
  if (tid == 0) {   // (measurement build: over the first bytes of the tile's first row)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    ts[5] = __builtin_amdgcn_s_memrealtime();
    for (int i = 0; i < 6; i++) ((uint64_t*)O)[i] = ts[i];
  }
#endif
}


// (rows of up to 256 halfs are taken by teams of 8 lanes, longer ones by a wave: what hc_log_softmax
// picks for rows of these lengths)
HC_KERNEL void hc_attention_f16_t256(hck_attention_args p) { attention_impl<256, 8>(p); }
HC_KERNEL void hc_attention_f16_t512(hck_attention_args p) { attention_impl<512, 64>(p); }
HC_KERNEL void hc_attention_f32_t256(hck_attention_args p) { attention_f32_impl<256>(p); }
