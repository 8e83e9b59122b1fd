// General MFMA GEMM for gfx950: C[M,N] = A[M,K] * B[K,N] per batch element, fp16 inputs
// with fp32 accumulation (v_mfma_f32_32x32x16_f16) and fp32 (v_mfma_f32_32x32x2_f32).
// Handles every transpose combination and ragged M, N, K; the tuned kernels in
// gemm_f16_fast.hip take over for large aligned fp16 problems.
//
// Tile: 128 x 128 outputs per 256-lane block, four waves in a 2 x 2 grid, each wave a
// 64 x 64 sub-tile = 2 x 2 MFMA 32x32 accumulators (64 fp32 VGPRs). K advances in steps
// of 128 bytes per row (64 halfs / 32 floats). Both operands live in LDS K-contiguous
// ([row][k], 144-byte pitch) so one ds_read_b128 per lane yields an MFMA operand:
//   lane l reads row (l % 32), 16-byte chunk (2*s + l / 32) at sub-step s.
// Any consistent k -> (lane group, slot) assignment is valid because A and B use the same.
//
// Global -> LDS, chosen per operand by the host:
//   LOAD_K   operand contiguous along k: 16-byte loads, 8 lanes per 128-byte row segment.
//   LOAD_MN  operand contiguous along m (or n): each lane loads 4 k-rows x 16 bytes,
//            transposes the 4 x P block in registers and writes P chunks of 4 k-values.
//   LOAD_ANY arbitrary strides / unaligned / ragged: predicated scalar loads.
// The next K-step is fetched into registers before the MFMAs of the current one.
#include "common.hip.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

enum { LOAD_K = 0, LOAD_MN = 1, LOAD_ANY = 2 };

#define G_BM 128
#define G_BN 128
#define G_ROW_BYTES 128
#define G_PITCH 144 /* bytes: 128 + 16 pad keeps ds_read_b128 of 32 rows off the same banks */

template <typename T> struct GemmTraits;
template <> struct GemmTraits<half_t> {
  static constexpr int P = 8;   // elements per 16 bytes
  static constexpr int BK = 64; // elements per K-step
};
template <> struct GemmTraits<float> {
  static constexpr int P = 4;
  static constexpr int BK = 32;
};

struct alignas(16) Chunk16 {
  uint32_t w[4];
};

__device__ __forceinline__ void mma_chunk(floatx16& acc, const Chunk16& a, const Chunk16& b, half_t) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8*>(&a),
                                               *reinterpret_cast<const half8*>(&b), acc, 0, 0, 0);
}
__device__ __forceinline__ void mma_chunk(floatx16& acc, const Chunk16& a, const Chunk16& b, float) {
  const float* af = reinterpret_cast<const float*>(&a);
  const float* bf = reinterpret_cast<const float*>(&b);
#pragma unroll
  for (int i = 0; i < 4; i++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[i], acc, 0, 0, 0);
}

// Registers holding one operand's share of a K-step (128 rows x 128 bytes / 256 lanes = 64 B).
template <typename T> struct Staged {
  Chunk16 v[4];
};

// Fetch this lane's part of the tile rows [r0, r0+128) x k [k0, k0+BK) of an operand whose
// logical element (r, k) sits at base[r*rs + k*cs]. Out-of-range elements read as zero.
template <typename T, int MODE>
__device__ __forceinline__ void fetch(Staged<T>& st, const T* base, uint32_t rs, uint32_t cs,
                                      uint32_t r0, uint32_t k0, uint32_t R, uint32_t K) {
  constexpr int P = GemmTraits<T>::P;
  constexpr int BK = GemmTraits<T>::BK;
  const uint32_t t = threadIdx.x;
  if (MODE == LOAD_K) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t id = t + 256 * i;
      const uint32_t r = r0 + id / 8, k = k0 + (id % 8) * P;
      Chunk16 z = {{0, 0, 0, 0}};
      if (r < R && k < K) z = *reinterpret_cast<const Chunk16*>(base + (size_t)r * rs + k);
      st.v[i] = z;
    }
  } else if (MODE == LOAD_MN) {
    constexpr int MB = G_BM / P;  // 16-byte blocks along the contiguous m/n axis
    const uint32_t r = r0 + (t % MB) * P, kb = k0 + (t / MB) * 4;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      Chunk16 z = {{0, 0, 0, 0}};
      if (r < R && kb + i < K) z = *reinterpret_cast<const Chunk16*>(base + (size_t)(kb + i) * cs + r);
      st.v[i] = z;
    }
  } else {
    T* e = reinterpret_cast<T*>(&st);
    constexpr int PER = G_BM * BK / 256;
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const uint32_t id = t + 256 * i;
      uint32_t r, k;
      if (cs <= rs) {  // k is the faster-varying axis in memory
        r = id / BK;
        k = id % BK;
      } else {
        k = id / G_BM;
        r = id % G_BM;
      }
      T val = (T)0;
      if (r0 + r < R && k0 + k < K) val = base[(size_t)(r0 + r) * rs + (size_t)(k0 + k) * cs];
      e[i] = val;
    }
  }
}

// Write the staged registers into the K-contiguous LDS tile.
template <typename T, int MODE>
__device__ __forceinline__ void stash(const Staged<T>& st, char* lds, uint32_t rs, uint32_t cs) {
  constexpr int P = GemmTraits<T>::P;
  constexpr int BK = GemmTraits<T>::BK;
  const uint32_t t = threadIdx.x;
  if (MODE == LOAD_K) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t id = t + 256 * i;
      *reinterpret_cast<Chunk16*>(lds + (id / 8) * G_PITCH + (id % 8) * 16) = st.v[i];
    }
  } else if (MODE == LOAD_MN) {
    constexpr int MB = G_BM / P;
    const uint32_t r = (t % MB) * P, kb = (t / MB) * 4;
    const T* e = reinterpret_cast<const T*>(&st);  // e[i*P + p] = element (k = kb+i, row r+p)
#pragma unroll
    for (int p = 0; p < P; p++) {
      T col[4];
#pragma unroll
      for (int i = 0; i < 4; i++) col[i] = e[i * P + p];
      *reinterpret_cast<Vec<T, 4>*>(lds + (r + p) * G_PITCH + kb * sizeof(T)) =
          *reinterpret_cast<Vec<T, 4>*>(col);
    }
  } else {
    const T* e = reinterpret_cast<const T*>(&st);
    constexpr int PER = G_BM * BK / 256;
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const uint32_t id = t + 256 * i;
      uint32_t r, k;
      if (cs <= rs) {
        r = id / BK;
        k = id % BK;
      } else {
        k = id / G_BM;
        r = id % G_BM;
      }
      *reinterpret_cast<T*>(lds + r * G_PITCH + k * sizeof(T)) = e[i];
    }
  }
}

template <typename T, int MODE_A, int MODE_B>
__device__ __forceinline__ void gemm_impl(const hck_gemm_args& p) {
  constexpr int BK = GemmTraits<T>::BK;
  __shared__ __attribute__((aligned(16))) char lds_a[G_BM * G_PITCH];
  __shared__ __attribute__((aligned(16))) char lds_b[G_BN * G_PITCH];

  const uint32_t tile = blockIdx.x;
  const uint32_t tm = tile / p.tiles_n, tn = tile % p.tiles_n;
  const uint32_t batch = blockIdx.y;
  const T* A = (const T*)p.a + batch * p.a_bs;
  const T* B = (const T*)p.b + batch * p.b_bs;
  T* C = (T*)p.c + batch * p.c_bs;
  const uint32_t m0 = tm * G_BM, n0 = tn * G_BN;

  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const uint32_t lrow = lane & 31, lgrp = lane >> 5;

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

  Staged<T> sa, sb;
  // B is addressed as rows = n, so its "row stride" is b_cs and its k stride is b_rs.
  fetch<T, MODE_A>(sa, A, p.a_rs, p.a_cs, m0, 0, p.M, p.K);
  fetch<T, MODE_B>(sb, B, p.b_cs, p.b_rs, n0, 0, p.N, p.K);

  for (uint32_t k0 = 0; k0 < p.K; k0 += BK) {
    __syncthreads();  // previous step's LDS reads are done
    stash<T, MODE_A>(sa, lds_a, p.a_rs, p.a_cs);
    stash<T, MODE_B>(sb, lds_b, p.b_cs, p.b_rs);
    __syncthreads();
    if (k0 + BK < p.K) {
      fetch<T, MODE_A>(sa, A, p.a_rs, p.a_cs, m0, k0 + BK, p.M, p.K);
      fetch<T, MODE_B>(sb, B, p.b_cs, p.b_rs, n0, k0 + BK, p.N, p.K);
    }
#pragma unroll
    for (int s = 0; s < 4; s++) {
      Chunk16 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; i++) {
        fa[i] = *reinterpret_cast<const Chunk16*>(lds_a + (wm + i * 32 + lrow) * G_PITCH + (2 * s + lgrp) * 16);
        fb[i] = *reinterpret_cast<const Chunk16*>(lds_b + (wn + i * 32 + lrow) * G_PITCH + (2 * s + lgrp) * 16);
      }
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) mma_chunk(acc[i][j], fa[i], fb[j], T());
    }
  }

  // 32x32 accumulator layout: lane l, register v holds row 8*(v/4) + 4*(l/32) + v%4,
  // column l%32 of the MFMA tile.
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const uint32_t col = n0 + wn + j * 32 + lrow;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const uint32_t row = m0 + wm + i * 32 + 8 * (v / 4) + 4 * lgrp + (v % 4);
        if (row < p.M && col < p.N) C[(size_t)row * p.c_rs + (size_t)col * p.c_cs] = narrow<T>(acc[i][j][v]);
      }
    }
}

#define DEF_GEMM(TN, T, AN, AM, BN_, BM_)                                                            \
  HC_KERNEL void hc_gemm_##TN##_##AN##BN_(hck_gemm_args p) { gemm_impl<T, AM, BM_>(p); }
#define DEF_GEMM_T(TN, T)                                                                            \
  DEF_GEMM(TN, T, k, LOAD_K, k, LOAD_K)                                                              \
  DEF_GEMM(TN, T, k, LOAD_K, n, LOAD_MN)                                                             \
  DEF_GEMM(TN, T, m, LOAD_MN, k, LOAD_K)                                                             \
  DEF_GEMM(TN, T, m, LOAD_MN, n, LOAD_MN)                                                            \
  DEF_GEMM(TN, T, x, LOAD_ANY, x, LOAD_ANY)
DEF_GEMM_T(f16, half_t)
DEF_GEMM_T(f32, float)

// int64 products (BackendCPU.swift:1307-1308 allows them; they are rare): there is no matrix
// instruction for 64-bit integers, so this is a plain LDS-tiled loop on the vector ALU, one
// output element per lane, 16 x 16 outputs per workgroup, sums wrapping like two's complement.
// tiles_m / tiles_n count 16 x 16 tiles; grid.y = batch.
HC_KERNEL void hc_gemm_i64(hck_gemm_args p) {
  __shared__ uint64_t sa[16][17], sb[16][17];
  const uint32_t tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const uint32_t tm = blockIdx.x / p.tiles_n, tn = blockIdx.x - tm * p.tiles_n;
  const uint32_t m = tm * 16 + ty, n = tn * 16 + tx;
  const uint64_t* A = (const uint64_t*)p.a + (uint64_t)blockIdx.y * p.a_bs;
  const uint64_t* B = (const uint64_t*)p.b + (uint64_t)blockIdx.y * p.b_bs;
  uint64_t* C = (uint64_t*)p.c + (uint64_t)blockIdx.y * p.c_bs;
  uint64_t acc = 0;
  for (uint32_t k0 = 0; k0 < p.K; k0 += 16) {
    // sa[row][k], sb[k][col]
    sa[ty][tx] = (m < p.M && k0 + tx < p.K) ? A[(size_t)m * p.a_rs + (size_t)(k0 + tx) * p.a_cs] : 0;
    sb[ty][tx] = (k0 + ty < p.K && n < p.N) ? B[(size_t)(k0 + ty) * p.b_rs + (size_t)n * p.b_cs] : 0;
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; kk++) acc += sa[ty][kk] * sb[kk][tx];
    __syncthreads();
  }
  if (m < p.M && n < p.N) C[(size_t)m * p.c_rs + (size_t)n * p.c_cs] = acc;
}

// Skinny products (one extent of C at most 4: matrix-vector products, the fringes of ragged
// GEMMs): bound by reading the long operand once, so no matrix instructions, fp32 accumulation
// on the vector ALU. C[p, q] = sum_k X[p, k] * Y[k, q], p long, q thin.
//
// Long operand contiguous along k: one wave per p. Lanes stride over k in 16-byte pieces, keep
// one partial sum per q, and the wave adds them up at the end.
template <typename T, int TQ> __device__ __forceinline__ void skinny_k_impl(const hck_skinny_args& a, const uint32_t block) {
  constexpr int V = 16 / sizeof(T);
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t p = block * (HCK_BLOCK / 64) + (threadIdx.x >> 6);
  if (p >= a.L) return;
  const T* X = (const T*)a.x + (uint64_t)blockIdx.y * a.x_bs + (size_t)p * a.x_ps;
  const T* Y = (const T*)a.y + (uint64_t)blockIdx.y * a.y_bs;
  T* C = (T*)a.c + (uint64_t)blockIdx.y * a.c_bs + (size_t)p * a.c_ps;
  float acc[TQ];
#pragma unroll
  for (int q = 0; q < TQ; q++) acc[q] = 0.0f;
  // U steps at a time with all their loads issued first (a row is a handful of steps: one load in
  // flight per lane would make it as many memory latencies in a row); the sums are formed in the
  // order of the plain loop below, which takes what is left
  constexpr int U = 8;
  uint32_t k0 = lane * V;
  for (; k0 + (U - 1) * 64 * V + V <= a.K; k0 += U * 64 * V) {
    T x[U][V];
#pragma unroll
    for (int u = 0; u < U; u++) load_vec_loose<T, V>(X + k0 + u * 64 * V, x[u]);
#pragma unroll
    for (int q = 0; q < TQ; q++) {
      if (q < (int)a.t) {
        T y[U][V];
#pragma unroll
        for (int u = 0; u < U; u++) load_vec<T, V>(Y + (size_t)q * a.y_qs, k0 + u * 64 * V, 1, y[u]);
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
          for (int e = 0; e < V; e++) acc[q] = acc[q] + (float)x[u][e] * (float)y[u][e];
      }
    }
  }
  for (; k0 < a.K; k0 += 64 * V) {
    T x[V];
    if (k0 + V <= a.K) {
      load_vec_loose<T, V>(X + k0, x);   // (rows of X start at any element)
    } else {
#pragma unroll
      for (int e = 0; e < V; e++) x[e] = k0 + e < a.K ? X[k0 + e] : (T)0;
    }
    // Y is contiguous along k with 16-byte aligned rows that are padded to a multiple of V (the
    // host packs it that way if need be), so the same piece of every q is one vector load
#pragma unroll
    for (int q = 0; q < TQ; q++) {
      if (q < (int)a.t) {
        T y[V];
        load_vec<T, V>(Y + (size_t)q * a.y_qs, k0, 1, y);
#pragma unroll
        for (int e = 0; e < V; e++) acc[q] = acc[q] + (float)x[e] * (float)y[e];
      }
    }
  }
#pragma unroll
  for (int q = 0; q < TQ; q++) {
    float v = acc[q];
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v += __shfl_down(v, d, 64);
    if (lane == 0 && q < (int)a.t) C[(size_t)q * a.c_qs] = narrow<T>(v);
  }
}

// Long operand contiguous along p: a lane owns V consecutive p, a
// wave reads 64 * V consecutive elements of a k-row per step; a workgroup covers one such
// p-tile and a chunk of the k-range (grid.x = p-tiles * k-chunks), its four waves take every
// fourth k-row and add their partial sums up in LDS; every chunk leaves its sums in a slice of its
// own of an fp32 buffer and hc_gemm_skinny_store adds the slices in a fixed order and rounds, so
// the result does not depend on which workgroup finishes first. Y is read one element per wave
// and step (wave-uniform), so it is taken as it lies, whatever its strides.
template <typename T, int TQ> __device__ __forceinline__ void skinny_p_impl(const hck_skinny_args& a, const uint32_t block) {
  constexpr int V = 16 / sizeof(T), WAVES = HCK_BLOCK / 64, TILE = 64 * V;
  __shared__ float part[WAVES][TQ][TILE];
  const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t ptiles = (a.L + TILE - 1) / TILE;
  const uint32_t chunk = block / ptiles, pt = block - chunk * ptiles;
  const uint32_t p0 = pt * TILE + lane * V;
  const uint32_t k_lo = chunk * a.kchunk, k_hi = k_lo + a.kchunk < a.K ? k_lo + a.kchunk : a.K;
  const T* X = (const T*)a.x + (uint64_t)blockIdx.y * a.x_bs;
  const T* Y = (const T*)a.y + (uint64_t)blockIdx.y * a.y_bs;
  float acc[TQ][V];
#pragma unroll
  for (int q = 0; q < TQ; q++)
#pragma unroll
    for (int e = 0; e < V; e++) acc[q][e] = 0.0f;
  // (k-rows of X start at any element; the one lane that straddles the end of a row takes its elements one by
  // one, lanes past the end have nothing to add. Two bodies, chosen once per lane: a test around every load
  // would put a wait at each join and the U loads of a step would no longer be in flight together.)
  const bool whole = p0 + V <= a.L, some = p0 < a.L;
  // U of this wave's k-rows at a time, loads first (see skinny_k_impl), sums in the plain loop's order
  constexpr int U = 6;
  auto run = [&](auto load_x) {
    uint32_t k = k_lo + wave;
    for (; k + (U - 1) * WAVES < k_hi; k += U * WAVES) {
      T x[U][V];
#pragma unroll
      for (int u = 0; u < U; u++) load_x(k + u * WAVES, x[u]);
#pragma unroll
      for (int q = 0; q < TQ; q++) {
        if (q < (int)a.t) {
          float y[U];
#pragma unroll
          for (int u = 0; u < U; u++) y[u] = (float)Y[(size_t)q * a.y_qs + (size_t)(k + u * WAVES) * a.y_ks];
#pragma unroll
          for (int u = 0; u < U; u++)
#pragma unroll
            for (int e = 0; e < V; e++) acc[q][e] = acc[q][e] + (float)x[u][e] * y[u];
        }
      }
    }
    for (; k < k_hi; k += WAVES) {
      T x[V];
      load_x(k, x);
#pragma unroll
      for (int q = 0; q < TQ; q++) {
        if (q < (int)a.t) {
          const float y = (float)Y[(size_t)q * a.y_qs + (size_t)k * a.y_ks];  // wave-uniform, any strides
#pragma unroll
          for (int e = 0; e < V; e++) acc[q][e] = acc[q][e] + (float)x[e] * y;
        }
      }
    }
  };
  if (whole) {
    run([&](uint32_t kk, T (&x)[V]) { load_vec_loose<T, V>(X + (size_t)kk * a.x_ks + p0, x); });
  } else if (some) {
    const uint32_t valid = a.L - p0;   // 1 .. V - 1 elements of this lane's piece lie inside the row
    run([&](uint32_t kk, T (&x)[V]) {
#pragma unroll
      for (int e = 0; e < V; e++) x[e] = (T)0;
      const T* src = X + (size_t)kk * a.x_ks + p0;
#pragma unroll
      for (int e = 0; e < V - 1; e++)
        if (e < (int)valid) x[e] = src[e];
    });
  }
#pragma unroll
  for (int q = 0; q < TQ; q++)
#pragma unroll
    for (int e = 0; e < V; e++) part[wave][q][lane * V + e] = acc[q][e];
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < a.t * TILE; i += HCK_BLOCK) {
    const uint32_t q = i / TILE, c = i - q * TILE;
    const uint32_t p = pt * TILE + c;
    if (p >= a.L) continue;
    float v = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; w++) v += part[w][q][c];
    a.acc[(((uint64_t)blockIdx.y * a.chunks + chunk) * a.L + p) * a.t + q] = v;
  }
}

// Y[k, q] (any strides) -> packed[q][k], rows padded with zeros to `y_qs` elements (a multiple of
// a 16-byte piece): a.c = packed, a.y = source, strides of the source in y_ks / c_qs.
template <typename T> __device__ __forceinline__ void skinny_pack_impl(const hck_skinny_args& a, const uint32_t block) {
  const uint64_t i = (uint64_t)block * HCK_BLOCK + threadIdx.x;
  if (i >= (uint64_t)a.t * a.y_qs) return;
  const uint32_t q = (uint32_t)(i / a.y_qs), k = (uint32_t)(i - (uint64_t)q * a.y_qs);
  const T* Y = (const T*)a.y + (uint64_t)blockIdx.y * a.y_bs;
  T* P = (T*)a.c + (uint64_t)blockIdx.y * a.t * a.y_qs;
  P[i] = k < a.K ? Y[(size_t)k * a.y_ks + (size_t)q * a.c_qs] : (T)0;
}

// The chunks' partial sums of one output -> the output: a team of 16 adjacent lanes per output. Lane j of the
// team adds the chunks j, j + 16, ... in this order (all its loads issued first: one load after the other would
// cost a memory latency per chunk), then the 16 lanes add up over lane distances 8, 4, 2, 1: a fixed order, the
// same on every run. A workgroup finishes 16 outputs (grid.x = ceil(L * t / 16)).
constexpr int SKINNY_STORE_TEAM = 16, SKINNY_STORE_ROUNDS = 8;   // chunks <= 16 * 8 (the host's limit)
template <typename T> __device__ __forceinline__ void skinny_store_impl(const hck_skinny_args& a, const uint32_t block) {
  const uint32_t j = threadIdx.x % SKINNY_STORE_TEAM;
  const uint64_t total = (uint64_t)a.L * a.t;
  uint64_t i = (uint64_t)block * (HCK_BLOCK / SKINNY_STORE_TEAM) + threadIdx.x / SKINNY_STORE_TEAM;
  const bool live = i < total;
  if (!live) i = total - 1;   // (whole teams: every lane takes part in the exchanges below)
  const uint32_t p = (uint32_t)(i / a.t), q = (uint32_t)(i - (uint64_t)p * a.t);
  const float* part = a.acc + (uint64_t)blockIdx.y * a.chunks * total + i;
  float t[SKINNY_STORE_ROUNDS];
#pragma unroll
  for (int r = 0; r < SKINNY_STORE_ROUNDS; r++) {
    const uint32_t c = j + r * SKINNY_STORE_TEAM;
    t[r] = c < a.chunks ? part[(uint64_t)c * total] : 0.0f;
  }
  float v = 0.0f;
#pragma unroll
  for (int r = 0; r < SKINNY_STORE_ROUNDS; r++)
    if (j + r * SKINNY_STORE_TEAM < a.chunks) v += t[r];
#pragma unroll
  for (int d = SKINNY_STORE_TEAM / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, 64);
  if (live && j == 0) {
    T* C = (T*)a.c + (uint64_t)blockIdx.y * a.c_bs;
    C[(size_t)p * a.c_ps + (size_t)q * a.c_qs] = narrow<T>(v);
  }
}

// Two skinny launches that do not depend on each other (the thin fringes of a ragged product: a
// column strip and a row strip of C) as one: workgroups below `split` work on `a`, the others on
// `b`, each with the kernel its `kind` names and the block index it would have had on its own.
template <typename T> __device__ __forceinline__ void skinny_pair_impl(const hck_skinny_pair_args& p) {
  const bool first = blockIdx.x < p.split;
  const uint32_t block = first ? blockIdx.x : blockIdx.x - p.split;
  const uint32_t kind = first ? p.kind_a : p.kind_b;
  const hck_skinny_args& a = first ? p.a : p.b;
  if (block >= (first ? p.split : p.blocks_b)) return;
  switch (kind) {
    case HCK_SKINNY_K: skinny_k_impl<T, 4>(a, block); break;
    case HCK_SKINNY_P: skinny_p_impl<T, 4>(a, block); break;
    case HCK_SKINNY_PACK: skinny_pack_impl<T>(a, block); break;
    default: skinny_store_impl<T>(a, block); break;
  }
}

#define DEF_SKINNY(TN, T)                                                                          \
  HC_KERNEL void hc_gemm_skinny_k_##TN##_q4(hck_skinny_args a) { skinny_k_impl<T, 4>(a, blockIdx.x); } \
  HC_KERNEL void hc_gemm_skinny_p_##TN##_q4(hck_skinny_args a) { skinny_p_impl<T, 4>(a, blockIdx.x); } \
  HC_KERNEL void hc_gemm_skinny_pack_##TN(hck_skinny_args a) { skinny_pack_impl<T>(a, blockIdx.x); }   \
  HC_KERNEL void hc_gemm_skinny_store_##TN(hck_skinny_args a) { skinny_store_impl<T>(a, blockIdx.x); } \
  HC_KERNEL void hc_gemm_skinny_pair_##TN(hck_skinny_pair_args p) { skinny_pair_impl<T>(p); }
DEF_SKINNY(f16, half_t)
DEF_SKINNY(f32, float)
