// fp32 MFMA GEMM building block for gfx950 (v_mfma_f32_32x32x2f32), used by the
// blocked Cholesky / triangular-inverse chain and by GPTQ's deferred rank-128
// update.  Plain fp32 in, fp32 accumulate: no reduced-precision tricks, the
// GPTQ code agreement depends on it.
//
//   C[M x N] = alpha * A[M x Kc] * op(B) + beta * C
//     A is row-major with the contraction index contiguous;
//     B_T  : B is [N x Kc] row-major (contraction contiguous)   -> A * B^T
//     !B_T : B is [Kc x N] row-major (output column contiguous) -> A * B
//
// One 256-thread workgroup per 128x128 tile of C, four waves of 64x64 (2x2 MFMA
// blocks each), contraction staged 32 at a time through LDS.  LDS pitches are
// chosen so that the 32 lanes that read one operand column hit 32 banks.
//
// Triangular structure is exploited by clipping the contraction range per
// tile (GEMM_K_FROM_N / GEMM_K_TO_M) and by skipping tiles above the diagonal
// (GEMM_LOWER_TILES).  Batched launches take per-problem offsets from
// GemmBatch (blockIdx.z).
#pragma once
#include <atomic>
#include <type_traits>

#include "common.h"

namespace lcq {

typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int GT = 128;            // C tile edge
constexpr int GK = 32;             // contraction slab
constexpr int GPA = GK + 1;        // pitch of a [rows][k] operand tile (floats)
constexpr int GPB = GT + 32;       // pitch of a [k][cols] operand tile (floats)

enum : int {
  GEMM_LOWER_TILES = 1,   // only tiles with n0 <= m0 (C symmetric / lower triangular)
  GEMM_K_FROM_N = 2,      // B is lower triangular [k][n]: terms with k < n0 vanish
  GEMM_K_TO_M = 4,        // A is lower triangular [m][k]: terms with k >= m0 + GT vanish
  GEMM_XCD_ORDER = 8,     // (set by launch_gemm) workgroups take their tile from the XCD-contiguous super-block order
};

struct GemmProblem {
  const float* A; const float* B; float* C;
  int M, N, Kc;
  int lda, ldb, ldc;
};

constexpr int GEMM_MAX_BATCH = 64;
struct GemmBatch {
  // element offsets added to the base pointers, and per-problem sizes
  long long offA[GEMM_MAX_BATCH], offB[GEMM_MAX_BATCH], offC[GEMM_MAX_BATCH];
  int M[GEMM_MAX_BATCH], N[GEMM_MAX_BATCH], Kc[GEMM_MAX_BATCH];
};

template <bool B_T, int TM = GT, bool DEEP = false>
__device__ __forceinline__ void gemm_tile(const float* A, int lda, const float* B, int ldb,
                                          float* C, int ldc, int M, int N, int Kc, float alpha, float beta,
                                          int flags, int m0, int n0, float* sA, float* sB) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // waves are 2 x 2 over the TM x 128 tile; the 32-row tile puts its four waves side by side, 32 columns each
  constexpr bool FLAT = TM == 32;
  const int wr = FLAT ? 0 : wave >> 1, wc = FLAT ? wave : wave & 1;
  constexpr int MI = FLAT ? 1 : TM / 64;       // 32-row MFMA blocks per wave
  constexpr int NJ = FLAT ? 1 : 2;             // 32-column MFMA blocks per wave
  constexpr int WM = FLAT ? 32 : TM / 2;       // rows per wave
  constexpr int WN = 32 * NJ;                  // columns per wave
  constexpr int AP = TM / 32;                  // float4 of the A slab per thread

  int kb = 0, ke = Kc;
  if (flags & GEMM_K_FROM_N) kb = (n0 / GK) * GK;
  if (flags & GEMM_K_TO_M) ke = min(Kc, m0 + TM);

  f32x16 acc[MI][NJ];
  #pragma unroll
  for (int i = 0; i < MI; ++i)
    #pragma unroll
    for (int j = 0; j < NJ; ++j)
      #pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // staging registers: A tile 128 x 32 floats = 1024 float4 -> 4 per thread; B likewise.
  // DEEP (contraction of at most 4 slabs): one register set per slab, so that all global loads of the tile are in
  // flight at once; with one set the tile pays one memory latency per slab, which is most of a rank-128 launch.
  constexpr int NS = DEEP ? 4 : 1;
  f32x4 ra[NS][AP], rb[NS][4];
  auto gload = [&](int k0, auto slot_tag) {
    constexpr int sl = decltype(slot_tag)::value;
    #pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int idx = p * 256 + tid;
      if (p < AP) {   // A: row = idx / 8, k4 = idx % 8
        const int r = idx >> 3, k = k0 + (idx & 7) * 4;
        const int gm = m0 + r;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (gm < M) {
          const float* p0 = A + (long long)gm * lda + k;
          if (k + 3 < ke && ((((uintptr_t)p0) & 15) == 0)) v = *(const f32x4*)p0;
          else {
            #pragma unroll
            for (int e = 0; e < 4; ++e) if (k + e < ke) v[e] = p0[e];
          }
        }
        ra[sl][p] = v;
      }
      if constexpr (B_T) {   // B[n][k]: same shape as A
        const int r = idx >> 3, k = k0 + (idx & 7) * 4;
        const int gn = n0 + r;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (gn < N) {
          const float* p0 = B + (long long)gn * ldb + k;
          if (k + 3 < ke && ((((uintptr_t)p0) & 15) == 0)) v = *(const f32x4*)p0;
          else {
            #pragma unroll
            for (int e = 0; e < 4; ++e) if (k + e < ke) v[e] = p0[e];
          }
        }
        rb[sl][p] = v;
      } else {               // B[k][n]: k = idx / 32, n4 = idx % 32
        const int k = k0 + (idx >> 5), n = n0 + (idx & 31) * 4;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (k < ke) {
          const float* p0 = B + (long long)k * ldb + n;
          if (n + 3 < N && ((((uintptr_t)p0) & 15) == 0)) v = *(const f32x4*)p0;
          else {
            #pragma unroll
            for (int e = 0; e < 4; ++e) if (n + e < N) v[e] = p0[e];
          }
        }
        rb[sl][p] = v;
      }
    }
  };
  auto lstore = [&](auto slot_tag) {
    constexpr int sl = decltype(slot_tag)::value;
    #pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int idx = p * 256 + tid;
      if (p < AP) {
        const int r = idx >> 3, k = (idx & 7) * 4;
        #pragma unroll
        for (int e = 0; e < 4; ++e) sA[r * GPA + k + e] = ra[sl][p][e];
      }
      if constexpr (B_T) {
        const int r = idx >> 3, k = (idx & 7) * 4;
        #pragma unroll
        for (int e = 0; e < 4; ++e) sB[r * GPA + k + e] = rb[sl][p][e];
      } else {
        const int k = idx >> 5, n = (idx & 31) * 4;
        *(f32x4*)(sB + k * GPB + n) = rb[sl][p];
      }
    }
  };

  const int lm = lane & 31, lk = lane >> 5;
  auto compute = [&]() {
    #pragma unroll
    for (int kk = 0; kk < GK; kk += 2) {
      float a[MI], b[NJ];
      #pragma unroll
      for (int i = 0; i < MI; ++i) a[i] = sA[(wr * WM + i * 32 + lm) * GPA + kk + lk];
      #pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if constexpr (B_T) b[j] = sB[(wc * WN + j * 32 + lm) * GPA + kk + lk];
        else b[j] = sB[(kk + lk) * GPB + wc * WN + j * 32 + lm];
      }
      #pragma unroll
      for (int i = 0; i < MI; ++i)
        #pragma unroll
        for (int j = 0; j < NJ; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  };
  using S0 = std::integral_constant<int, 0>;
  float oldc[DEEP ? MI : 1][NJ][16];                       // DEEP: the old C values, fetched with the operands
  if constexpr (DEEP) {
    gload(kb, S0{});
    if (kb + GK < ke) gload(kb + GK, std::integral_constant<int, 1>{});
    if (kb + 2 * GK < ke) gload(kb + 2 * GK, std::integral_constant<int, 2>{});
    if (kb + 3 * GK < ke) gload(kb + 3 * GK, std::integral_constant<int, 3>{});
    if (beta != 0.0f) {
      #pragma unroll
      for (int i = 0; i < MI; ++i)
        #pragma unroll
        for (int j = 0; j < NJ; ++j) {
          const int gn = n0 + wc * WN + j * 32 + lm;
          const int gm0 = m0 + wr * WM + i * 32 + 4 * lk;
          const float* p0 = C + (long long)gm0 * ldc + gn;
          #pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int dm = 8 * (r >> 2) + (r & 3);
            oldc[i][j][r] = (gm0 + dm < M && gn < N) ? p0[(long long)dm * ldc] : 0.0f;
          }
        }
    }
    __syncthreads(); lstore(S0{}); __syncthreads(); compute();
    if (kb + GK < ke) { __syncthreads(); lstore(std::integral_constant<int, 1>{}); __syncthreads(); compute(); }
    if (kb + 2 * GK < ke) { __syncthreads(); lstore(std::integral_constant<int, 2>{}); __syncthreads(); compute(); }
    if (kb + 3 * GK < ke) { __syncthreads(); lstore(std::integral_constant<int, 3>{}); __syncthreads(); compute(); }
  } else {
    if (kb < ke) gload(kb, S0{});
    for (int k0 = kb; k0 < ke; k0 += GK) {
      __syncthreads();                       // previous slab fully consumed
      lstore(S0{});
      __syncthreads();
      if (k0 + GK < ke) gload(k0 + GK, S0{});   // next slab in flight while this one is multiplied
      compute();
    }
  }

  // accumulator register r of lane l: row 8*(r/4) + 4*(l/32) + r%4, column l%32.
  // With beta != 0 all 16 old values of a 32x32 block are fetched before the first store: interleaved, every load
  // would have to wait behind the store in front of it (they may alias), 64 memory latencies in a row per tile.
  #pragma unroll
  for (int i = 0; i < MI; ++i)
    #pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int gn = n0 + wc * WN + j * 32 + lm;
      const int gm0 = m0 + wr * WM + i * 32 + 4 * lk;
      float* p0 = C + (long long)gm0 * ldc + gn;
      float old[16];
      if (beta != 0.0f) {
        #pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int dm = 8 * (r >> 2) + (r & 3);
          if constexpr (DEEP) old[r] = oldc[i][j][r];
          else old[r] = (gm0 + dm < M && gn < N) ? p0[(long long)dm * ldc] : 0.0f;
        }
      }
      #pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int dm = 8 * (r >> 2) + (r & 3);
        if (gm0 + dm < M && gn < N) {
          const float v = alpha * acc[i][j][r];
          p0[(long long)dm * ldc] = (beta != 0.0f) ? (beta * old[r] + v) : v;
        }
      }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The same product on the bf16 matrix pipe: every fp32 operand is split into three bf16 planes
//   x = hi + mid + lo,  hi = bf16(x), mid = bf16(x - hi), lo = bf16(x - hi - mid)        (both differences exact)
// which carry 24 bits of x between them, and a product a * b is accumulated (fp32, inside the MFMA) as the six
// partial products of weight >= 2^-16:  lo*hi + hi*lo + mid*mid + mid*hi + hi*mid + hi*hi.  The dropped terms
// (mid*lo, lo*mid, lo*lo) are below 2^-24 of the product - the rounding of an fp32 multiply - so the result is as
// accurate as the fp32 pipe's, at 16 / 6 times its rate (v_mfma_f32_32x32x16_bf16 against v_mfma_f32_32x32x2f32).
// Used for the launches that fill the chip (more than one 128x128 tile per CU); small launches stay on the fp32 pipe.
// LDS: per operand three planes of [128 rows][32 k] bf16 (64-byte rows, 16-byte chunks XOR-swizzled by the row) or, for B given as [k][n], of [32 k][128 n] (row pitch 320 B) read through the transposing
// ds_read_b64_tr_b16 (a 16-lane group addresses 4 k-rows x 16 columns and receives 4 k-values of one column each).
typedef __attribute__((ext_vector_type(8))) __bf16 s3_bf16x8;
typedef __attribute__((ext_vector_type(4))) short s3_s16x4;
typedef __attribute__((ext_vector_type(2))) float s3_f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 s3_bf16x2;
constexpr int S3_P = 32;              // bf16 per row of a [row][k] plane: 64 bytes, four 16-byte chunks, XOR-swizzled
constexpr int S3_PN = 160;            // bf16 per row of a [k][n] plane
constexpr int S3_PLANE = GK * S3_PN;  // 5120 bf16 per plane (a [row][k] plane needs 4096 of them)
// chunk q (8 k-values) of row r sits at chunk q ^ ((r >> 2) & 3): 16 consecutive rows reading the same q hit 16
// different bank quads, and the 4 rows x 64 bytes of a store instruction's 32 lanes cover all 64 banks once
__device__ __forceinline__ int s3_rk(int row, int q) { return row * S3_P + ((q ^ ((row >> 2) & 3)) << 3); }

__device__ __forceinline__ uint32_t s3_pack(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(s3_f32x2{a, b}, s3_bf16x2));
}
// four fp32 -> 4 bf16 (8 bytes) per plane
__device__ __forceinline__ void s3_split(const f32x4& v, u32x2& hi, u32x2& mid, u32x2& lo) {
  #pragma unroll
  for (int h = 0; h < 2; ++h) {
    const float a = v[2 * h], b = v[2 * h + 1];
    const uint32_t ph = s3_pack(a, b);
    const float ra = a - u2f(ph << 16), rb = b - u2f(ph & 0xffff0000u);
    const uint32_t pm = s3_pack(ra, rb);
    const float sa = ra - u2f(pm << 16), sb = rb - u2f(pm & 0xffff0000u);
    hi[h] = ph; mid[h] = pm; lo[h] = s3_pack(sa, sb);
  }
}

template <bool B_T>
__device__ __forceinline__ void gemm_tile_s3(const float* A, int lda, const float* B, int ldb, float* C, int ldc, int M, int N,
                                             int Kc, float alpha, float beta, int flags, int m0, int n0, uint16_t* sA,
                                             uint16_t* sB) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1;
  int kb = 0, ke = Kc;
  if (flags & GEMM_K_FROM_N) kb = (n0 / GK) * GK;
  if (flags & GEMM_K_TO_M) ke = min(Kc, m0 + GT);

  f32x16 acc[2][2];
  #pragma unroll
  for (int i = 0; i < 2; ++i)
    #pragma unroll
    for (int j = 0; j < 2; ++j)
      #pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  f32x4 ra[4], rb[4];
  auto gload = [&](int k0) {
    #pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int idx = p * 256 + tid;
      {
        const int r = idx >> 3, k = k0 + (idx & 7) * 4, gm = m0 + r;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (gm < M) {
          const float* p0 = A + (long long)gm * lda + k;
          if (k + 3 < ke && ((((uintptr_t)p0) & 15) == 0)) v = *(const f32x4*)p0;
          else {
            #pragma unroll
            for (int e = 0; e < 4; ++e) if (k + e < ke) v[e] = p0[e];
          }
        }
        ra[p] = v;
      }
      if constexpr (B_T) {
        const int r = idx >> 3, k = k0 + (idx & 7) * 4, gn = n0 + r;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (gn < N) {
          const float* p0 = B + (long long)gn * ldb + k;
          if (k + 3 < ke && ((((uintptr_t)p0) & 15) == 0)) v = *(const f32x4*)p0;
          else {
            #pragma unroll
            for (int e = 0; e < 4; ++e) if (k + e < ke) v[e] = p0[e];
          }
        }
        rb[p] = v;
      } else {
        const int k = k0 + (idx >> 5), n = n0 + (idx & 31) * 4;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (k < ke) {
          const float* p0 = B + (long long)k * ldb + n;
          if (n + 3 < N && ((((uintptr_t)p0) & 15) == 0)) v = *(const f32x4*)p0;
          else {
            #pragma unroll
            for (int e = 0; e < 4; ++e) if (n + e < N) v[e] = p0[e];
          }
        }
        rb[p] = v;
      }
    }
  };
  auto lstore = [&]() {
    #pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int idx = p * 256 + tid;
      u32x2 h, m, l;
      s3_split(ra[p], h, m, l);
      const int oa = s3_rk(idx >> 3, (idx & 7) >> 1) + (idx & 1) * 4;
      *(u32x2*)(sA + oa) = h; *(u32x2*)(sA + S3_PLANE + oa) = m; *(u32x2*)(sA + 2 * S3_PLANE + oa) = l;
      s3_split(rb[p], h, m, l);
      const int ob = B_T ? oa : (idx >> 5) * S3_PN + (idx & 31) * 4;
      *(u32x2*)(sB + ob) = h; *(u32x2*)(sB + S3_PLANE + ob) = m; *(u32x2*)(sB + 2 * S3_PLANE + ob) = l;
    }
  };
  const int lm = lane & 31, lk = lane >> 5;
  const int L = lane & 15, g16 = (lane >> 4) & 1;
  auto compute = [&]() {
    #pragma unroll
    for (int ks = 0; ks < GK / 16; ++ks) {
      s3_bf16x8 fa[2][3], fb[2][3];
      #pragma unroll
      for (int i = 0; i < 2; ++i)
        #pragma unroll
        for (int pl = 0; pl < 3; ++pl)
          fa[i][pl] = *(const s3_bf16x8*)(sA + pl * S3_PLANE + s3_rk(wr * 64 + i * 32 + lm, ks * 2 + lk));
      #pragma unroll
      for (int j = 0; j < 2; ++j)
        #pragma unroll
        for (int pl = 0; pl < 3; ++pl) {
          if constexpr (B_T) {
            fb[j][pl] = *(const s3_bf16x8*)(sB + pl * S3_PLANE + s3_rk(wc * 64 + j * 32 + lm, ks * 2 + lk));
          } else {
            const uint16_t* q = sB + pl * S3_PLANE + (ks * 16 + lk * 8 + (L >> 2)) * S3_PN + wc * 64 + j * 32 + g16 * 16 + (L & 3) * 4;
            const s3_s16x4 b0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s3_s16x4 __attribute__((address_space(3)))*)(q));
            const s3_s16x4 b1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s3_s16x4 __attribute__((address_space(3)))*)(q + 4 * S3_PN));
            fb[j][pl] = __builtin_bit_cast(s3_bf16x8, __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7));
          }
        }
      #pragma unroll
      for (int i = 0; i < 2; ++i)
        #pragma unroll
        for (int j = 0; j < 2; ++j) {
          f32x16 c = acc[i][j];
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i][2], fb[j][0], c, 0, 0, 0);      // small terms first
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i][0], fb[j][2], c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i][1], fb[j][1], c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i][1], fb[j][0], c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i][0], fb[j][1], c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i][0], fb[j][0], c, 0, 0, 0);
          acc[i][j] = c;
        }
    }
  };
  // Tiles that lie inside the matrices with 16-byte aligned rows (nearly all of a large launch) fetch a full slab
  // with eight unconditional 16-byte loads from per-thread pointers; the general path above costs ~15 instructions
  // per load in bounds and alignment checks, more than the matrix pipe leaves room for at this rate.
  const bool interior = (m0 + GT <= M) && (n0 + GT <= N) && (lda % 4 == 0) && (ldb % 4 == 0) &&
                        (((uintptr_t)A | (uintptr_t)B) % 16 == 0) && (kb % 4 == 0);
  const float* pa[4]; const float* pb[4];
  #pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int idx = p * 256 + tid;
    pa[p] = A + (long long)(m0 + (idx >> 3)) * lda + (idx & 7) * 4;
    pb[p] = B_T ? B + (long long)(n0 + (idx >> 3)) * ldb + (idx & 7) * 4
                : B + (long long)(idx >> 5) * ldb + n0 + (idx & 31) * 4;
  }
  auto gload_fast = [&](int k0) {
    #pragma unroll
    for (int p = 0; p < 4; ++p) {
      ra[p] = *(const f32x4*)(pa[p] + k0);
      rb[p] = *(const f32x4*)(pb[p] + (B_T ? (long long)k0 : (long long)k0 * ldb));
    }
  };
  auto fetch = [&](int k0) {
    if (interior && k0 + GK <= ke) gload_fast(k0); else gload(k0);
  };
  if (kb < ke) fetch(kb);
  for (int k0 = kb; k0 < ke; k0 += GK) {
    __syncthreads();                       // previous slab fully consumed
    lstore();
    __syncthreads();
    if (k0 + GK < ke) fetch(k0 + GK);      // next slab in flight while this one is multiplied
    compute();
  }
  // accumulator register r of lane l: row 8*(r/4) + 4*(l/32) + r%4, column l%32 (the fp32 kernel's epilogue)
  #pragma unroll
  for (int i = 0; i < 2; ++i)
    #pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int gn = n0 + wc * 64 + j * 32 + lm;
      const int gm0 = m0 + wr * 64 + i * 32 + 4 * lk;
      float* p0 = C + (long long)gm0 * ldc + gn;
      float old[16];
      if (beta != 0.0f) {
        #pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int dm = 8 * (r >> 2) + (r & 3);
          old[r] = (gm0 + dm < M && gn < N) ? p0[(long long)dm * ldc] : 0.0f;
        }
      }
      #pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int dm = 8 * (r >> 2) + (r & 3);
        if (gm0 + dm < M && gn < N) {
          const float v = alpha * acc[i][j][r];
          p0[(long long)dm * ldc] = (beta != 0.0f) ? (beta * old[r] + v) : v;
        }
      }
    }
}

// Workgroup -> tile for the big launches.  Workgroups go to the 8 XCDs round-robin (block b runs on XCD b % 8) and
// every XCD has its own 4 MB L2, while a 128 x 128 tile reads 2 x 128 x Kc x 4 bytes of operands: in the plain
// row-major order the tiles an XCD holds at one time share one operand and stream the other from beyond L2
// (4.4 TB/s at 140 TFLOP/s with Kc = 512, served by the Infinity Cache: worth 2 % of the chain).  Here XCD x works through the contiguous range [x * per, (x + 1) * per)
// of a tile order made of square super-blocks (SB x SB tiles, row-major inside and between them), so what it holds
// at one time draws on SB + SB operand tiles instead of 1 + SB * SB.
template <int SB>
__device__ __forceinline__ void s3_tile_of(int gx, int gy, int& tm, int& tn) {
  const int total = gx * gy, base = total >> 3, rem = total & 7;
  const int lin = blockIdx.y * gx + blockIdx.x, x = lin & 7;
  int v = x * base + min(x, rem) + (lin >> 3);            // XCD x holds base (+1 for x < rem) consecutive tiles
  const int sr = v / (SB * gx), r0 = sr * SB, nr = min(SB, gy - r0);      // super-row: nr tile rows x gx tile columns
  v -= r0 * gx;
  const int sc = min(v / (nr * SB), (gx - 1) / SB), c0 = sc * SB, nc = min(SB, gx - c0);
  v -= sc * nr * SB;
  tm = r0 + v / nc;
  tn = c0 + v % nc;
}

template <bool B_T>
__global__ __launch_bounds__(256, 2) void gemm_s3_kernel(GemmProblem g, float alpha, float beta, int flags) {
  __shared__ __attribute__((aligned(16))) uint16_t sA[3 * S3_PLANE];
  __shared__ __attribute__((aligned(16))) uint16_t sB[3 * S3_PLANE];
  int tm = blockIdx.y, tn = blockIdx.x;
  if (flags & GEMM_XCD_ORDER) s3_tile_of<8>(gridDim.x, gridDim.y, tm, tn);
  const int m0 = tm * GT, n0 = tn * GT;
  if ((flags & GEMM_LOWER_TILES) && n0 >= m0 + GT) return;
  gemm_tile_s3<B_T>(g.A, g.lda, g.B, g.ldb, g.C, g.ldc, g.M, g.N, g.Kc, alpha, beta, flags, m0, n0, sA, sB);
}

// The lower triangle of a square launch whose side is a whole number of 4 x 4 super-blocks (the deep trailing updates
// of the Cholesky chain): a 1-D grid over the super-blocks on and below the diagonal only, 16 tiles each, in the
// XCD-contiguous order described above.  (A 2-D grid launches as many workgroups again that return at once.)
template <bool B_T>
__global__ __launch_bounds__(256, 2) void gemm_s3_lower_kernel(GemmProblem g, float alpha, float beta, int flags, int nsb) {
  __shared__ __attribute__((aligned(16))) uint16_t sA[3 * S3_PLANE];
  __shared__ __attribute__((aligned(16))) uint16_t sB[3 * S3_PLANE];
  const int total = 16 * (nsb * (nsb + 1) / 2);            // a multiple of 8: the grid
  const int lin = blockIdx.x;
  const int v = (lin & 7) * (total >> 3) + (lin >> 3);
  const int sb = v >> 4, t = v & 15;
  int sr = (int)((__builtin_sqrtf(8.0f * (float)sb + 1.0f) - 1.0f) * 0.5f);
  while (sr * (sr + 1) / 2 > sb) --sr;
  while ((sr + 1) * (sr + 2) / 2 <= sb) ++sr;
  const int sc = sb - sr * (sr + 1) / 2;
  const int m0 = (sr * 4 + (t >> 2)) * GT, n0 = (sc * 4 + (t & 3)) * GT;
  if (n0 >= m0 + GT) return;
  gemm_tile_s3<B_T>(g.A, g.lda, g.B, g.ldb, g.C, g.ldc, g.M, g.N, g.Kc, alpha, beta, flags, m0, n0, sA, sB);
}

template <bool B_T>
__global__ __launch_bounds__(256, 2) void gemm_s3_batched_kernel(const float* A, int lda, const float* B, int ldb, float* C,
                                                                 int ldc, GemmBatch bt, float alpha, float beta, int flags) {
  __shared__ __attribute__((aligned(16))) uint16_t sA[3 * S3_PLANE];
  __shared__ __attribute__((aligned(16))) uint16_t sB[3 * S3_PLANE];
  const int z = blockIdx.z;
  const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
  if (m0 >= bt.M[z] || n0 >= bt.N[z]) return;
  gemm_tile_s3<B_T>(A + bt.offA[z], lda, B + bt.offB[z], ldb, C + bt.offC[z], ldc, bt.M[z], bt.N[z], bt.Kc[z], alpha, beta,
                    flags, m0, n0, sA, sB);
}

// 1 (default): launches of more than 256 tiles run on the bf16 matrix pipe (three-way split operands); 0: fp32 pipe only
extern std::atomic<int> g_gemm_split;

// TM = 128, 64 or 32 rows of C per workgroup.  The short tiles are for launches that would not give every CU a
// 128-row tile (rank-128 updates and panel solves of the blocked chains): twice the workgroups, half the serial
// MFMA work in each.
template <bool B_T, int TM, bool DEEP = false>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmProblem g, float alpha, float beta, int flags) {
  __shared__ float sA[TM * GPA];
  __shared__ float sB[B_T ? GT * GPA : GK * GPB];
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * GT;
  if ((flags & GEMM_LOWER_TILES) && n0 >= m0 + TM) return;
  gemm_tile<B_T, TM, DEEP>(g.A, g.lda, g.B, g.ldb, g.C, g.ldc, g.M, g.N, g.Kc, alpha, beta, flags, m0, n0, sA, sB);
}

template <bool B_T>
__global__ __launch_bounds__(256) void gemm_f32_batched_kernel(const float* A, int lda, const float* B, int ldb, float* C,
                                                               int ldc, GemmBatch bt, float alpha, float beta, int flags) {
  __shared__ float sA[GT * GPA];
  __shared__ float sB[B_T ? GT * GPA : GK * GPB];
  const int z = blockIdx.z;
  const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
  if (m0 >= bt.M[z] || n0 >= bt.N[z]) return;
  gemm_tile<B_T>(A + bt.offA[z], lda, B + bt.offB[z], ldb, C + bt.offC[z], ldc, bt.M[z], bt.N[z], bt.Kc[z], alpha, beta,
                 flags, m0, n0, sA, sB);
}

template <bool B_T>
inline void launch_gemm(const GemmProblem& g, float alpha, float beta, int flags, hipStream_t st) {
  if (g.M <= 0 || g.N <= 0) return;
  const unsigned gx = (unsigned)((g.N + GT - 1) / GT), gy = (unsigned)((g.M + GT - 1) / GT);
  const bool split = g_gemm_split.load(std::memory_order_relaxed) != 0;
  // the bf16 pipe also pays for launches of at most one tile per CU when the contraction is long: a tile's time is
  // its serial chain of slabs, 2.7x shorter there
  if (split && (long long)gx * gy >= 64 && (long long)gx * gy <= 256 && g.Kc >= 256)
    gemm_s3_kernel<B_T><<<dim3(gx, gy), dim3(256), 0, st>>>(g, alpha, beta, flags);
  // at most 128 of the 64-row tiles: 32-row tiles instead, twice the CUs and half the serial MFMA work in each (a
  // 64 x 128 tile with a 128-deep contraction is 3.9 us of fp32 MFMA on its CU; K = 4096 chain 2.14 -> 1.99 ms)
  else if ((long long)gx * ((g.M + 63) / 64) <= 128 && g.Kc > 0 && g.Kc <= 4 * GK &&
           !(flags & (GEMM_K_FROM_N | GEMM_K_TO_M)))
    gemm_f32_kernel<B_T, 32, true><<<dim3(gx, (unsigned)((g.M + 31) / 32)), dim3(256), 0, st>>>(g, alpha, beta, flags);
  else if ((long long)gx * gy <= 256 && g.Kc > 0 && g.Kc <= 4 * GK && !(flags & (GEMM_K_FROM_N | GEMM_K_TO_M)))
    gemm_f32_kernel<B_T, 64, true><<<dim3(gx, (unsigned)((g.M + 63) / 64)), dim3(256), 0, st>>>(g, alpha, beta, flags);
  else if ((long long)gx * gy <= 256)
    gemm_f32_kernel<B_T, 64><<<dim3(gx, (unsigned)((g.M + 63) / 64)), dim3(256), 0, st>>>(g, alpha, beta, flags);
  else if (split && (flags & GEMM_LOWER_TILES) && g.M == g.N && g.M % (4 * GT) == 0) {
    const int nsb = g.M / (4 * GT), total = 16 * (nsb * (nsb + 1) / 2);
    gemm_s3_lower_kernel<B_T><<<dim3((unsigned)total), dim3(256), 0, st>>>(g, alpha, beta, flags, nsb);
  } else if (split)
    gemm_s3_kernel<B_T><<<dim3(gx, gy), dim3(256), 0, st>>>(g, alpha, beta, flags | GEMM_XCD_ORDER);
  else
    gemm_f32_kernel<B_T, GT><<<dim3(gx, gy), dim3(256), 0, st>>>(g, alpha, beta, flags);
}

}  // namespace lcq
