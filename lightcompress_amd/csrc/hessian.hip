// GPTQ Hessian accumulation for gfx950:  H <- alpha*H + beta * X^T X
//
// Replaces GPTQ.add_batch (llmc/compression/quantization/gptq.py:253-295):
//   H *= n/(n+b);  n += b;  H += (sqrt(2/n) X.float())^T (sqrt(2/n) X.float())
// with alpha = n/(n+b), beta = 2/(n+b).  X is the layer input [T, K] (tokens x
// in_features, row-major, bf16 or fp16), H is [K, K] fp32.
//
// bf16 x bf16 products are exact in fp32, so a bf16-in / fp32-accumulate MFMA
// GEMM differs from the reference's fp32 SGEMM only in summation order.
//
// Shape of the kernel
//  * one 256-thread workgroup (4 waves, 2x2) per 256x128 tile of H; each wave
//    owns 128x64 = 4x2 blocks of v_mfma_f32_32x32x16 (128 accumulator
//    registers per lane).  Two workgroups fit a CU (registers and 56 KiB of
//    LDS each), so one tile's epilogue / barriers overlap the other's MFMAs;
//  * H is symmetric: only tiles that touch the upper triangle are computed
//    (the lower triangle is filled once, when H is consumed, by lcq_symmetrize);
//  * X is streamed 32 tokens at a time through double-buffered LDS in its
//    natural [token][feature] layout; the feature-major operand layout MFMA
//    needs (8 consecutive tokens per lane) is produced by the LDS transpose
//    read ds_read_b64_tr_b16, so no VALU shuffles are spent on the transpose;
//  * LDS rows are padded by 64 bytes so the four token rows a transpose read
//    touches fall into different banks.
#include "common.h"
#include "lcq_internal.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int TM = 256;                   // H tile rows (A operand: 256 features)
constexpr int TN = 128;                   // H tile columns (B operand: 128 features)
constexpr int BT = 32;                    // tokens per LDS stage
constexpr int PITCH_A = TM * 2 + 64;      // bytes per token row in LDS
constexpr int PITCH_B = TN * 2 + 64;
constexpr int BYTES_A = BT * PITCH_A, BYTES_B = BT * PITCH_B;
constexpr int STAGE_BYTES = BYTES_A + BYTES_B;

__device__ __forceinline__ s16x4 lds_tr_read(const char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p));
}

template <bool IS_BF16>
__device__ __forceinline__ f32x16 mfma(const s16x8& a, const s16x8& b, const f32x16& c) {
  if constexpr (IS_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Workgroup -> tile map.  Tile (ti, tj) covers rows [256 ti, +256) and columns [128 tj, +128);
// it is needed when it reaches the upper triangle: tj >= 2 ti.  Workgroups are handed to the 8
// XCDs round-robin (block b runs on XCD b % 8) and each XCD has its own L2, so every XCD gets a
// contiguous range of a tile order in which consecutive tiles form 4x8 super-blocks: the tiles
// an XCD works on at one time then share a handful of column stripes of X.
constexpr int SB_R = 4, SB_C = 8;
__device__ __forceinline__ bool decode_tile(int v, int ntr, int ntc, int& ti, int& tj) {
  for (int r0 = 0; r0 < ntr; r0 += SB_R) {
    const int r1 = min(r0 + SB_R, ntr);
    for (int c0 = (2 * r0 / SB_C) * SB_C; c0 < ntc; c0 += SB_C) {
      const int c1 = min(c0 + SB_C, ntc);
      int cnt = 0;
      for (int r = r0; r < r1; ++r) cnt += max(0, c1 - max(c0, 2 * r));
      if (v < cnt) {
        for (int r = r0; r < r1; ++r) {
          const int lo = max(c0, 2 * r), n = max(0, c1 - lo);
          if (v < n) { ti = r; tj = lo + v; return true; }
          v -= n;
        }
      }
      v -= cnt;
    }
  }
  return false;
}

// EDGE = false: K % 256 == 0 and T % 64 == 0, no bounds checks anywhere.
template <bool IS_BF16, bool EDGE>
__global__ __launch_bounds__(256, 2) void hessian_kernel(float* __restrict__ H, int K, const uint16_t* __restrict__ X,
                                                         int T, float alpha, float beta, int ntr, int ntc, int total) {
  __shared__ __attribute__((aligned(16))) char lds[2 * STAGE_BYTES];
  int ti = 0, tj = 0;
  {
    const int per_xcd = (total + 7) / 8;
    const int slot = blockIdx.x >> 3, xcd = blockIdx.x & 7;
    if (slot >= per_xcd || !decode_tile(xcd * per_xcd + slot, ntr, ntc, ti, tj)) return;
  }

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1;

  // global -> LDS staging.  A: 32 threads per 512-byte token row, 8 rows per pass, 4 passes;
  // B: 16 threads per 256-byte token row, 16 rows per pass, 2 passes.  Per-thread element offsets
  // inside a 32-token slab are 32-bit; the slab base is uniform.
  const int a_row = tid >> 5, a_c16 = tid & 31, b_row = tid >> 4, b_c16 = tid & 15;
  const int colA = ti * TM + a_c16 * 8, colB = tj * TN + b_c16 * 8;
  const bool okA = colA < K, okB = colB < K;
  uint32_t gofA[4], gofB[2];
  #pragma unroll
  for (int p = 0; p < 4; ++p) gofA[p] = (uint32_t)((p * 8 + a_row) * K + colA);
  #pragma unroll
  for (int p = 0; p < 2; ++p) gofB[p] = (uint32_t)((p * 16 + b_row) * K + colB);
  u32x4 sA0[4], sB0[2], sA1[4], sB1[2];     // two slabs of global loads stay in flight

  auto gload = [&](int t0, u32x4* sa, u32x4* sb) {
    const uint16_t* Xs = X + (int64_t)t0 * K;
    #pragma unroll
    for (int p = 0; p < 4; ++p) {
      if constexpr (EDGE) {
        sa[p] = u32x4{0, 0, 0, 0};
        if (okA && t0 + p * 8 + a_row < T) sa[p] = *(const u32x4*)(Xs + gofA[p]);
      } else sa[p] = *(const u32x4*)(Xs + gofA[p]);
    }
    #pragma unroll
    for (int p = 0; p < 2; ++p) {
      if constexpr (EDGE) {
        sb[p] = u32x4{0, 0, 0, 0};
        if (okB && t0 + p * 16 + b_row < T) sb[p] = *(const u32x4*)(Xs + gofB[p]);
      } else sb[p] = *(const u32x4*)(Xs + gofB[p]);
    }
  };
  char* const stA = lds + a_row * PITCH_A + a_c16 * 16;
  char* const stB = lds + BYTES_A + b_row * PITCH_B + b_c16 * 16;
  auto lstore = [&](int buf, const u32x4* sa, const u32x4* sb) {
    #pragma unroll
    for (int p = 0; p < 4; ++p) *(u32x4*)(stA + buf * STAGE_BYTES + p * 8 * PITCH_A) = sa[p];
    #pragma unroll
    for (int p = 0; p < 2; ++p) *(u32x4*)(stB + buf * STAGE_BYTES + p * 16 * PITCH_B) = sb[p];
  };

  // transpose-read lane addressing (see file header): a group of 16 lanes reads a
  // 4(token) x 16(feature) block; lane s supplies row s/4, features 4*(s%4)..+3 and
  // receives tokens 0..3 of feature s.
  const int L = lane & 15, g16 = (lane >> 4) & 1, kh = lane >> 5;
  const int fcol = (g16 * 16 + (L & 3) * 4) * 2, frow = kh * 8 + (L >> 2);
  const char* const rdA = lds + frow * PITCH_A + fcol + wr * 128 * 2;
  const char* const rdB = lds + BYTES_A + frow * PITCH_B + fcol + wc * 64 * 2;

  f32x16 acc[4][2];
  #pragma unroll
  for (int i = 0; i < 4; ++i)
    #pragma unroll
    for (int j = 0; j < 2; ++j)
      #pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  auto compute = [&](int buf) {
    const char* tA = rdA + buf * STAGE_BYTES;
    const char* tB = rdB + buf * STAGE_BYTES;
    #pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      s16x8 fa[4];
      #pragma unroll
      for (int b = 0; b < 4; ++b) {
        const s16x4 a0 = lds_tr_read(tA + ks * 16 * PITCH_A + b * 64);
        const s16x4 a1 = lds_tr_read(tA + ks * 16 * PITCH_A + 4 * PITCH_A + b * 64);
        fa[b] = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
      }
      #pragma unroll
      for (int j = 0; j < 2; ++j) {
        const s16x4 b0 = lds_tr_read(tB + ks * 16 * PITCH_B + j * 64);
        const s16x4 b1 = lds_tr_read(tB + ks * 16 * PITCH_B + 4 * PITCH_B + j * 64);
        const s16x8 fb = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
        #pragma unroll
        for (int i = 0; i < 4; ++i) acc[i][j] = mfma<IS_BF16>(fa[i], fb, acc[i][j]);
      }
    }
  };

  // slabs are processed in pairs; a ragged tail is zero-filled by the EDGE loads
  const int nsteps = ((T + 2 * BT - 1) / (2 * BT)) * 2;
  gload(0, sA0, sB0);
  gload(BT, sA1, sB1);
  lstore(0, sA0, sB0);
  __syncthreads();
  for (int s = 0; s + 2 < nsteps; s += 2) {
    gload((s + 2) * BT, sA0, sB0);
    compute(0);
    lstore(1, sA1, sB1);
    __syncthreads();
    gload((s + 3) * BT, sA1, sB1);
    compute(1);
    lstore(0, sA0, sB0);
    __syncthreads();
  }
  compute(0);
  lstore(1, sA1, sB1);
  __syncthreads();
  compute(1);

  // epilogue: accumulator register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32.
  // The old values of two 32-row bands (64 per lane) are fetched before any is used so the
  // loads overlap; alpha == 0 (first batch) never reads H.
  const int row_l = 4 * (lane >> 5), col_l = lane & 31;
  const int grow = ti * TM + wr * 128 + row_l, gcol = tj * TN + wc * 64 + col_l;
  float* const Hb = H + (int64_t)grow * K + gcol;
  const bool rmw = (alpha != 0.0f);
  #pragma unroll
  for (int ih = 0; ih < 2; ++ih) {
    float old[2][2][16];
    if (rmw) {
      #pragma unroll
      for (int i2 = 0; i2 < 2; ++i2)
        #pragma unroll
        for (int j = 0; j < 2; ++j)
          #pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int dr = (ih * 2 + i2) * 32 + 8 * (r >> 2) + (r & 3), dc = j * 32;
            const bool ok = !EDGE || ((grow + dr < K) && (gcol + dc < K));
            old[i2][j][r] = ok ? Hb[(int64_t)dr * K + dc] : 0.0f;
          }
    }
    #pragma unroll
    for (int i2 = 0; i2 < 2; ++i2)
      #pragma unroll
      for (int j = 0; j < 2; ++j)
        #pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int dr = (ih * 2 + i2) * 32 + 8 * (r >> 2) + (r & 3), dc = j * 32;
          const bool ok = !EDGE || ((grow + dr < K) && (gcol + dc < K));
          float v = beta * acc[ih * 2 + i2][j][r];
          if (rmw) v = alpha * old[i2][j][r] + v;
          if (ok) Hb[(int64_t)dr * K + dc] = v;
        }
  }
}

// fill the lower triangle from the upper one: H[j][i] = H[i][j], i < j
__global__ __launch_bounds__(256) void symmetrize_kernel(float* __restrict__ H, int K) {
  __shared__ float tile[32][33];
  const int bi = blockIdx.y, bj = blockIdx.x;
  if (bj < bi) return;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int r = ty; r < 32; r += 8) {
    const int64_t i = (int64_t)bi * 32 + r, j = (int64_t)bj * 32 + tx;
    tile[r][tx] = (i < K && j < K) ? H[i * K + j] : 0.0f;
  }
  __syncthreads();
  for (int r = ty; r < 32; r += 8) {
    const int64_t j = (int64_t)bj * 32 + r, i = (int64_t)bi * 32 + tx;     // writes H[j][i]
    if (i < K && j < K && j > i) H[j * K + i] = tile[tx][r];
  }
}

}  // namespace

extern "C" {

int lcq_hessian_accum(float* H, int64_t K, const void* X, int dtype, int64_t T, float alpha, float beta, void* stream) {
  if (!H || !X || K <= 0 || T < 0) return LCQ_EINVAL;
  if (K % 8 != 0 || K > (1 << 20) || T > 0x7fffffff) return LCQ_EINVAL;
  if (((uintptr_t)X % 16) != 0 || ((uintptr_t)H % 4) != 0) return LCQ_EALIGN;
  if (T == 0) return LCQ_OK;
  const int ntr = (int)((K + TM - 1) / TM), ntc = (int)((K + TN - 1) / TN);
  int64_t total = 0;
  for (int r = 0; r < ntr; ++r) total += (ntc - 2 * r > 0) ? (ntc - 2 * r) : 0;
  const int64_t grid = (total + 7) / 8 * 8;                       // 8 XCD queues of equal length
  hipStream_t st = (hipStream_t)stream;
  const bool edge = (K % TM != 0) || (T % (2 * BT) != 0);
  #define LCQ_HESS(BF, E) hessian_kernel<BF, E><<<dim3((unsigned)grid), dim3(256), 0, st>>>(H, (int)K, (const uint16_t*)X, (int)T, alpha, beta, ntr, ntc, (int)total)
  if (dtype == LCQ_BF16) { if (edge) LCQ_HESS(true, true); else LCQ_HESS(true, false); }
  else if (dtype == LCQ_F16) { if (edge) LCQ_HESS(false, true); else LCQ_HESS(false, false); }
  else return LCQ_EDTYPE;
  #undef LCQ_HESS
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_symmetrize(float* H, int64_t K, void* stream) {
  if (!H || K <= 0 || K > (1 << 20)) return LCQ_EINVAL;
  const unsigned nb = (unsigned)((K + 31) / 32);
  symmetrize_kernel<<<dim3(nb, nb), dim3(256), 0, (hipStream_t)stream>>>(H, (int)K);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
