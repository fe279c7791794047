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
//  * one 256-thread workgroup (4 waves, 2x2) per 256x256 tile of H; each wave
//    owns 128x128 = 4x4 blocks of v_mfma_f32_32x32x16 (256 accumulator
//    registers per lane);
//  * H is symmetric: only tiles on or above the diagonal are computed (the
//    lower triangle is filled once, when H is consumed, by lcq_symmetrize);
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

constexpr int TILE = 256;                 // H tile edge
constexpr int BT = 32;                    // tokens per LDS stage
constexpr int PITCH = TILE * 2 + 64;      // bytes per token row in LDS
constexpr int TILE_BYTES = BT * PITCH;    // one operand tile, one stage

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

// tile index -> (ti, tj) with ti <= tj, row-major over the upper triangle
__device__ __forceinline__ void decode_upper(int idx, int nt, int& ti, int& tj) {
  int i = 0, rowlen = nt;
  while (idx >= rowlen) { idx -= rowlen; ++i; --rowlen; }
  ti = i; tj = i + idx;
}

template <bool IS_BF16>
__global__ __launch_bounds__(256) void hessian_kernel(float* __restrict__ H, int K, const uint16_t* __restrict__ X,
                                                      int T, float alpha, float beta, int nt) {
  __shared__ __attribute__((aligned(16))) char lds[2 * 2 * TILE_BYTES];
  int ti, tj;
  decode_upper(blockIdx.x, nt, ti, tj);
  const bool diag = (ti == tj);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1;

  // global -> LDS staging: 32 threads cover one 512-byte token row, 8 rows per pass
  const int ld_row = tid >> 5, ld_c16 = tid & 31;
  const int64_t colA = (int64_t)ti * TILE + ld_c16 * 8, colB = (int64_t)tj * TILE + ld_c16 * 8;
  const bool okA = colA < K, okB = colB < K;
  u32x4 stA[4], stB[4];

  auto gload = [&](int t0) {
    #pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int t = t0 + p * 8 + ld_row;
      const bool rok = t < T;
      stA[p] = (rok && okA) ? *(const u32x4*)(X + (int64_t)t * K + colA) : u32x4{0, 0, 0, 0};
      if (!diag) stB[p] = (rok && okB) ? *(const u32x4*)(X + (int64_t)t * K + colB) : u32x4{0, 0, 0, 0};
    }
  };
  auto lstore = [&](int buf) {
    char* a = lds + (buf * 2 + 0) * TILE_BYTES + ld_row * PITCH + ld_c16 * 16;
    char* b = lds + (buf * 2 + 1) * TILE_BYTES + ld_row * PITCH + ld_c16 * 16;
    #pragma unroll
    for (int p = 0; p < 4; ++p) {
      *(u32x4*)(a + p * 8 * PITCH) = stA[p];
      if (!diag) *(u32x4*)(b + p * 8 * PITCH) = stB[p];
    }
  };

  // transpose-read lane addressing (see file header): a group of 16 lanes reads a
  // 4(token) x 16(feature) block; lane s supplies row s/4, features 4*(s%4)..+3 and
  // receives tokens 0..3 of feature s.
  const int L = lane & 15, g16 = (lane >> 4) & 1, kh = lane >> 5;
  const int frag_off = (kh * 8 + (L >> 2)) * PITCH + (g16 * 16 + (L & 3) * 4) * 2;
  const int offA = frag_off + wr * 128 * 2, offB = frag_off + wc * 128 * 2;

  f32x16 acc[4][4];
  #pragma unroll
  for (int i = 0; i < 4; ++i)
    #pragma unroll
    for (int j = 0; j < 4; ++j)
      #pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int nsteps = (T + BT - 1) / BT;
  gload(0);
  lstore(0);
  __syncthreads();
  for (int s = 0; s < nsteps; ++s) {
    const int buf = s & 1;
    if (s + 1 < nsteps) gload((s + 1) * BT);
    const char* tA = lds + (buf * 2 + 0) * TILE_BYTES + offA;
    const char* tB = lds + (buf * 2 + (diag ? 0 : 1)) * TILE_BYTES + offB;
    #pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      s16x8 fa[4], fb[4];
      #pragma unroll
      for (int b = 0; b < 4; ++b) {
        const s16x4 a0 = lds_tr_read(tA + ks * 16 * PITCH + b * 64);
        const s16x4 a1 = lds_tr_read(tA + ks * 16 * PITCH + 4 * PITCH + b * 64);
        fa[b] = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
        const s16x4 b0 = lds_tr_read(tB + ks * 16 * PITCH + b * 64);
        const s16x4 b1 = lds_tr_read(tB + ks * 16 * PITCH + 4 * PITCH + b * 64);
        fb[b] = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
      }
      #pragma unroll
      for (int i = 0; i < 4; ++i)
        #pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mfma<IS_BF16>(fa[i], fb[j], acc[i][j]);
    }
    if (s + 1 < nsteps) lstore(buf ^ 1);
    __syncthreads();
  }

  // epilogue: accumulator register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32
  const int row_l = 4 * (lane >> 5), col_l = lane & 31;
  #pragma unroll
  for (int i = 0; i < 4; ++i) {
    #pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t gj = (int64_t)tj * TILE + wc * 128 + j * 32 + col_l;
      #pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t gi = (int64_t)ti * TILE + wr * 128 + i * 32 + 8 * (r >> 2) + row_l + (r & 3);
        if (gi < K && gj < K) {
          float* p = H + gi * K + gj;
          const float v = beta * acc[i][j][r];
          *p = (alpha != 0.0f) ? (alpha * *p + v) : v;
        }
      }
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
  const int nt = (int)((K + TILE - 1) / TILE);
  const int64_t tiles = (int64_t)nt * (nt + 1) / 2;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LCQ_BF16)
    hessian_kernel<true><<<dim3((unsigned)tiles), dim3(256), 0, st>>>(H, (int)K, (const uint16_t*)X, (int)T, alpha, beta, nt);
  else if (dtype == LCQ_F16)
    hessian_kernel<false><<<dim3((unsigned)tiles), dim3(256), 0, st>>>(H, (int)K, (const uint16_t*)X, (int)T, alpha, beta, nt);
  else return LCQ_EDTYPE;
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
