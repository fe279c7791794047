// Block-wise float8 (e4m3) casts for gfx950: one fp32 scale per 128x128 weight block or per
// 128-element activation block.
//
// Replaces the reference's Triton kernels weight_cast_to_fp8 / weight_cast_to_bf16 / act_quant
// (llmc/compression/quantization/kernel.py:7-138) and its non-Hopper fallback through
// FloatQuantizer(granularity='per_block') (quant.py:20-45, 138-140, 634-638, 1194-1220):
//   s = max|x| / 448        (fallback: clamp(max|x|, 1e-5) / 448, LCQ_FLAG_CLAMP_RANGE)
//   y = float8_e4m3fn(x / s)   in fp32 arithmetic whatever the input type
//   back:  out = float(y) * s
// Rounding to float8 is the hardware convert (round to nearest even, what Triton's and torch's casts
// do); LCQ_FLAG_TIE_AWAY nudges exact ties one ulp outwards first (the add-half-then-truncate model of
// float_quantize).  x / s is evaluated as x * (1/s) unless the product is within 8 ulp of a float8
// rounding boundary, where the lane divides.
#include "rowquant.h"

namespace {
using namespace lcq;

constexpr int BS = 128;

// value handed to the float8 convert.  model = false: x / s itself (Triton / torch cast: one rounding, to
// nearest even, done by the convert).  model = true: the FloatQuantizer route, "x / s + 0" rounded by the
// float_quantize model first - add-half-then-truncate on the fp32 mantissa (ties away; tie_even: to even),
// and below the minimum normal 2^-6 the same on |t| + 2^-6 (whose fp32 addition already rounds once) - so the
// convert only re-encodes an exact grid value.
__device__ __forceinline__ float fp8_input(float x, float s, float r, bool fast, bool tie_away, bool model) {
  float t = x * r;
  const uint32_t lowm = f2u(t) & 0xfffffu;                  // 20 dropped mantissa bits of e4m3
  const bool sub = !(fabsf(t) >= 0.015625f);                // below the minimum normal 2^-6: fixed step 2^-9
  if (__builtin_expect(!fast || sub || (lowm - 0x7fff8u) <= 16u, 0)) t = x / s;
  if (!model) return t;
  t = t + 0.0f;                                             // "+ zeros": -0 becomes +0
  if (fabsf(t) >= 0.015625f) {
    if (tie_away && (f2u(t) & 0xfffffu) == 0x80000u) t = u2f(f2u(t) + 1u);   // an exact tie: push it outwards
    return t;
  }
  if (!(fabsf(t) == fabsf(t))) return t;                    // NaN
  const uint32_t b = f2u(fabsf(t) + 0.015625f);
  const uint32_t rb = tie_away ? (b + 0x80000u) & 0xfff00000u : (b + 0x7ffffu + ((b >> 20) & 1u)) & 0xfff00000u;
  return __builtin_copysignf(u2f(rb) - 0.015625f, t);
}

struct BlkArgs {
  const void* x; uint8_t* y; float* scales;
  int64_t M, N;
  int nbn, clamp_range, tie_away;
};

// one workgroup per 128x128 block: 2048 (bf16) / 4096 (fp32) 16-byte chunks, 8 / 16 per thread in registers
template <bool BF>
__global__ __launch_bounds__(256) void block_quant_kernel(BlkArgs a) {
  constexpr int N = Vec<BF>::N, CPR = BS / N, PER = BS * CPR / 256;
  __shared__ float sm[4];
  const int bm = blockIdx.y, bn = blockIdx.x;
  u32x4 raw[PER];
  bool ok[PER];
  float amax = 0.0f;
  #pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int ci = threadIdx.x + k * 256, r = ci / CPR, c = ci % CPR;
    const int64_t row = (int64_t)bm * BS + r, col = (int64_t)bn * BS + c * N;
    ok[k] = row < a.M && col < a.N;
    raw[k] = ok[k] ? __builtin_nontemporal_load((const u32x4*)a.x + (row * a.N + col) / N) : u32x4{0, 0, 0, 0};
    float v[N];
    unpack<BF>(raw[k], v);
    #pragma unroll
    for (int i = 0; i < N; ++i) amax = nan_max(amax, fabsf(v[i]));
  }
  amax = team_reduce<64, true>(amax);
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = nan_max(nan_max(sm[0], sm[1]), nan_max(sm[2], sm[3]));
  if (a.clamp_range) amax = nan_max(amax, 1e-5f);
  const float s = amax / 448.0f;
  const float r = __builtin_amdgcn_rcpf(s);
  const bool fast = (s > 8.6736174e-19f) && (s < 1.1529215e18f);
  if (threadIdx.x == 0) a.scales[(int64_t)bm * a.nbn + bn] = s;
  #pragma unroll
  for (int k = 0; k < PER; ++k) {
    if (!ok[k]) continue;
    const int ci = threadIdx.x + k * 256, rr = ci / CPR, c = ci % CPR;
    const int64_t row = (int64_t)bm * BS + rr, col = (int64_t)bn * BS + c * N;
    float v[N];
    unpack<BF>(raw[k], v);
    #pragma unroll
    for (int i = 0; i < N; ++i) v[i] = fp8_input(v[i], s, r, fast, a.tie_away, a.clamp_range);
    uint32_t w[N / 4];
    #pragma unroll
    for (int q = 0; q < N / 4; ++q) {
      int u = 0;
      u = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * q], v[4 * q + 1], u, false);
      u = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * q + 2], v[4 * q + 3], u, true);
      w[q] = (uint32_t)u;
    }
    uint8_t* dst = a.y + row * a.N + col;
    if constexpr (N == 8) *(u32x2*)dst = u32x2{w[0], w[1]};
    else *(uint32_t*)dst = w[0];
  }
}

// activations: one 128-element block per 16-lane (bf16) / 32-lane (fp32) team, one chunk per lane
template <bool BF>
__global__ __launch_bounds__(256) void act_quant_kernel(const u32x4* __restrict__ x, int64_t nblocks, uint8_t* __restrict__ y,
                                                        float* __restrict__ scales, int clamp_range, int tie_away) {
  constexpr int N = Vec<BF>::N, TEAM = BS / N;
  const int64_t blk = ((int64_t)blockIdx.x * 256 + threadIdx.x) / TEAM;
  const int t = threadIdx.x % TEAM;
  const bool okb = blk < nblocks;
  const u32x4 raw = okb ? __builtin_nontemporal_load(x + blk * TEAM + t) : u32x4{0, 0, 0, 0};
  float v[N];
  unpack<BF>(raw, v);
  float amax = 0.0f;
  #pragma unroll
  for (int i = 0; i < N; ++i) amax = nan_max(amax, fabsf(v[i]));
  amax = team_reduce<TEAM, true>(amax);
  if (clamp_range) amax = nan_max(amax, 1e-5f);
  const float s = amax / 448.0f;
  const float r = __builtin_amdgcn_rcpf(s);
  const bool fast = (s > 8.6736174e-19f) && (s < 1.1529215e18f);
  if (!okb) return;
  if (t == 0) scales[blk] = s;
  #pragma unroll
  for (int i = 0; i < N; ++i) v[i] = fp8_input(v[i], s, r, fast, tie_away, clamp_range);
  uint32_t w[N / 4];
  #pragma unroll
  for (int q = 0; q < N / 4; ++q) {
    int u = 0;
    u = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * q], v[4 * q + 1], u, false);
    u = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * q + 2], v[4 * q + 3], u, true);
    w[q] = (uint32_t)u;
  }
  uint8_t* dst = y + (blk * TEAM + t) * N;
  if constexpr (N == 8) *(u32x2*)dst = u32x2{w[0], w[1]};
  else *(uint32_t*)dst = w[0];
}

// out = float(y) * s[block]; 8 float8 per thread
template <int OUT>   // LCQ_F32 | LCQ_BF16
__global__ __launch_bounds__(256) void block_dequant_kernel(const uint8_t* __restrict__ y, const float* __restrict__ scales,
                                                            int64_t M, int64_t N, int nbn, void* __restrict__ out) {
  const int64_t npr = N / 8, total = M * npr;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < total; c += (int64_t)gridDim.x * 256) {
    const int64_t row = c / npr, col = (c % npr) * 8;
    const float s = scales[(row / BS) * nbn + col / BS];
    const u32x2 w = *(const u32x2*)(y + row * N + col);
    float v[8];
    #pragma unroll
    for (int q = 0; q < 2; ++q) {
      const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[q], false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[q], true);
      v[4 * q] = lo[0] * s; v[4 * q + 1] = lo[1] * s; v[4 * q + 2] = hi[0] * s; v[4 * q + 3] = hi[1] * s;
    }
    if constexpr (OUT == LCQ_BF16) {
      *((u32x4*)out + c) = pack_rne<true>(v);
    } else {
      *((u32x4*)out + 2 * c) = u32x4{f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])};
      *((u32x4*)out + 2 * c + 1) = u32x4{f2u(v[4]), f2u(v[5]), f2u(v[6]), f2u(v[7])};
    }
  }
}

}  // namespace

extern "C" {

int lcq_fp8_block_quant(const void* x, int dtype, int64_t M, int64_t N, int block_rows, int flags, void* y, float* scales,
                        void* stream) {
  if (!x || !y || !scales || M <= 0 || N <= 0) return LCQ_EINVAL;
  if (dtype != LCQ_F32 && dtype != LCQ_BF16) return LCQ_EDTYPE;
  if (block_rows != 1 && block_rows != BS) return LCQ_EINVAL;
  const int n = dtype == LCQ_BF16 ? 8 : 4;
  if (N % n != 0 || ((uintptr_t)x % 16) != 0 || ((uintptr_t)y % 8) != 0) return LCQ_EALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int clamp_range = (flags & LCQ_FLAG_CLAMP_RANGE) != 0, tie_away = (flags & LCQ_FLAG_TIE_AWAY) != 0;
  if (block_rows == 1) {
    if (N % BS != 0) return LCQ_EINVAL;
    const int64_t nblocks = M * (N / BS);
    const int team = BS / n;
    const int64_t grid = (nblocks * team + 255) / 256;
    if (grid > 0x7fffffff) return LCQ_EINVAL;
    if (dtype == LCQ_BF16) act_quant_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)x, nblocks, (uint8_t*)y, scales, clamp_range, tie_away);
    else act_quant_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)x, nblocks, (uint8_t*)y, scales, clamp_range, tie_away);
  } else {
    BlkArgs a;
    a.x = x; a.y = (uint8_t*)y; a.scales = scales; a.M = M; a.N = N;
    a.nbn = (int)((N + BS - 1) / BS); a.clamp_range = clamp_range; a.tie_away = tie_away;
    const dim3 grid((unsigned)a.nbn, (unsigned)((M + BS - 1) / BS));
    if (grid.y > 65535) return LCQ_EINVAL;
    if (dtype == LCQ_BF16) block_quant_kernel<true><<<grid, dim3(256), 0, st>>>(a);
    else block_quant_kernel<false><<<grid, dim3(256), 0, st>>>(a);
  }
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_fp8_block_dequant(const void* y, const float* scales, int64_t M, int64_t N, void* out, int out_dtype, void* stream) {
  if (!y || !scales || !out || M <= 0 || N <= 0) return LCQ_EINVAL;
  if (N % 8 != 0 || ((uintptr_t)y % 8) != 0 || ((uintptr_t)out % 16) != 0) return LCQ_EALIGN;
  const int nbn = (int)((N + BS - 1) / BS);
  int64_t grid = (M * (N / 8) + 255) / 256;
  if (grid > 262144) grid = 262144;
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == LCQ_BF16) block_dequant_kernel<LCQ_BF16><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const uint8_t*)y, scales, M, N, nbn, out);
  else if (out_dtype == LCQ_F32) block_dequant_kernel<LCQ_F32><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const uint8_t*)y, scales, M, N, nbn, out);
  else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
