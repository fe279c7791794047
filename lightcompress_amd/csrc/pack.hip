// int4 / int8 code packing for gfx950.
//
//  * lcq_pack_ct      : compressed-tensors "pack-quantized" layout used by the
//                       vLLM / SGLang / LightLLM exporters
//                       (VllmRealQuantLinear.pack, module_utils.py:929-955):
//                       u = uint8(code + 2^(bits-1)); word j of a row holds
//                       u[pf*j + i] << (bits*i), pf = 32 / bits, tail zero-padded.
//                       The reference round-trips through numpy on the host.
//  * lcq_pack_awq     : AutoAWQ / MLC "gemm_pack" layout
//                       (AutoawqRealQuantLinear.gemm_pack, module_utils.py:1097-1158):
//                       iw[r,k] = int(round((w[r,k] + z*s) / s)) with fp16 scales,
//                       NOT clamped; qweight[k, c] = OR_i iw[8c+order[i], k] << 4i,
//                       order = 0,2,4,6,1,3,5,7; qzeros likewise; scales -> fp16 [K/g, R].
//                       The reference loops over K columns and R/8 x 8 nibbles in Python.
// Both are pure HBM-bound byte shuffles: one read of the codes / weights, one
// write of the packed words.
#include "common.h"
#include "lcq_internal.h"

namespace {

template <typename CodeT>
__global__ __launch_bounds__(256) void pack_ct_kernel(const CodeT* __restrict__ codes, int64_t R, int64_t K, int bits,
                                                      int64_t words_per_row, uint32_t* __restrict__ packed) {
  const int pf = 32 / bits;
  const int offset = 1 << (bits - 1);
  const int64_t total = R * words_per_row;
  for (int64_t w = (int64_t)blockIdx.x * 256 + threadIdx.x; w < total; w += (int64_t)gridDim.x * 256) {
    const int64_t r = w / words_per_row, j = w % words_per_row;
    const CodeT* src = codes + r * K + j * pf;
    uint32_t acc = 0;
    if (sizeof(CodeT) == 4 && pf == 8 && (j + 1) * pf <= K && (K % 4) == 0) {
      const u32x4 a = *(const u32x4*)src, b = *(const u32x4*)(src + 4);
      #pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc |= ((a[i] + (uint32_t)offset) & 0xffu) << (4 * i);
        acc |= ((b[i] + (uint32_t)offset) & 0xffu) << (4 * (i + 4));
      }
    } else {
      for (int i = 0; i < pf; ++i) {
        const int64_t col = j * pf + i;
        if (col < K) acc |= (((uint32_t)(int32_t)src[i] + (uint32_t)offset) & 0xffu) << (bits * i);
      }
    }
    packed[w] = acc;
  }
}

template <int WDT> __device__ __forceinline__ float load_w(const void* w, int64_t i);
template <> __device__ __forceinline__ float load_w<LCQ_F32>(const void* w, int64_t i) { return ((const float*)w)[i]; }
template <> __device__ __forceinline__ float load_w<LCQ_BF16>(const void* w, int64_t i) { return u2f((uint32_t)((const uint16_t*)w)[i] << 16); }
template <> __device__ __forceinline__ float load_w<LCQ_F16>(const void* w, int64_t i) { return (float)((const _Float16*)w)[i]; }

constexpr int AWQ_TR = 256;   // output channels per tile
constexpr int AWQ_TK = 32;    // input channels per tile
constexpr int AWQ_PITCH = AWQ_TR + 1;

// one tile: iw for AWQ_TR rows x AWQ_TK columns through LDS, then R/8 words per column
template <int WDT>
__global__ __launch_bounds__(256) void pack_awq_kernel(const void* __restrict__ w, const void* __restrict__ scales,
                                                       const int32_t* __restrict__ zeros, int64_t R, int64_t K, int g,
                                                       int32_t* __restrict__ qweight) {
  extern __shared__ int32_t tile[];                         // [AWQ_TK][AWQ_PITCH]
  const int64_t r0 = (int64_t)blockIdx.y * AWQ_TR, k0 = (int64_t)blockIdx.x * AWQ_TK;
  const int64_t G = K / g;
  const int tk = threadIdx.x & 31, tr = threadIdx.x >> 5;
  for (int rr = tr; rr < AWQ_TR; rr += 8) {
    const int64_t r = r0 + rr, k = k0 + tk;
    int32_t iw = 0;
    if (r < R && k < K) {
      const int64_t gi = r * G + k / g;
      const float s16 = f16_round(load_w<WDT>(scales, gi));            // scales.to(float16)
      const float sz = f16_round((float)zeros[gi] * s16);              // zeros * scales, fp16 result
      const float x = load_w<WDT>(w, r * K + k);
      float t;
      if (WDT == LCQ_F16) t = f16_round(f16_round(x + sz) / s16);      // all-fp16 tensor ops
      else t = (x + sz) / s16;                                         // promoted to fp32
      iw = (int32_t)rintf(t);
    }
    tile[tk * AWQ_PITCH + rr] = iw;
  }
  __syncthreads();
  const int order[8] = {0, 2, 4, 6, 1, 3, 5, 7};
  const int c = threadIdx.x & 31;
  for (int kk = threadIdx.x >> 5; kk < AWQ_TK; kk += 8) {
    const int64_t k = k0 + kk;
    const int64_t cg = r0 / 8 + c;
    if (k < K && cg < R / 8) {
      uint32_t acc = 0;
      #pragma unroll
      for (int i = 0; i < 8; ++i) acc |= (uint32_t)tile[kk * AWQ_PITCH + 8 * c + order[i]] << (4 * i);
      qweight[k * (R / 8) + cg] = (int32_t)acc;
    }
  }
}

template <int WDT>
__global__ __launch_bounds__(256) void pack_awq_qparams_kernel(const void* __restrict__ scales, const int32_t* __restrict__ zeros,
                                                               int64_t R, int64_t G, uint16_t* __restrict__ scales_out,
                                                               int32_t* __restrict__ qzeros) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < G * R) {                                          // scales.t().contiguous().to(float16)
    const int64_t gi = i / R, r = i % R;
    const _Float16 h = (_Float16)load_w<WDT>(scales, r * G + gi);
    scales_out[i] = __builtin_bit_cast(uint16_t, h);
  }
  if (i < G * (R / 8)) {
    const int order[8] = {0, 2, 4, 6, 1, 3, 5, 7};
    const int64_t gi = i / (R / 8), c = i % (R / 8);
    uint32_t acc = 0;
    #pragma unroll
    for (int j = 0; j < 8; ++j) acc |= (uint32_t)zeros[(8 * c + order[j]) * G + gi] << (4 * j);
    qzeros[i] = (int32_t)acc;
  }
}

}  // namespace

extern "C" {

int lcq_pack_ct(const void* codes, int code_dtype, int64_t R, int64_t K, int bits, int32_t* packed, void* stream) {
  if (!codes || !packed || R < 0 || K <= 0) return LCQ_EINVAL;
  if (bits != 4 && bits != 8 && bits != 2 && bits != 16) return LCQ_EINVAL;
  if (R == 0) return LCQ_OK;
  const int pf = 32 / bits;
  const int64_t wpr = (K + pf - 1) / pf;
  int64_t grid = (R * wpr + 255) / 256;
  if (grid > 1 << 20) grid = 1 << 20;
  hipStream_t st = (hipStream_t)stream;
  if (code_dtype == LCQ_CODE_I32) pack_ct_kernel<int32_t><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const int32_t*)codes, R, K, bits, wpr, (uint32_t*)packed);
  else if (code_dtype == LCQ_CODE_I8) pack_ct_kernel<int8_t><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const int8_t*)codes, R, K, bits, wpr, (uint32_t*)packed);
  else if (code_dtype == LCQ_CODE_U8) pack_ct_kernel<uint8_t><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const uint8_t*)codes, R, K, bits, wpr, (uint32_t*)packed);
  else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_pack_awq(const void* w, int dtype, const void* scales, const int32_t* zeros, int64_t R, int64_t K, int group_size,
                 int32_t* qweight, void* scales_f16_out, int32_t* qzeros, void* stream) {
  if (!w || !scales || !zeros || !qweight || !scales_f16_out || !qzeros) return LCQ_EINVAL;
  if (R <= 0 || K <= 0 || group_size <= 0 || K % group_size != 0 || R % 32 != 0) return LCQ_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)((K + AWQ_TK - 1) / AWQ_TK), (unsigned)((R + AWQ_TR - 1) / AWQ_TR));
  const size_t lds = (size_t)AWQ_TK * AWQ_PITCH * sizeof(int32_t);
  const int64_t G = K / group_size;
  const int64_t n = G * R;
  const unsigned g2 = (unsigned)((n + 255) / 256);
  if (dtype == LCQ_F32) {
    pack_awq_kernel<LCQ_F32><<<grid, dim3(256), lds, st>>>(w, scales, zeros, R, K, group_size, qweight);
    pack_awq_qparams_kernel<LCQ_F32><<<dim3(g2), dim3(256), 0, st>>>(scales, zeros, R, G, (uint16_t*)scales_f16_out, qzeros);
  } else if (dtype == LCQ_BF16) {
    pack_awq_kernel<LCQ_BF16><<<grid, dim3(256), lds, st>>>(w, scales, zeros, R, K, group_size, qweight);
    pack_awq_qparams_kernel<LCQ_BF16><<<dim3(g2), dim3(256), 0, st>>>(scales, zeros, R, G, (uint16_t*)scales_f16_out, qzeros);
  } else if (dtype == LCQ_F16) {
    pack_awq_kernel<LCQ_F16><<<grid, dim3(256), lds, st>>>(w, scales, zeros, R, K, group_size, qweight);
    pack_awq_qparams_kernel<LCQ_F16><<<dim3(g2), dim3(256), 0, st>>>(scales, zeros, R, G, (uint16_t*)scales_f16_out, qzeros);
  } else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
