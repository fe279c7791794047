// Histogram of a tensor for the static_hist observer (gfx950).
//
// Replaces the torch.histc(tensor.float(), bins, min, max) calls of BaseQuantizer.get_static_hist_range
// (llmc/compression/quantization/quant.py:461-511).  torch's device kernel puts value v into
//   bin = (int)((v - min) * bins / (max - min)),   bin == bins -> bins - 1,   only for min <= v <= max
// in fp32 (bins converted to fp32, multiply before divide); min == max widens the range to [min - 1, max + 1].
// HBM-bound: one read of the tensor.  A workgroup counts into an LDS histogram (32-bit integers, so counts stay
// exact beyond 2^24 where torch's fp32 atomics start to depend on their order), then adds its non-empty bins to the
// global counters with vector atomics; a second tiny kernel converts the counters to fp32.
#include "rowquant.h"

namespace {
using namespace lcq;

constexpr int HIST_MAX_BINS = 8192;

__global__ __launch_bounds__(256) void hist_zero_kernel(uint32_t* __restrict__ counts, int bins) {
  for (int i = blockIdx.x * 256 + threadIdx.x; i < bins; i += gridDim.x * 256) counts[i] = 0u;
}

template <bool BF, bool HALF>
__global__ __launch_bounds__(256) void hist_kernel(const void* __restrict__ x, int64_t n, int bins, float lo, float hi,
                                                   uint32_t* __restrict__ counts) {
  __shared__ uint32_t lh[HIST_MAX_BINS];
  for (int i = threadIdx.x; i < bins; i += 256) lh[i] = 0u;
  __syncthreads();
  const float fb = (float)bins, span = hi - lo;
  auto put = [&](float v) {
    if (v >= lo && v <= hi) {
      int b = (int)((v - lo) * fb / span);
      if (b == bins) b -= 1;
      atomicAdd(&lh[b], 1u);
    }
  };
  constexpr int N = (BF || HALF) ? 8 : 4;
  const int64_t nch = n / N;
  for (int64_t ch = (int64_t)blockIdx.x * 256 + threadIdx.x; ch < nch; ch += (int64_t)gridDim.x * 256) {
    const u32x4 raw = __builtin_nontemporal_load((const u32x4*)x + ch);
    if constexpr (HALF) {
      #pragma unroll
      for (int i = 0; i < 4; ++i) {
        const _Float16 a = __builtin_bit_cast(_Float16, (uint16_t)(raw[i] & 0xffffu));
        const _Float16 b = __builtin_bit_cast(_Float16, (uint16_t)(raw[i] >> 16));
        put((float)a);
        put((float)b);
      }
    } else {
      float v[N];
      unpack<BF>(raw, v);
      #pragma unroll
      for (int i = 0; i < N; ++i) put(v[i]);
    }
  }
  if (blockIdx.x == 0) {                                   // ragged tail (n % N elements)
    for (int64_t i = nch * N + threadIdx.x; i < n; i += 256) {
      if constexpr (HALF) put((float)((const _Float16*)x)[i]);
      else put(load_scalar<BF>(x, i));
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < bins; i += 256) {
    const uint32_t c = lh[i];
    if (c) atomicAdd(&counts[i], c);
  }
}

__global__ __launch_bounds__(256) void hist_to_float_kernel(const uint32_t* __restrict__ counts, int bins, float* __restrict__ hist) {
  for (int i = blockIdx.x * 256 + threadIdx.x; i < bins; i += gridDim.x * 256) hist[i] = (float)counts[i];
}

}  // namespace

extern "C" {

int lcq_histc(const void* x, int dtype, int64_t n, int bins, float lo, float hi, void* counts, float* hist, void* stream) {
  if (!x || !counts || !hist || n < 0 || bins <= 0 || bins > HIST_MAX_BINS) return LCQ_EINVAL;
  if (!(lo <= hi) || !(__builtin_isfinite(lo) && __builtin_isfinite(hi))) return LCQ_EINVAL;   // torch: "max must be larger than min", finite range
  if (dtype != LCQ_F32 && dtype != LCQ_BF16 && dtype != LCQ_F16) return LCQ_EDTYPE;     // before anything is launched
  if (((uintptr_t)x % 16) != 0) return LCQ_EALIGN;
  if (lo == hi) { lo -= 1.0f; hi += 1.0f; }
  hipStream_t st = (hipStream_t)stream;
  const unsigned zb = (unsigned)((bins + 255) / 256);
  hist_zero_kernel<<<dim3(zb), dim3(256), 0, st>>>((uint32_t*)counts, bins);
  const int per = (dtype == LCQ_F32) ? 4 : 8;
  int64_t grid = (n / per + 256 * 8 - 1) / (256 * 8);
  if (grid < 1) grid = 1;
  if (grid > 2048) grid = 2048;
  if (dtype == LCQ_F32) hist_kernel<false, false><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, n, bins, lo, hi, (uint32_t*)counts);
  else if (dtype == LCQ_BF16) hist_kernel<true, false><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, n, bins, lo, hi, (uint32_t*)counts);
  else hist_kernel<false, true><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, n, bins, lo, hi, (uint32_t*)counts);
  hist_to_float_kernel<<<dim3(zb), dim3(256), 0, st>>>((const uint32_t*)counts, bins, hist);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
