// Streaming probe (gfx950): what this GPU sustains for a kernel that does nothing but stream, at a given ratio of
// bytes read to bytes written.  The quantizer kernels are HBM-bound with ratios from 4:5 (fp32 in, fp32 + codes out)
// to 4:1 (bf16 in, packed nibbles out); the rate of a plain copy is the ceiling of the first kind only.  Not part
// of the quantization path: the benchmark calls it to put each kernel's rate beside the ceiling of its own mix.
//
// Each thread reads W 16-byte chunks (one workgroup covers contiguous 4 KiB runs, as the quantizers do) and writes
// their xor as one chunk; W == 0 reads eight chunks and writes nothing (the store is behind a test no data passes).
#include "common.h"
#include "lcq_internal.h"

namespace {


template <int W>
__global__ __launch_bounds__(256) void stream_probe_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                           int64_t n16) {
  constexpr int U = W == 0 ? 8 : (W < 4 ? 4 : W);            // chunks per thread
  const int64_t base = (int64_t)blockIdx.x * 256 * U;
  u32x4 v[U];
  #pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = base + k * 256 + threadIdx.x;
    v[k] = i < n16 ? __builtin_nontemporal_load(src + i) : u32x4{0, 0, 0, 0};
  }
  if constexpr (W == 0) {
    u32x4 a = v[0];
    #pragma unroll
    for (int k = 1; k < U; ++k) a ^= v[k];
    if (a[0] == 0x12345678u && a[1] == 0x9abcdef0u && a[2] == 0x0fedcba9u && a[3] == 0x87654321u) dst[threadIdx.x] = a;
  } else {
    constexpr int NW = U / W;                                // chunks written per thread
    #pragma unroll
    for (int j = 0; j < NW; ++j) {
      u32x4 a = v[j * W];
      #pragma unroll
      for (int k = 1; k < W; ++k) a ^= v[j * W + k];
      const int64_t o = ((int64_t)blockIdx.x * NW + j) * 256 + threadIdx.x;
      if (o * W < n16) __builtin_nontemporal_store(a, dst + o);
    }
  }
}

}  // namespace

extern "C" {

int lcq_stream_probe(const void* src, void* dst, int64_t bytes, int64_t dst_bytes, int reads_per_write, void* stream) {
  if (!src || !dst || bytes <= 0 || bytes % 16 != 0) return LCQ_EINVAL;
  if ((((uintptr_t)src | (uintptr_t)dst) % 16) != 0) return LCQ_EALIGN;
  const int64_t n16 = bytes / 16;
  // the kernel writes chunk o of dst for every o with o * reads_per_write < n16 (256 chunks when it only reads)
  const int64_t need = reads_per_write > 0 ? (n16 + reads_per_write - 1) / reads_per_write * 16 : 4096;
  if (dst_bytes < need) return LCQ_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  #define LCQ_PROBE(W, U) do { const int64_t g = (n16 + 256 * U - 1) / (256 * U); if (g > 0x7fffffff) return LCQ_EINVAL; \
    stream_probe_kernel<W><<<dim3((unsigned)g), dim3(256), 0, st>>>((const u32x4*)src, (u32x4*)dst, n16); } while (0)
  switch (reads_per_write) {
    case 0: LCQ_PROBE(0, 8); break;
    case 1: LCQ_PROBE(1, 4); break;
    case 2: LCQ_PROBE(2, 4); break;
    case 4: LCQ_PROBE(4, 4); break;
    case 8: LCQ_PROBE(8, 8); break;
    default: return LCQ_EINVAL;
  }
  #undef LCQ_PROBE
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
