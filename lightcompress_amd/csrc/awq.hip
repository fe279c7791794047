// AWQ scale-search helpers for gfx950 (the weight side, W*s -> fake quant, is
// lcq_awq_scale_quant in quant_int.hip).
//
//   lcq_absmean_cols   Awq.get_act_scale            awq.py:74-85     mean_t |x[t, k]|
//   lcq_div_cols       scaling_input                base_blockwise_quantization.py:899-912   x / s[None, :]
//   lcq_sq_err_mean    Awq.calculate_loss           awq.py:134-145   mean(((a - b) in the tensor dtype).float()^2)
//   lcq_awq_weight_scale  Awq.get_weight_scale      awq.py:48-72     mean_r (|W| / group max)
//
// All four are single-pass HBM-bound streams: 16-byte loads per lane,
// per-thread fp32 partial sums, one small second stage.
#include <mutex>

#include "rowquant.h"

namespace {
using namespace lcq;

constexpr int PARTS_MAX = 1024;
constexpr int SQERR_PARTS_MAX = 8192;          // workgroups (= partial sums) of a squared-error launch

// Partial sums of lcq_sq_err_mean_static, 64 KiB.  Every GPU the library runs on holds its own copy of this array
// for the life of the process.  In host code the NAME of the array is only a handle: its device address is looked
// up once per device with hipGetSymbolAddress (static_scratch() below) and only that pointer is handed to kernels.
static __device__ __align__(256) double scratch[SQERR_PARTS_MAX];

constexpr int MAX_DEVICES = 64;
double* scratch_ptr[MAX_DEVICES] = {};
std::mutex scratch_mutex;

// device address of `scratch` on the current device, or nullptr
double* static_scratch() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
    scratch_ptr[dev] = (double*)p;
  }
  return scratch_ptr[dev];
}

// ---- column-wise mean of |x| over T rows ------------------------------------------------
// grid = (column blocks of 256 * N, row splits); every thread owns one 16-byte column chunk
template <int BF>
__global__ __launch_bounds__(256) void absmean_stage1(const u32x4* __restrict__ x, int64_t T, int64_t K,
                                                      float* __restrict__ part) {
  constexpr int N = Vec<BF>::N;
  const int64_t nch = K / N;
  const int64_t ch = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (ch >= nch) return;
  const int64_t rows_per = (T + gridDim.y - 1) / gridDim.y;
  const int64_t r0 = blockIdx.y * rows_per, r1 = min(T, r0 + rows_per);
  float acc[N];
  #pragma unroll
  for (int i = 0; i < N; ++i) acc[i] = 0.0f;
  for (int64_t r = r0; r < r1; ++r) {
    float v[N];
    unpack<BF>(__builtin_nontemporal_load(x + r * nch + ch), v);
    #pragma unroll
    for (int i = 0; i < N; ++i) acc[i] += fabsf(v[i]);
  }
  float* p = part + (int64_t)blockIdx.y * K + ch * N;
  #pragma unroll
  for (int i = 0; i < N; ++i) p[i] = acc[i];
}
// torch's GPU mean is sum * factor with the fp32 factor = float(outputs) / elements (not a division by the count, which
// is what its CPU kernel does); the fp32 product is then cast to the output type.  (In torch's ROCm build the compiler
// has fused that multiply with the cast to fp16 - one rounding of the exact product, which differs when sum * factor
// is an fp16 tie; the CUDA build rounds twice, and so does this kernel, like every other fp16 product here.)
template <int BF>
__global__ __launch_bounds__(256) void absmean_stage2(const float* __restrict__ part, int nparts, float factor, int64_t K,
                                                      void* __restrict__ out) {
  const int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (k >= K) return;
  float s = 0.0f;
  for (int p = 0; p < nparts; ++p) s += part[(int64_t)p * K + k];
  store_scalar<BF>(out, k, rnd<BF>(s * factor));
}

// float(outputs) / elements as torch's mean over the first dimension of [T, K] evaluates it
inline float mean_factor(int64_t T, int64_t K) { return (float)K / (float)(T * K); }

// ---- x / s[None, :] -----------------------------------------------------------------------
template <int BF>
__global__ __launch_bounds__(256) void div_cols_kernel(const u32x4* __restrict__ x, const u32x4* __restrict__ s,
                                                       int64_t nchunks_total, int64_t nch_row, u32x4* __restrict__ out) {
  constexpr int N = Vec<BF>::N;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < nchunks_total; c += (int64_t)gridDim.x * 256) {
    float v[N], sv[N];
    unpack<BF>(__builtin_nontemporal_load(x + c), v);
    unpack<BF>(s[c % nch_row], sv);
    #pragma unroll
    for (int i = 0; i < N; ++i) v[i] = rnd_e<BF>(v[i] / sv[i]);
    __builtin_nontemporal_store(pack<BF>(v), out + c);
  }
}

// ---- in-place capable w (*|/) s[col]  or  w (*|/) s[row] -------------------------------------
// mode: 0 multiply by a column vector, 1 divide by a column vector, 2 multiply by a row vector, 3 divide by one
template <int BF>
__global__ __launch_bounds__(256) void scale_kernel(const u32x4* x, const void* __restrict__ s, int64_t nchunks_total,
                                                    int64_t nch_row, int mode, u32x4* out) {
  constexpr int N = Vec<BF>::N;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < nchunks_total; c += (int64_t)gridDim.x * 256) {
    float v[N], sv[N];
    unpack<BF>(x[c], v);
    if (mode < 2) {
      unpack<BF>(((const u32x4*)s)[c % nch_row], sv);
    } else {
      const float r = load_scalar<BF>(s, c / nch_row);
      #pragma unroll
      for (int i = 0; i < N; ++i) sv[i] = r;
    }
    if (mode & 1) {
      #pragma unroll
      for (int i = 0; i < N; ++i) v[i] = v[i] / sv[i];
    } else {
      #pragma unroll
      for (int i = 0; i < N; ++i) v[i] = v[i] * sv[i];
    }
    out[c] = pack_rne<BF>(v);
  }
}

// ---- mean of squared differences ------------------------------------------------------------
template <int BF>
__global__ __launch_bounds__(256) void sqerr_stage1(const u32x4* __restrict__ a, const u32x4* __restrict__ b,
                                                    int64_t nchunks, double* __restrict__ part) {
  constexpr int N = Vec<BF>::N;
  __shared__ float sm[4];
  float acc = 0.0f;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < nchunks; c += (int64_t)gridDim.x * 256) {
    float va[N], vb[N];
    unpack<BF>(__builtin_nontemporal_load(a + c), va);
    unpack<BF>(__builtin_nontemporal_load(b + c), vb);
    #pragma unroll
    for (int i = 0; i < N; ++i) { const float d = rnd_e<BF>(va[i] - vb[i]); acc += d * d; }
  }
  acc = team_sum<64>(acc);
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) part[blockIdx.x] = (double)sm[0] + (double)sm[1] + (double)sm[2] + (double)sm[3];
}
__global__ __launch_bounds__(256) void sqerr_stage2(const double* __restrict__ part, int nparts, double n,
                                                    float* __restrict__ out) {
  __shared__ double sm[256];
  double s = 0.0;
  for (int i = threadIdx.x; i < nparts; i += 256) s += part[i];
  sm[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) sm[threadIdx.x] += sm[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[0] = (float)(sm[0] / n);
}

// ---- mean over rows of |W| / (group max of |W|) -----------------------------------------------
// one workgroup per slab of rows; a group of g columns is shared by g/N consecutive lanes
template <int BF, int TEAM>
__global__ __launch_bounds__(256) void wscale_stage1(const u32x4* __restrict__ w, int64_t R, int64_t K,
                                                     float* __restrict__ part) {
  constexpr int N = Vec<BF>::N;
  const int64_t nch = K / N;
  const int64_t rows_per = (R + gridDim.x - 1) / gridDim.x;
  const int64_t r0 = blockIdx.x * rows_per, r1 = min(R, r0 + rows_per);
  for (int64_t ch0 = 0; ch0 < nch; ch0 += 256) {
    const int64_t ch = ch0 + threadIdx.x;
    float acc[N];
    #pragma unroll
    for (int i = 0; i < N; ++i) acc[i] = 0.0f;
    for (int64_t r = r0; r < r1; ++r) {
      float v[N];
      float mx = 0.0f;
      if (ch < nch) {
        unpack<BF>(w[r * nch + ch], v);
        #pragma unroll
        for (int i = 0; i < N; ++i) { v[i] = fabsf(v[i]); mx = fmaxf(mx, v[i]); }
      }
      mx = team_reduce<TEAM, true>(mx);
      if (ch < nch) {
        #pragma unroll
        for (int i = 0; i < N; ++i) acc[i] += rnd_e<BF>(v[i] / mx);
      }
    }
    if (ch < nch) {
      float* p = part + (int64_t)blockIdx.x * K + ch * N;
      #pragma unroll
      for (int i = 0; i < N; ++i) p[i] = acc[i];
    }
  }
}

template <int BF>
int absmean(const void* x, int64_t T, int64_t K, void* out, float* part, hipStream_t st) {
  constexpr int N = Vec<BF>::N;
  if (K % N != 0 || ((uintptr_t)x % 16) != 0) return LCQ_EALIGN;
  const int64_t nch = K / N;
  int splits = (int)((T + 63) / 64);
  if (splits > PARTS_MAX) splits = PARTS_MAX;
  if (splits < 1) splits = 1;
  absmean_stage1<BF><<<dim3((unsigned)((nch + 255) / 256), (unsigned)splits), dim3(256), 0, st>>>((const u32x4*)x, T, K, part);
  absmean_stage2<BF><<<dim3((unsigned)((K + 255) / 256)), dim3(256), 0, st>>>(part, splits, mean_factor(T, K), K, out);
  return LCQ_OK;
}

template <int BF>
int wscale(const void* w, int64_t R, int64_t K, int g, void* out, float* part, hipStream_t st) {
  constexpr int N = Vec<BF>::N;
  if (K % N != 0 || g % N != 0 || K % g != 0 || ((uintptr_t)w % 16) != 0) return LCQ_EALIGN;
  const int team = g / N;
  int splits = (int)((R + 15) / 16);
  if (splits > PARTS_MAX) splits = PARTS_MAX;
  #define LCQ_WS(T) wscale_stage1<BF, T><<<dim3((unsigned)splits), dim3(256), 0, st>>>((const u32x4*)w, R, K, part)
  if (team == 1) LCQ_WS(1); else if (team == 2) LCQ_WS(2); else if (team == 4) LCQ_WS(4); else if (team == 8) LCQ_WS(8);
  else if (team == 16) LCQ_WS(16); else if (team == 32) LCQ_WS(32); else if (team == 64) LCQ_WS(64);
  else return LCQ_EINVAL;
  #undef LCQ_WS
  absmean_stage2<BF><<<dim3((unsigned)((K + 255) / 256)), dim3(256), 0, st>>>(part, splits, mean_factor(R, K), K, out);
  return LCQ_OK;
}

}  // namespace

extern "C" {

int64_t lcq_awq_workspace_bytes(int64_t K) { return (int64_t)PARTS_MAX * K * 4 + 8192 * 8; }

int lcq_absmean_cols(const void* x, int dtype, int64_t T, int64_t K, void* out, void* workspace, void* stream) {
  if (!x || !out || !workspace || T <= 0 || K <= 0) return LCQ_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (dtype == LCQ_F32) rc = absmean<false>(x, T, K, out, (float*)workspace, st);
  else if (dtype == LCQ_BF16) rc = absmean<true>(x, T, K, out, (float*)workspace, st);
  else if (dtype == LCQ_F16) rc = absmean<ROW_F16>(x, T, K, out, (float*)workspace, st);
  else return LCQ_EDTYPE;
  if (rc != LCQ_OK) return rc;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_awq_weight_scale(const void* w, int dtype, int64_t R, int64_t K, int group_size, void* out, void* workspace,
                         void* stream) {
  if (!w || !out || !workspace || R <= 0 || K <= 0 || group_size <= 0) return LCQ_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (dtype == LCQ_F32) rc = wscale<false>(w, R, K, group_size, out, (float*)workspace, st);
  else if (dtype == LCQ_BF16) rc = wscale<true>(w, R, K, group_size, out, (float*)workspace, st);
  else if (dtype == LCQ_F16) rc = wscale<ROW_F16>(w, R, K, group_size, out, (float*)workspace, st);
  else return LCQ_EDTYPE;
  if (rc != LCQ_OK) return rc;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_div_cols(const void* x, int dtype, int64_t T, int64_t K, const void* s, void* out, void* stream) {
  if (!x || !s || !out || T <= 0 || K <= 0) return LCQ_EINVAL;
  const int n = dtype == LCQ_F32 ? 4 : 8;
  if (dtype != LCQ_BF16 && dtype != LCQ_F32 && dtype != LCQ_F16) return LCQ_EDTYPE;
  if (K % n != 0 || (((uintptr_t)x | (uintptr_t)s | (uintptr_t)out) % 16) != 0) return LCQ_EALIGN;
  const int64_t nch_row = K / n, total = T * nch_row;
  int64_t grid = (total + 255) / 256;
  if (grid > 65536 * 4) grid = 65536 * 4;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LCQ_BF16) div_cols_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)x, (const u32x4*)s, total, nch_row, (u32x4*)out);
  else if (dtype == LCQ_F16) div_cols_kernel<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)x, (const u32x4*)s, total, nch_row, (u32x4*)out);
  else div_cols_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)x, (const u32x4*)s, total, nch_row, (u32x4*)out);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_scale_matrix(const void* x, int dtype, int64_t T, int64_t K, const void* s, int mode, void* out, void* stream) {
  if (!x || !s || !out || T <= 0 || K <= 0 || mode < 0 || mode > 3) return LCQ_EINVAL;
  const int n = dtype == LCQ_F32 ? 4 : 8;
  if (dtype != LCQ_BF16 && dtype != LCQ_F32 && dtype != LCQ_F16) return LCQ_EDTYPE;
  if (K % n != 0 || (((uintptr_t)x | (uintptr_t)out) % 16) != 0 || (mode < 2 && ((uintptr_t)s % 16) != 0)) return LCQ_EALIGN;
  const int64_t nch_row = K / n, total = T * nch_row;
  int64_t grid = (total + 255) / 256;
  if (grid > 65536 * 4) grid = 65536 * 4;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LCQ_BF16) scale_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)x, s, total, nch_row, mode, (u32x4*)out);
  else if (dtype == LCQ_F16) scale_kernel<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)x, s, total, nch_row, mode, (u32x4*)out);
  else scale_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)x, s, total, nch_row, mode, (u32x4*)out);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

static int sq_err_mean_launch(const void* a, const void* b, int dtype, int64_t n, float* out, double* part, hipStream_t st) {
  const int nn = dtype == LCQ_F32 ? 4 : 8;
  if (dtype != LCQ_BF16 && dtype != LCQ_F32 && dtype != LCQ_F16) return LCQ_EDTYPE;
  if (n % nn != 0 || (((uintptr_t)a | (uintptr_t)b) % 16) != 0) return LCQ_EALIGN;
  const int64_t nchunks = n / nn;
  int64_t grid = (nchunks + 255) / 256;
  if (grid > SQERR_PARTS_MAX) grid = SQERR_PARTS_MAX;
  if (dtype == LCQ_BF16) sqerr_stage1<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)a, (const u32x4*)b, nchunks, part);
  else if (dtype == LCQ_F16) sqerr_stage1<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)a, (const u32x4*)b, nchunks, part);
  else sqerr_stage1<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)a, (const u32x4*)b, nchunks, part);
  sqerr_stage2<<<dim3(1), dim3(256), 0, st>>>(part, (int)grid, (double)n, out);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_sq_err_mean(const void* a, const void* b, int dtype, int64_t n, float* out, void* workspace, void* stream) {
  if (!a || !b || !out || !workspace || n <= 0) return LCQ_EINVAL;
  return sq_err_mean_launch(a, b, dtype, n, out, (double*)workspace, (hipStream_t)stream);
}

int lcq_sq_err_mean_static(const void* a, const void* b, int dtype, int64_t n, float* out, void* stream) {
  if (!a || !b || !out || n <= 0) return LCQ_EINVAL;
  if (n > LCQ_SQ_ERR_STATIC_MAX_N) return LCQ_ESIZE;
  double* part = static_scratch();
  if (!part) return LCQ_ELAUNCH;
  // stage 1 writes every partial sum that stage 2 reads (the first `grid` entries), so nothing has to start at zero
  return sq_err_mean_launch(a, b, dtype, n, out, part, (hipStream_t)stream);
}

}  // extern "C"
