// Integer quantizer for gfx950: row-wise min/max -> scale/zero -> quantize ->
// dequantize / integer codes in ONE pass over HBM (skeleton in rowquant.h).
//
// Replaces the ~9 eager torch kernels behind
//   IntegerQuantizer.get_tensor_qparams / quant / dequant / quant_dequant /
//   fake_quant_*_dynamic|static / real_quant_weight_dynamic|static
// (llmc/compression/quantization/quant.py:134-145, 544-558, 689-716, 753-952).
//
// A "row" is one row of the reshaped tensor (quant.py:611-641): a group of
// `group_size` weights (per_group), a whole weight row (per_channel), a token
// (per_token) or a head (per_head).
//
// Arithmetic contract (bit-exact with the reference's torch op sequence):
//   fp32 rows : every step is one IEEE fp32 op (true division, rintf).
//   bf16 rows : every step is computed in fp32 and rounded to bf16 (RNE)
//               before the next step, as torch does for bf16 tensors.
//   fp16 rows : the same with fp16 roundings, through the element-wise kernel and true divisions only (one wave per
//               row, one element per lane and step: a compatibility path, not a tuned one).
// The per-element division x/s is evaluated as x*(1/s) with an exactness
// guard: whenever the approximate quotient is close enough to a rounding
// boundary that the IEEE quotient could round differently, the lane falls
// back to the true division.  Both paths give the same bits by construction.
#include "intop.h"

namespace {
using namespace lcq;

template <int BF>
int run(const void* x, int64_t rows, int64_t cols, float qmin, float qmax, int flags, float osf, void* dq,
        void* codes, int code_dtype, void* scales, void* zeros, hipStream_t st) {
  const bool big = (qmax > 256.0f) || (qmin < -256.0f);
  const bool general = big || (flags & LCQ_FLAG_NO_ROUND_ZP) || BF == ROW_F16;     // fp16 rows: the element-wise kernel
  if constexpr (BF == ROW_F16) {
    if (code_dtype == LCQ_CODE_CT4) return LCQ_EDTYPE;      // nibbles come from the vectorised bf16 / fp32 kernels only
  }
  if (general)
    return dispatch_rows(x, rows, cols, dq, codes, scales, zeros,
                         make_op<IntOp<BF, false>>(qmin, qmax, flags, osf, code_dtype), true, st);
  // the common storage formats get kernels with the store path fixed at compile time
  if constexpr (BF == ROW_F16) return LCQ_EDTYPE;            // not reached: `general` above
  else {
  #define LCQ_RUN(CDV) return dispatch_rows(x, rows, cols, dq, codes, scales, zeros, \
                         make_op<IntOp<BF, true, false, CDV>>(qmin, qmax, flags, osf, code_dtype), false, st)
  switch (code_dtype) {
    case LCQ_CODE_NONE: LCQ_RUN(LCQ_CODE_NONE);
    case LCQ_CODE_U8: LCQ_RUN(LCQ_CODE_U8);
    case LCQ_CODE_I32: LCQ_RUN(LCQ_CODE_I32);
    case LCQ_CODE_CT4: LCQ_RUN(LCQ_CODE_CT4);
    default: LCQ_RUN(-1);
  }
  #undef LCQ_RUN
  }
}

// get_minmax_range (row-wise), quant.py:141-143
template <int BF>
__global__ __launch_bounds__(256) void minmax_rows_kernel(const void* __restrict__ x, int64_t rows, int64_t cols,
                                                          void* __restrict__ mn_out, void* __restrict__ mx_out) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= rows) return;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int64_t j = lane; j < cols; j += 64) {
    const float v = load_scalar<BF>(x, row * cols + j);
    mn = nan_min(mn, v); mx = nan_max(mx, v);
  }
  mn = team_reduce<64, false>(mn);
  mx = team_reduce<64, true>(mx);
  if (lane == 0) { store_scalar<BF>(mn_out, row, mn); store_scalar<BF>(mx_out, row, mx); }
}

// per_tensor range, quant.py:135-137: stage 1 writes one (min,max) per workgroup
template <int BF>
__global__ __launch_bounds__(256) void minmax_all_stage1(const void* __restrict__ x, int64_t n, float* __restrict__ part) {
  __shared__ float sm[8];
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x; j < n; j += (int64_t)gridDim.x * 256) {
    const float v = load_scalar<BF>(x, j);
    mn = nan_min(mn, v); mx = nan_max(mx, v);
  }
  mn = block_reduce<false>(mn, sm);
  mx = block_reduce<true>(mx, sm);
  if (threadIdx.x == 0) { part[2 * blockIdx.x] = mn; part[2 * blockIdx.x + 1] = mx; }
}
template <int BF>
__global__ __launch_bounds__(256) void minmax_all_stage2(const float* __restrict__ part, int nparts,
                                                         void* __restrict__ mn_out, void* __restrict__ mx_out) {
  __shared__ float sm[8];
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int j = threadIdx.x; j < nparts; j += 256) { mn = nan_min(mn, part[2 * j]); mx = nan_max(mx, part[2 * j + 1]); }
  mn = block_reduce<false>(mn, sm);
  mx = block_reduce<true>(mx, sm);
  if (threadIdx.x == 0) { store_scalar<BF>(mn_out, 0, mn); store_scalar<BF>(mx_out, 0, mx); }
}

// get_qparams on explicit ranges, quant.py:544-558
template <int BF>
__global__ void qparams_kernel(const void* __restrict__ mn, const void* __restrict__ mx, int64_t n,
                               void* __restrict__ scales, void* __restrict__ zeros, IntOp<BF, false> op) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const IntRow p = op.make(load_scalar<BF>(mn, i), load_scalar<BF>(mx, i));
  op.store_qp(scales, zeros, i, p);
}

// dequant, quant.py:709-711, on stored float codes
template <int BF>
__global__ __launch_bounds__(256) void dequant_kernel(const void* __restrict__ q, int64_t rows, int64_t cols,
                                                      const void* __restrict__ scales, const void* __restrict__ zeros,
                                                      void* __restrict__ out, int scalar_qp, int scale_f32, float osf) {
  const int64_t n = rows * cols;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
    const int64_t row = scalar_qp ? 0 : e / cols;
    // fp32 parameters (0-dim next to a 16-bit tensor) are rounded to the row type where they meet the rows
    const float s = scale_f32 ? ((const float*)scales)[row] : load_scalar<BF>(scales, row);
    const float z = !zeros ? 0.0f : (scale_f32 ? rnd<BF>(((const float*)zeros)[row]) : load_scalar<BF>(zeros, row));
    const float d = rnd<BF>(load_scalar<BF>(q, e) - z);
    store_scalar<BF>(out, e, rnd<BF>(d * rnd<BF>(s * osf)));
  }
}

// get_mse_range, quant.py:147-205: per row, shrink steps i = 0 .. steps-1 with p = 1 - i / grid:
//   xmin = p * cur_min, xmax = p * cur_max;  err = sum_j |quant_dequant(x_j; xmin, xmax) - x_j| ^ norm
//   err < best  ->  best = err, cur_min = xmin, cur_max = xmax
// cur_min / cur_max start as the row's min / max and - as in the reference, whose best_min_val / best_max_val
// alias the range tensors - are the values the NEXT step shrinks.  All arithmetic in fp32 (tensor.float()).
// One wave per row; the row is re-read from L1/L2 on every step.
template <int BF>
__global__ __launch_bounds__(256) void mse_range_kernel(const void* __restrict__ x, int64_t rows, int64_t cols, int steps,
                                                        int grid_n, float norm, IntOp<0, false> op,
                                                        float* __restrict__ mn_out, float* __restrict__ mx_out) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int64_t j = lane; j < cols; j += 64) {
    const float v = load_scalar<BF>(x, row * cols + j);
    mn = nan_min(mn, v); mx = nan_max(mx, v);
  }
  float cur_min = team_reduce<64, false>(mn), cur_max = team_reduce<64, true>(mx);
  float best = __builtin_inff();
  for (int i = 0; i < steps; ++i) {
    const float p = (float)(1.0 - (double)i / (double)grid_n);
    const float xmin = p * cur_min, xmax = p * cur_max;
    const IntRow prm = op.make(xmin, xmax);
    float err = 0.0f;
    for (int64_t j = lane; j < cols; j += 64) {
      const float v = load_scalar<BF>(x, row * cols + j);
      const float d = fabsf(op.deq(op.code(v, prm), prm) - v);
      err += __builtin_powf(d, norm);
    }
    err = team_sum<64>(err);
    if (err < best) { best = err; cur_min = xmin; cur_max = xmax; }
  }
  if (lane == 0) { mn_out[row] = cur_min; mx_out[row] = cur_max; }
}

// One proximal iteration of the HQQ zero-point solver (optimize_weights_proximal, quant.py:587-609):
//   W_q = clamp(round(x * inv_s + z), qmin, qmax);  W_r = (W_q - z) / inv_s;  W_e = shrink(x - W_r)
//   z'  = mean(W_q - (x - W_e) * inv_s)  per row;   abs_err = sum |x - W_r|  per row
// with inv_s = 1 / s and shrink(d) = sign(d) * relu(|d| - inv_beta * |d|^(p-1))  (p == 1: |d| - inv_beta).
// One pass over x; LANES lanes share a row and combine their partial sums with a DPP butterfly.
template <int LANES>
__global__ __launch_bounds__(256) void hqq_step_kernel(const float* __restrict__ x, long long rows, int cols,
                                                       const float* __restrict__ scales, const float* __restrict__ zeros_in,
                                                       float* __restrict__ zeros_out, float* __restrict__ abs_err,
                                                       float* __restrict__ scales_rt, float inv_beta, float p, float qmin,
                                                       float qmax) {
  const int lane = threadIdx.x % LANES;
  const long long row = (long long)blockIdx.x * (256 / LANES) + threadIdx.x / LANES;
  const bool ok = row < rows;
  const long long r = ok ? row : 0;
  const float inv_s = 1.0f / scales[r];
  const float z = zeros_in ? zeros_in[r] : 0.0f;
  const float* xr = x + r * cols;
  float acc_z = 0.0f, acc_e = 0.0f;
  for (int c = lane; c < cols; c += LANES) {
    const float v = xr[c];
    const float wq = __builtin_amdgcn_fmed3f(rintf(v * inv_s + z), qmin, qmax);
    const float wr = (wq - z) / inv_s;
    const float d = v - wr;
    const float ad = fabsf(d);
    const float thr = (p == 1.0f) ? inv_beta : inv_beta * powf(ad, p - 1.0f);
    const float mag = fmaxf(ad - thr, 0.0f);
    const float sgn = (d > 0.0f) ? 1.0f : ((d < 0.0f) ? -1.0f : 0.0f);
    const float we = sgn * mag;
    acc_z += wq - (v - we) * inv_s;
    acc_e += ad;
  }
  acc_z = team_sum<LANES>(acc_z);
  acc_e = team_sum<LANES>(acc_e);
  if (ok && lane == 0) {
    zeros_out[row] = acc_z * (1.0f / (float)cols);      // torch.mean on the GPU: the sum times an fp32 factor
    abs_err[row] = acc_e;
    if (scales_rt) scales_rt[row] = 1.0f / inv_s;
  }
}

}  // namespace

extern "C" {

int lcq_quant_int(const void* x, int dtype, int64_t rows, int64_t cols, float qmin, float qmax, int flags,
                  float out_scale_factor, void* dq, void* codes, int code_dtype, void* scales, void* zeros,
                  void* stream) {
  if (!x || rows < 0 || cols <= 0 || !scales) return LCQ_EINVAL;
  if (rows == 0) return LCQ_OK;
  if (codes && !(code_dtype == LCQ_CODE_U8 || code_dtype == LCQ_CODE_I8 || code_dtype == LCQ_CODE_I32 ||
                 code_dtype == LCQ_CODE_SAME || code_dtype == LCQ_CODE_CT4)) return LCQ_EDTYPE;
  if (!(qmax > qmin)) return LCQ_EINVAL;
  if (codes && code_dtype == LCQ_CODE_CT4) {
    // only the vectorised kernels store nibbles: 16-byte chunks, codes + 8 within a nibble
    if (qmin < -8.0f || qmax > 7.0f || (flags & LCQ_FLAG_NO_ROUND_ZP) || cols % 8 != 0) return LCQ_EINVAL;
    if ((((uintptr_t)x | (uintptr_t)dq) % 16) != 0 || ((uintptr_t)codes % 4) != 0) return LCQ_EALIGN;
  }
  if ((flags & LCQ_FLAG_SCALAR_QP) && !(flags & LCQ_FLAG_STATIC)) return LCQ_EINVAL;
  if ((flags & LCQ_FLAG_SCALE_F32) && !(flags & LCQ_FLAG_STATIC)) return LCQ_EINVAL;
  if (!codes) code_dtype = LCQ_CODE_NONE;
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (dtype == LCQ_F32) rc = run<false>(x, rows, cols, qmin, qmax, flags, out_scale_factor, dq, codes, code_dtype, scales, zeros, st);
  else if (dtype == LCQ_BF16) rc = run<true>(x, rows, cols, qmin, qmax, flags, out_scale_factor, dq, codes, code_dtype, scales, zeros, st);
  else if (dtype == LCQ_F16) rc = run<ROW_F16>(x, rows, cols, qmin, qmax, flags, out_scale_factor, dq, codes, code_dtype, scales, zeros, st);
  else return LCQ_EDTYPE;
  if (rc != LCQ_OK) return rc;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_mse_range(const void* x, int dtype, int64_t rows, int64_t cols, float qmin, float qmax, int flags, int steps,
                  int grid_n, float norm, float* min_out, float* max_out, void* stream) {
  if (!x || !min_out || !max_out || rows <= 0 || cols <= 0 || steps <= 0 || grid_n <= 0) return LCQ_EINVAL;
  if (!(qmax > qmin) || (flags & LCQ_FLAG_STATIC)) return LCQ_EINVAL;
  auto op = make_op<IntOp<false, false>>(qmin, qmax, flags, 1.0f, LCQ_CODE_NONE);
  const int64_t grid = (rows + 3) / 4;
  if (grid > 0x7fffffff) return LCQ_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LCQ_F32) mse_range_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, rows, cols, steps, grid_n, norm, op, min_out, max_out);
  else if (dtype == LCQ_BF16) mse_range_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, rows, cols, steps, grid_n, norm, op, min_out, max_out);
  else if (dtype == LCQ_F16) mse_range_kernel<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, rows, cols, steps, grid_n, norm, op, min_out, max_out);
  else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_hqq_step(const float* x, int64_t rows, int64_t cols, const float* scales, const float* zeros_in, float* zeros_out,
                 float* abs_err_rowsum, float* scales_roundtrip, float inv_beta, float lp_norm, float qmin, float qmax,
                 void* stream) {
  if (!x || !scales || !zeros_out || !abs_err_rowsum || rows <= 0 || cols <= 0 || cols > 0x7fffffff) return LCQ_EINVAL;
  if (!(qmax > qmin) || zeros_in == zeros_out) return LCQ_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  if (cols <= 256) {
    const int64_t grid = (rows + 15) / 16;
    if (grid > 0x7fffffff) return LCQ_EINVAL;
    hqq_step_kernel<16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, rows, (int)cols, scales, zeros_in, zeros_out,
                                                                     abs_err_rowsum, scales_roundtrip, inv_beta, lp_norm, qmin, qmax);
  } else {
    const int64_t grid = (rows + 3) / 4;
    if (grid > 0x7fffffff) return LCQ_EINVAL;
    hqq_step_kernel<64><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, rows, (int)cols, scales, zeros_in, zeros_out,
                                                                     abs_err_rowsum, scales_roundtrip, inv_beta, lp_norm, qmin, qmax);
  }
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_awq_scale_quant(const void* w, int dtype, int64_t R, int64_t K, const void* colscale, int group_size,
                        float qmin, float qmax, int flags, void* out, void* stream) {
  if (!w || !colscale || !out || R <= 0 || K <= 0 || K > 0x7fffffff) return LCQ_EINVAL;
  if (!(qmax > qmin) || (flags & (LCQ_FLAG_STATIC | LCQ_FLAG_NO_ROUND_ZP))) return LCQ_EINVAL;
  if (qmax > 256.0f || qmin < -256.0f) return LCQ_EINVAL;
  const int64_t cols = group_size > 0 ? group_size : K;
  if (K % cols != 0) return LCQ_EINVAL;
  const int64_t rows = R * (K / cols);
  const int n = dtype == LCQ_F32 ? 4 : 8;
  if (cols % n != 0 || K % n != 0 || ((uintptr_t)colscale % 16) != 0) return LCQ_EALIGN;
  hipStream_t st = (hipStream_t)stream;
  int rc;
  // the group scales / zeros stay in registers: fake_quantize_weight does not return them
  if (dtype == LCQ_F32) {
    auto op = make_op<IntOp<false, true, true>>(qmin, qmax, flags, 1.0f, LCQ_CODE_NONE);
    op.colscale = colscale; op.wrow_cols = (int)K; op.is_static = 0;
    rc = dispatch_rows(w, rows, cols, out, (void*)nullptr, (void*)nullptr, (void*)nullptr, op, false, st);
  } else if (dtype == LCQ_BF16) {
    auto op = make_op<IntOp<true, true, true>>(qmin, qmax, flags, 1.0f, LCQ_CODE_NONE);
    op.colscale = colscale; op.wrow_cols = (int)K; op.is_static = 0;
    rc = dispatch_rows(w, rows, cols, out, (void*)nullptr, (void*)nullptr, (void*)nullptr, op, false, st);
  } else if (dtype == LCQ_F16) {                           // element-wise kernel
    auto op = make_op<IntOp<ROW_F16, false, true>>(qmin, qmax, flags, 1.0f, LCQ_CODE_NONE);
    op.colscale = colscale; op.wrow_cols = (int)K; op.is_static = 0;
    rc = dispatch_rows(w, rows, cols, out, (void*)nullptr, (void*)nullptr, (void*)nullptr, op, true, st);
  } else return LCQ_EDTYPE;
  if (rc != LCQ_OK) return rc;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_minmax_rows(const void* x, int dtype, int64_t rows, int64_t cols, void* min_out, void* max_out, void* stream) {
  if (!x || !min_out || !max_out || rows < 0 || cols <= 0) return LCQ_EINVAL;
  if (rows == 0) return LCQ_OK;
  const int64_t grid = (rows + 3) / 4;
  if (grid > 0x7fffffff) return LCQ_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LCQ_F32) minmax_rows_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, rows, cols, min_out, max_out);
  else if (dtype == LCQ_BF16) minmax_rows_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, rows, cols, min_out, max_out);
  else if (dtype == LCQ_F16) minmax_rows_kernel<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, rows, cols, min_out, max_out);
  else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int64_t lcq_minmax_all_workspace_bytes(void) { return 2 * 2048 * sizeof(float); }

int lcq_minmax_all(const void* x, int dtype, int64_t n, void* min_out, void* max_out, void* workspace, void* stream) {
  if (!x || !min_out || !max_out || !workspace || n <= 0) return LCQ_EINVAL;
  int64_t blocks = (n + 256 * 16 - 1) / (256 * 16);
  if (blocks > 2048) blocks = 2048;
  hipStream_t st = (hipStream_t)stream;
  float* part = (float*)workspace;
  if (dtype == LCQ_F32) {
    minmax_all_stage1<false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(x, n, part);
    minmax_all_stage2<false><<<dim3(1), dim3(256), 0, st>>>(part, (int)blocks, min_out, max_out);
  } else if (dtype == LCQ_BF16) {
    minmax_all_stage1<true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(x, n, part);
    minmax_all_stage2<true><<<dim3(1), dim3(256), 0, st>>>(part, (int)blocks, min_out, max_out);
  } else if (dtype == LCQ_F16) {
    minmax_all_stage1<ROW_F16><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(x, n, part);
    minmax_all_stage2<ROW_F16><<<dim3(1), dim3(256), 0, st>>>(part, (int)blocks, min_out, max_out);
  } else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_qparams_int(const void* min_in, const void* max_in, int dtype, int64_t n, float qmin, float qmax, int flags,
                    void* scales, void* zeros, void* stream) {
  if (!min_in || !max_in || !scales || n <= 0) return LCQ_EINVAL;
  const int64_t grid = (n + 255) / 256;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LCQ_F32)
    qparams_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>(
        min_in, max_in, n, scales, zeros, make_op<IntOp<false, false>>(qmin, qmax, flags, 1.0f, LCQ_CODE_NONE));
  else if (dtype == LCQ_BF16)
    qparams_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>(
        min_in, max_in, n, scales, zeros, make_op<IntOp<true, false>>(qmin, qmax, flags, 1.0f, LCQ_CODE_NONE));
  else if (dtype == LCQ_F16)
    qparams_kernel<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(
        min_in, max_in, n, scales, zeros, make_op<IntOp<ROW_F16, false>>(qmin, qmax, flags, 1.0f, LCQ_CODE_NONE));
  else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_dequant_int(const void* q, int dtype, int64_t rows, int64_t cols, const void* scales, const void* zeros,
                    int flags, float out_scale_factor, void* out, void* stream) {
  if (!q || !scales || !out || rows < 0 || cols <= 0) return LCQ_EINVAL;
  if (rows == 0) return LCQ_OK;
  const int scalar_qp = (flags & LCQ_FLAG_SCALAR_QP) != 0;
  const int scale_f32 = (flags & LCQ_FLAG_SCALE_F32) != 0;
  int64_t grid = (rows * cols + 255) / 256;
  if (grid > 65536) grid = 65536;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LCQ_F32) dequant_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>(q, rows, cols, scales, zeros, out, scalar_qp, scale_f32, out_scale_factor);
  else if (dtype == LCQ_BF16) dequant_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>(q, rows, cols, scales, zeros, out, scalar_qp, scale_f32, out_scale_factor);
  else if (dtype == LCQ_F16) dequant_kernel<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(q, rows, cols, scales, zeros, out, scalar_qp, scale_f32, out_scale_factor);
  else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
