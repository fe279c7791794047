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
// The per-element division x/s is evaluated as x*(1/s) with an exactness
// guard: whenever the approximate quotient is close enough to a rounding
// boundary that the IEEE quotient could round differently, the lane falls
// back to the true division.  Both paths give the same bits by construction.
#include "rowquant.h"

namespace {
using namespace lcq;

struct IntRow {
  float s, z, r, sdq;
  float lo, hi;      // qmin - z, qmax - z: clamp bounds of the code minus the zero point
  int fast;          // x * (1/s) + guard may replace x / s
  int zint;          // zero point is a small integer: rint(t) + z and q - z are exact
};

// FAST: round_zp and |qmin|,qmax <= 256 (every stock configuration).
template <bool BF_, bool FAST, bool PRESCALE = false, int CD_ = -1>
struct IntOp {
  static constexpr bool BF = BF_;
  static constexpr bool HAS_PRESCALE = PRESCALE;
  static constexpr bool HAS_FUSED_DQ = FAST;
  static constexpr bool HAS_CUSTOM_EMIT = false;
  static constexpr int CD = CD_;
  using Row = IntRow;
  float qmin, qmax, qrange, osf;
  float rqmax, rqrange;         // 1 / qmax, 1 / qrange (fp32-rounded)
  int sym, round_zp, is_static, scalar_qp, dq_f32, code_dtype, range_bf16, scale_f32;
  // optional per-column factor applied first (AWQ: W * s), rows of the reshaped tensor tile a
  // weight row of wrow_cols columns
  const void* colscale;
  int wrow_cols;

  __device__ __forceinline__ float prescale1(float x, int64_t row, int64_t col, int64_t cols) const {
    const int64_t c = (row * cols + col) % wrow_cols;
    return rnd_e<BF>(x * load_scalar<BF>(colscale, c));
  }
  __device__ __forceinline__ u32x4 prescale(const u32x4& raw, int64_t row, int ch, int nchunks) const {
    constexpr int N = Vec<BF>::N;
    const int64_t c0 = ((row * nchunks + ch) * N) % wrow_cols;       // wrow_cols % N == 0 on this path
    const u32x4 sraw = *((const u32x4*)colscale + c0 / N);
    float v[N], sv[N];
    unpack<BF>(raw, v);
    unpack<BF>(sraw, sv);
    #pragma unroll
    for (int i = 0; i < N; ++i) v[i] = rnd_e<BF>(v[i] * sv[i]);
    return pack<BF>(v);
  }

  __device__ __forceinline__ Row finish(float s, float z) const {
    Row p;
    p.s = s; p.z = z;
    p.r = __builtin_amdgcn_rcpf(s);      // 1 ulp: inside the error the exactness guards of x * r allow for
    const float a = fabsf(s);
    p.fast = (a > 8.6736174e-19f) && (a < 1.1529215e18f) && (fabsf(z) <= 512.0f);   // s in 2^-60 .. 2^60
    p.zint = (z == rintf(z)) && (fabsf(z) <= 512.0f);       // caller-given zero points need not be integers
    p.sdq = scale_f32 ? s * osf : rnd<BF>(s * osf);
    p.lo = qmin - z; p.hi = qmax - z;                       // exact: small integers
    return p;
  }

  // a / c for a per-launch constant c (rc = 1/c rounded to fp32), rounded to the row type.  bf16 rows:
  // the product a * rc stands for the quotient unless it lies within 8 ulp of a bf16 rounding
  // midpoint; fp32 rows need the correctly rounded quotient itself.
  __device__ __forceinline__ float div_const(float a, float c, float rc) const {
    if constexpr (BF) {
      float q = a * rc;
      if (__builtin_expect(((f2u(q) & 0xffffu) - 0x7ff8u) <= 0x10u, 0)) q = a / c;
      return rnd<BF>(q);
    } else {
      return a / c;
    }
  }

  // get_qparams, quant.py:544-558
  __device__ __forceinline__ Row make(float mn, float mx) const {
    const float cmin = (BF || range_bf16) ? 1.0013580322265625e-05f : 1e-5f;   // clamp(min=1e-5) in the range dtype
    float s, z;
    if (sym) {
      float a = nan_max(fabsf(mx), fabsf(mn));
      a = clamp_min_nan(a, cmin);
      s = div_const(a, qmax, rqmax);
      z = 0.0f;
    } else {
      float d = rnd<BF>(mx - mn);
      if (range_bf16) d = bf16_round(d);
      d = clamp_min_nan(d, cmin);
      s = div_const(d, qrange, rqrange);
      // mn / s through the reciprocal, with the same exactness guards as the per-element quotients
      float t = mn * __builtin_amdgcn_rcpf(s);
      const float as = fabsf(s);
      bool ok = (as > 8.6736174e-19f) && (as < 1.1529215e18f);
      if constexpr (BF) {
        ok = ok && (((f2u(t) & 0xffffu) - 0x7ff8u) > 0x10u);
      } else {
        const float fr = t - rintf(t);
        ok = ok && (fabsf(fabsf(fr) - 0.5f) > 4.8828125e-04f) && (fabsf(t) <= 1024.0f) && round_zp;
      }
      if (__builtin_expect(!ok, 0)) t = mn / s;
      t = rnd<BF>(t);
      if (round_zp) {
        z = rnd<BF>(qmin - rintf(t));
        z = fminf(fmaxf(z, qmin), qmax);
      } else {
        z = rnd<BF>(qmin - t);
      }
    }
    return finish(s, z);
  }

  __device__ __forceinline__ Row load(const void* scales, const void* zeros, int64_t row) const {
    const int64_t i = scalar_qp ? 0 : row;
    if (scale_f32) return finish(((const float*)scales)[i], zeros ? ((const float*)zeros)[i] : 0.0f);
    const float s = load_scalar<BF>(scales, i);
    const float z = zeros ? load_scalar<BF>(zeros, i) : 0.0f;
    return finish(s, z);
  }

  __device__ __forceinline__ void store_qp(void* scales, void* zeros, int64_t row, const Row& p) const {
    if (scales) store_scalar<BF>(scales, row, p.s);
    if (zeros && !sym) store_scalar<BF>(zeros, row, p.z);
  }

  // quant, quant.py:698-707: the integer code as a float (element-wise form, any configuration)
  __device__ __forceinline__ float code(float x, const Row& p) const {
    float q;
    if (round_zp) {
      const float t = rnd<BF>(x / p.s);
      q = rnd<BF>(rintf(t) + p.z);
    } else {
      const float lo = BF ? 1.00044417e-09f : 1e-9f;         // scales.clamp_min(1e-9)
      const float t = rnd<BF>(x / clamp_min_nan(p.s, lo));
      q = rintf(rnd<BF>(t + p.z));
    }
    return __builtin_amdgcn_fmed3f(q, qmin, qmax);
  }

  // One 16-byte chunk.  FAST configurations (round_zp, |qmin|,qmax <= 256, |z| <= 512) evaluate
  // x/s as x*(1/s); the chunk falls back to IEEE divisions when any product lies so close to a
  // rounding boundary that the true quotient could round the other way:
  //   fp32: |t - x/s| <= 2^-22 |t|; for |t| <= 1024 that is <= 2^-12, so a product farther than
  //         2^-11 from every half integer rounds like the quotient; beyond 1024 both land outside
  //         the clamp range on the same side (|z| <= 512), and a huge t has d == 0;
  //   bf16: the quotient is rounded to bf16 first; the product is safe unless its low 16 bits
  //         are within 8 ulp of the bf16 midpoint pattern 0x8000.
  // x / s for a chunk, rounded to the row type
  template <int N>
  __device__ __forceinline__ void quotients(const float* x, float* t, const Row& p) const {
    bool ok = p.fast;
    #pragma unroll
    for (int i = 0; i < N; ++i) {
      t[i] = x[i] * p.r;
      if constexpr (BF) {
        ok = ok && (((f2u(t[i]) & 0xffffu) - 0x7ff8u) > 0x10u);
      } else {
        const float d = t[i] - rintf(t[i]);
        ok = ok && (fabsf(fabsf(d) - 0.5f) > 4.8828125e-04f);
      }
    }
    if (__builtin_expect(!ok, 0)) {
      #pragma unroll
      for (int i = 0; i < N; ++i) t[i] = x[i] / p.s;
    }
    #pragma unroll
    for (int i = 0; i < N; i += 2) rnd_pair<BF>(t[i], t[i + 1]);
  }

  template <int N>
  __device__ __forceinline__ void codes(const float* x, float* q, const Row& p) const {
    if constexpr (!FAST) {
      #pragma unroll
      for (int i = 0; i < N; ++i) q[i] = code(x[i], p);
    } else {
      if (__builtin_expect(!p.zint, 0)) {
        #pragma unroll
        for (int i = 0; i < N; ++i) q[i] = code(x[i], p);
        return;
      }
      float t[N];
      quotients<N>(x, t, p);
      #pragma unroll
      for (int i = 0; i < N; ++i)
        q[i] = __builtin_amdgcn_fmed3f(rintf(t[i]) + p.z, qmin, qmax);
    }
  }

  // fake quant without the codes (FAST only): (clamp(rint(t) + z, qmin, qmax) - z) * s equals
  // clamp(rint(t), qmin - z, qmax - z) * s when z is a small integer (all terms exact); "+ 0" turns the
  // -0 that rint(-0.3) leaves into the +0 that (q - z) gives.  The products are left unrounded: the
  // caller rounds to the row type while packing.
  template <int N>
  __device__ __forceinline__ void fused_dq(const float* x, float* d, const Row& p) const {
    if (__builtin_expect(!p.zint, 0)) {
      #pragma unroll
      for (int i = 0; i < N; ++i) d[i] = deq_raw(code(x[i], p), p);
      return;
    }
    float t[N];
    quotients<N>(x, t, p);
    #pragma unroll
    for (int i = 0; i < N; ++i) d[i] = (__builtin_amdgcn_fmed3f(rintf(t[i]), p.lo, p.hi) + 0.0f) * p.sdq;
  }

  // dequant, quant.py:709-711 (scale already multiplied by output_scale_factor)
  __device__ __forceinline__ float deq_raw(float q, const Row& p) const {   // before the rounding to the row type
    float d = q - p.z;                                       // exact for small integer codes
    if constexpr (BF) { if (!FAST || !p.zint) d = bf16_round(d); }
    return d * p.sdq;
  }
  __device__ __forceinline__ float deq(float q, const Row& p) const { return rnd_e<BF>(deq_raw(q, p)); }

  __device__ __forceinline__ uint32_t byte(float q) const { return (uint32_t)(int32_t)q & 0xffu; }
  __device__ __forceinline__ uint32_t pack4(const float* q) const {
    uint32_t w = 0;
    if ((CD >= 0 ? CD : code_dtype) == LCQ_CODE_U8) {        // integral values in [0, 255]: v_cvt_pk_u8_f32
      #pragma unroll
      for (int j = 0; j < 4; ++j) w = __builtin_amdgcn_cvt_pk_u8_f32(q[j], j, w);
    } else {
      #pragma unroll
      for (int j = 0; j < 4; ++j) w |= byte(q[j]) << (8 * j);
    }
    return w;
  }
};

template <class Op>
Op make_op(float qmin, float qmax, int flags, float osf, int code_dtype) {
  Op c;
  c.qmin = qmin; c.qmax = qmax; c.qrange = qmax - qmin; c.osf = osf;
  c.rqmax = (float)(1.0 / (double)qmax); c.rqrange = (float)(1.0 / (double)(qmax - qmin));
  c.sym = (flags & LCQ_FLAG_SYM) != 0;
  c.round_zp = (flags & LCQ_FLAG_NO_ROUND_ZP) == 0;
  c.is_static = (flags & LCQ_FLAG_STATIC) != 0;
  c.scalar_qp = (flags & LCQ_FLAG_SCALAR_QP) != 0;
  c.dq_f32 = 0;
  c.range_bf16 = (flags & LCQ_FLAG_RANGE_BF16) != 0;
  c.scale_f32 = (flags & LCQ_FLAG_SCALE_F32) != 0;
  c.colscale = nullptr; c.wrow_cols = 1;
  c.code_dtype = code_dtype;
  return c;
}

template <bool BF>
int run(const void* x, int64_t rows, int64_t cols, float qmin, float qmax, int flags, float osf, void* dq,
        void* codes, int code_dtype, void* scales, void* zeros, hipStream_t st) {
  const bool big = (qmax > 256.0f) || (qmin < -256.0f);
  const bool general = big || (flags & LCQ_FLAG_NO_ROUND_ZP);
  if (general)
    return dispatch_rows(x, rows, cols, dq, codes, scales, zeros,
                         make_op<IntOp<BF, false>>(qmin, qmax, flags, osf, code_dtype), true, st);
  // the common storage formats get kernels with the store path fixed at compile time
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

// get_minmax_range (row-wise), quant.py:141-143
template <bool BF>
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
template <bool BF>
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
template <bool BF>
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
template <bool BF>
__global__ void qparams_kernel(const void* __restrict__ mn, const void* __restrict__ mx, int64_t n,
                               void* __restrict__ scales, void* __restrict__ zeros, IntOp<BF, false> op) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const IntRow p = op.make(load_scalar<BF>(mn, i), load_scalar<BF>(mx, i));
  op.store_qp(scales, zeros, i, p);
}

// dequant, quant.py:709-711, on stored float codes
template <bool BF>
__global__ __launch_bounds__(256) void dequant_kernel(const void* __restrict__ q, int64_t rows, int64_t cols,
                                                      const void* __restrict__ scales, const void* __restrict__ zeros,
                                                      void* __restrict__ out, int scalar_qp, int scale_f32, float osf) {
  const int64_t n = rows * cols;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
    const int64_t row = scalar_qp ? 0 : e / cols;
    const float s = scale_f32 ? ((const float*)scales)[row] : load_scalar<BF>(scales, row);
    const float z = !zeros ? 0.0f : (scale_f32 ? ((const float*)zeros)[row] : load_scalar<BF>(zeros, row));
    const float d = rnd<BF>(load_scalar<BF>(q, e) - z);
    store_scalar<BF>(out, e, rnd<BF>(d * (scale_f32 ? s * osf : rnd<BF>(s * osf))));
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
  else return LCQ_EDTYPE;
  if (rc != LCQ_OK) return rc;
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
  const int n = dtype == LCQ_BF16 ? 8 : 4;
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
  else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
