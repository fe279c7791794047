// Minifloat ("FPx": e4m3, e5m2, e2m1, e3m2, e4m7) quantizer for gfx950,
// the qtorch branch of FloatQuantizer:
//   get_tensor_qparams / quant / dequant / quant_dequant, fake_quant_*_dynamic|
//   static, real_quant_weight_dynamic|static
// (llmc/compression/quantization/quant.py:962-1002, 1042-1080, 1099-1220).
//
// Per row:  s = clamp(absmax, 1e-5) / qmax ;  per element:
//   t = x / s + 0.0            (in the row dtype: bf16 rows round to bf16)
//   q = float_quantize(float(t), e_bits, m_bits, 'nearest')   (fp32, on the grid)
//   dq = (q - 0.0) * s         (fp32 arithmetic, then cast to the output type)
//
// float_quantize is third-party (QPyTorch); its algorithm on the fp32 bit
// pattern is restated here: add half of the dropped-mantissa ulp and truncate
// (ties away from zero; LCQ_FLAG_TIE_EVEN switches to round-half-even, which
// is what a native float8 cast does), fixed-step rounding below the minimum
// normal (LCQ_FLAG_NO_SUBNORMALS flushes instead), exponent clipped at
// 2^(e_bits-1).
#include "rowquant.h"

namespace {
using namespace lcq;

struct FpRow {
  float s, r, sm;   // divisor, its reciprocal, multiplier of the dequantization
  int fast;
  int inrange;      // dynamic rows: every |x / s| of the row stays below hw_lim, no per-element check needed
};

template <int BF_>
struct FpOp {
  static constexpr int BF = BF_;          // row type: 0 fp32, 1 bf16, 2 fp16 (element-wise forms only)
  static constexpr bool HAS_PRESCALE = false;
  static constexpr bool HAS_FUSED_DQ = false;
  static constexpr bool HAS_CUSTOM_EMIT = true;
  static constexpr bool ABS_ONLY = true;
  static constexpr int CD = -1;
  using Row = FpRow;
  float qmax, rqmax;
  int e_bits, m_bits, tie_even, subnormals;
  int is_static, scalar_qp, dq_f32, code_dtype, scale_f32;
  // derived
  uint32_t half, keep, max_mag;
  int drop, min_exp, max_exp;
  float min_normal;
  int hw;            // 1: e4m3, 2: e5m2 with subnormals -> v_cvt_pk_fp8_f32 / v_cvt_pk_bf8_f32 do the rounding
  float hw_lim;      // quotients below this stay inside the float8 range (bf16 rows: also after their rounding to bf16)

  __device__ __forceinline__ Row finish(float s) const {
    Row p;
    if (s == 0.0f) s = 1.0f;                               // scales[scales == 0] = 1, quant.py:1061
    p.sm = s;
    p.s = s;
    p.r = __builtin_amdgcn_rcpf(s);      // 1 ulp: inside the error the exactness guards of x * r allow for
    const float a = fabsf(s);
    p.fast = (a > 8.6736174e-19f) && (a < 1.1529215e18f);
    p.inrange = 0;
    return p;
  }
  // get_qparams symmetric branch, quant.py:548-552 (qmax is a float tensor here)
  __device__ __forceinline__ Row make(float mn, float mx) const {
    const float cmin = BF ? 1.0013580322265625e-05f : 1e-5f;
    const float amax = nan_max(fabsf(mx), fabsf(mn));
    const float a = clamp_min_nan(amax, cmin);
    Row p;
    if constexpr (BF == ROW_BF16) {                       // a * (1/qmax) unless the product is within 8 ulp of a bf16 midpoint
      float q = a * rqmax;
      if (__builtin_expect(((f2u(q) & 0xffffu) - 0x7ff8u) <= 0x10u, 0)) q = a / qmax;
      p = finish(rnd<BF>(q));
    } else {
      p = finish(rnd<BF>(a / qmax));
    }
    // the largest quotient of the row, with room for the reciprocal's and the product's rounding (NaN: false)
    p.inrange = (amax * p.r) * 1.001f < hw_lim;
    return p;
  }
  __device__ __forceinline__ Row load(const void* scales, const void*, int64_t row) const {
    const int64_t i = scalar_qp ? 0 : row;
    if (scale_f32) {
      // a 0-dim fp32 scale next to a 16-bit tensor: the quotient sees it rounded to the row type (torch on a GPU
      // converts a 0-dim tensor operand first), the dequantization multiplies the fp32 codes by it as it is
      // (scales[scales == 0] = 1 acts on the fp32 value; a scale that only the rounding turns into 0 divides as 0)
      Row p = finish(((const float*)scales)[i]);
      const float s32 = p.s;
      p.s = rnd<BF>(s32);
      p.r = __builtin_amdgcn_rcpf(p.s);
      const float a = fabsf(p.s);
      p.fast = (a > 8.6736174e-19f) && (a < 1.1529215e18f);
      p.sm = s32;
      return p;
    }
    return finish(load_scalar<BF>(scales, i));
  }
  __device__ __forceinline__ void store_qp(void* scales, void*, int64_t row, const Row& p) const {
    store_scalar<BF>(scales, row, p.s);
  }

  __device__ __forceinline__ uint32_t round_mag(uint32_t m) const {
    if (tie_even) return (m + half - 1u + ((m >> drop) & 1u)) & keep;
    return (m + half) & keep;
  }

  // rounding of an fp32 value to the (e_bits, m_bits) grid
  __device__ __forceinline__ float grid_round(float t) const {
    const uint32_t bits = f2u(t);
    const uint32_t sign = bits & 0x80000000u;
    const uint32_t mag = bits & 0x7fffffffu;
    const int ex = (int)(mag >> 23) - 127;
    uint32_t out;
    if (ex == 128) {
      out = mag;                                           // inf / nan pass through
    } else if (ex < min_exp) {
      float v;
      if (subnormals) {
        const float sh = u2f(mag) + min_normal;
        v = u2f(round_mag(f2u(sh))) - min_normal;
      } else {
        v = (u2f(mag) > 0.5f * min_normal) ? min_normal : 0.0f;
      }
      out = f2u(v);
    } else {
      out = round_mag(mag);
      if ((int)(out >> 23) - 127 > max_exp) out = max_mag;
    }
    return u2f(out | sign);
  }

  __device__ __forceinline__ float code(float x, const Row& p) const {
    float t = x * p.r;
    bool ok;
    if constexpr (BF == ROW_F16) {
      ok = false;                                          // fp16 rows: always the division
    } else if constexpr (BF == ROW_BF16) {
      const uint32_t low = f2u(t) & 0xffffu;               // bf16 rounding midpoint nearby?
      ok = (low - 0x7ff8u) > 0x10u;
    } else {
      // grid midpoints sit at mantissa pattern 1000.. below the kept bits; the
      // sub-minimum-normal range uses absolute steps, so it always divides.
      const uint32_t lowm = f2u(t) & ((1u << drop) - 1u);
      ok = ((lowm - (half - 8u)) > 16u) && (fabsf(t) >= 1.0001f * min_normal);
    }
    ok = ok && p.fast;
    if (__builtin_expect(!ok, 0)) t = x / p.s;
    t = rnd_e<BF>(t);
    t = t + 0.0f;                                          // "+ zeros": turns -0 into +0
    return grid_round(t);
  }

  template <int N>
  __device__ __forceinline__ void codes(const float* x, float* q, const Row& p) const {
    #pragma unroll
    for (int i = 0; i < N; ++i) q[i] = code(x[i], p);
  }

  // One chunk through the hardware float8 converts (OCP e4m3fn / e5m2: round to nearest even,
  // subnormals, checked against torch's casts for every bf16 value).  Used when the whole chunk is
  // clear of every case where the converts and the emulated grid could disagree:
  //   * a quotient x*(1/s) too close to a rounding boundary to stand for x/s (as in code());
  //   * |t| >= hw_lim (the grid continues past the float8 maximum), inf, NaN;
  //   * fp32 rows: an exact tie (ties-away differs from the hardware's ties-even) or a value below
  //     the minimum normal - both are inside the boundary test above.
  // bf16 rows hold ties all the time (8 significant bits), so ties-away is produced by the convert
  // itself: t is scaled by 1 + 2^-10 first.  Every tie is a bf16 number, so a bf16 value that is
  // not a tie is at least one bf16 ulp away from the nearest one and the nudge (1/4 ulp at most)
  // cannot carry it across; an exact tie moves to the far side.  The fma also adds the "+ zeros"
  // of the reference, which turns -0 into +0.
  template <int N>
  __device__ __forceinline__ bool emit_fast(const float* x, const Row& p, int64_t cidx, void* dq, void* codes) const {
    if (!hw) return false;
    const int cd = code_dtype;
    float t[N];
    bool near = !p.fast, far = false;
    if constexpr (BF) {
      // distance of the low 16 bits from the midpoint window, two products per packed 16-bit instruction
      lcq_u16x2 nearest = {0xffff, 0xffff};
      #pragma unroll
      for (int i = 0; i < N; i += 2) {
        t[i] = x[i] * p.r;
        t[i + 1] = x[i + 1] * p.r;
        const uint32_t lows = __builtin_amdgcn_perm(f2u(t[i + 1]), f2u(t[i]), 0x05040100u);
        nearest = __builtin_elementwise_min(nearest, __builtin_bit_cast(lcq_u16x2, lows) - lcq_u16x2{0x7ff8, 0x7ff8});
      }
      near = near || nearest.x <= 0x10 || nearest.y <= 0x10;
    } else {
      #pragma unroll
      for (int i = 0; i < N; ++i) {
        t[i] = x[i] * p.r;
        const uint32_t lowm = f2u(t[i]) & ((1u << drop) - 1u);
        far = far || ((lowm - (half - 8u)) <= 16u) || !(fabsf(t[i]) >= 1.0001f * min_normal);
      }
    }
    if (!p.inrange) {                                        // static scales: any magnitude may turn up
      float m = 0.0f;
      #pragma unroll
      for (int i = 0; i < N; i += 2) m = nan_max(nan_max(m, fabsf(t[i])), fabsf(t[i + 1]));
      far = far || !(m < hw_lim);
    }
    if (__builtin_expect(far, 0)) return false;              // left to the emulated grid (rare: ties of fp32 rows, inf, NaN)
    if constexpr (BF) {
      if (__builtin_expect(near, 0)) {                       // the product may round unlike the quotient: divide
        #pragma unroll
        for (int i = 0; i < N; ++i) t[i] = x[i] / p.s;
        #pragma unroll
        for (int i = 0; i < N; ++i) far = far || !(fabsf(t[i]) < hw_lim);
        if (far) return false;
      }
    } else {
      if (!p.fast) return false;
    }
    #pragma unroll
    for (int i = 0; i < N; i += 2) rnd_pair<BF>(t[i], t[i + 1]);
    const float nudge = (BF && !tie_even) ? 1.0009765625f : 1.0f;
    #pragma unroll
    for (int i = 0; i < N; ++i) t[i] = __builtin_fmaf(t[i], nudge, 0.0f);
    uint32_t w[N / 4];
    #pragma unroll
    for (int k = 0; k < N / 4; ++k) {
      int u = 0;
      if (hw == 1) {
        u = __builtin_amdgcn_cvt_pk_fp8_f32(t[4 * k], t[4 * k + 1], u, false);
        u = __builtin_amdgcn_cvt_pk_fp8_f32(t[4 * k + 2], t[4 * k + 3], u, true);
      } else {
        u = __builtin_amdgcn_cvt_pk_bf8_f32(t[4 * k], t[4 * k + 1], u, false);
        u = __builtin_amdgcn_cvt_pk_bf8_f32(t[4 * k + 2], t[4 * k + 3], u, true);
      }
      w[k] = (uint32_t)u;
    }
    if (codes && cd == LCQ_CODE_FP8) {
      if constexpr (N == 8) *(u32x2*)((uint8_t*)codes + cidx * N) = u32x2{w[0], w[1]};
      else *(uint32_t*)((uint8_t*)codes + cidx * N) = w[0];
    }
    if (dq || (codes && cd == LCQ_CODE_F32)) {
      float q[N];
      #pragma unroll
      for (int k = 0; k < N / 4; ++k) {
        f32x2 lo, hi;
        if (hw == 1) { lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k], false); hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k], true); }
        else { lo = __builtin_amdgcn_cvt_pk_f32_bf8((int)w[k], false); hi = __builtin_amdgcn_cvt_pk_f32_bf8((int)w[k], true); }
        q[4 * k] = lo[0]; q[4 * k + 1] = lo[1]; q[4 * k + 2] = hi[0]; q[4 * k + 3] = hi[1];
      }
      if (codes && cd == LCQ_CODE_F32) {
        #pragma unroll
        for (int i = 0; i < N; i += 4) *(f32x4*)((float*)codes + cidx * N + i) = f32x4{q[i], q[i + 1], q[i + 2], q[i + 3]};
      }
      if (dq) {
        #pragma unroll
        for (int i = 0; i < N; ++i) q[i] = deq_raw(q[i], p);
        if (dq_f32) {
          #pragma unroll
          for (int i = 0; i < N; i += 4)
            __builtin_nontemporal_store(u32x4{f2u(q[i]), f2u(q[i + 1]), f2u(q[i + 2]), f2u(q[i + 3])},
                                        (u32x4*)dq + (cidx * N + i) / 4);
        } else {
          __builtin_nontemporal_store(pack_rne<BF>(q), (u32x4*)dq + cidx);
        }
      }
    }
    return true;
  }

  // (q - 0.0) * s in fp32, then the cast of fake_quant_* (quant.py:1107,1153)
  __device__ __forceinline__ float deq_raw(float q, const Row& p) const { return (q - 0.0f) * p.sm; }
  __device__ __forceinline__ float deq(float q, const Row& p) const {
    const float d = deq_raw(q, p);
    return dq_f32 ? d : rnd_e<BF>(d);
  }

  __device__ __forceinline__ uint32_t pack4(const float* q) const {
    uint32_t w = 0;
    #pragma unroll
    for (int j = 0; j < 4; ++j) w |= byte(q[j]) << (8 * j);
    return w;
  }

  // float8 storage of an on-grid value
  __device__ __forceinline__ uint32_t byte(float q) const {
    const uint32_t bits = f2u(q);
    const uint32_t sign = (bits >> 24) & 0x80u;
    const uint32_t mag = bits & 0x7fffffffu;
    if (e_bits == 4) {                                     // float8_e4m3fn: bias 7, no inf, 0x7f = nan
      if (mag > 0x43e00000u) return sign | 0x7fu;          // > 448 (or nan/inf)
      const int ex = (int)(mag >> 23) - 127;
      if (ex < -6) return sign | (uint32_t)(u2f(mag) * 512.0f);   // multiples of 2^-9
      return sign | ((uint32_t)(ex + 7) << 3) | ((mag >> 20) & 7u);
    }
    // float8_e5m2: the top byte of the fp16 encoding
    if (mag > 0x7f800000u) return sign | 0x7fu;
    if (mag > 0x47600000u) return sign | 0x7cu;            // > 57344 -> inf
    const int ex = (int)(mag >> 23) - 127;
    if (ex < -14) return sign | (uint32_t)(u2f(mag) * 65536.0f);  // multiples of 2^-16
    return sign | ((uint32_t)(ex + 15) << 2) | ((mag >> 21) & 3u);
  }
};

template <int BF>
FpOp<BF> make_op(int e_bits, int m_bits, float qmax, int flags, int code_dtype) {
  FpOp<BF> c;
  c.qmax = qmax; c.rqmax = (float)(1.0 / (double)qmax); c.e_bits = e_bits; c.m_bits = m_bits;
  c.tie_even = (flags & LCQ_FLAG_TIE_EVEN) != 0;
  c.subnormals = (flags & LCQ_FLAG_NO_SUBNORMALS) == 0;
  c.is_static = (flags & LCQ_FLAG_STATIC) != 0;
  c.scalar_qp = (flags & LCQ_FLAG_SCALAR_QP) != 0;
  c.dq_f32 = (flags & LCQ_FLAG_DQ_F32) != 0;
  c.scale_f32 = (flags & LCQ_FLAG_SCALE_F32) != 0;
  c.code_dtype = code_dtype;
  c.drop = 23 - m_bits;
  c.half = 1u << (c.drop - 1);
  c.keep = ~((1u << c.drop) - 1u);
  c.min_exp = -((1 << (e_bits - 1)) - 2);
  c.max_exp = 1 << (e_bits - 1);
  c.max_mag = ((uint32_t)(c.max_exp + 127) << 23) | (((1u << m_bits) - 1u) << c.drop);
  c.min_normal = __builtin_ldexpf(1.0f, c.min_exp);
  c.hw = 0; c.hw_lim = 0.0f;
  // 448 / 57344 are the float8 maxima; the emulated grid goes on (480 / 65536 come next), reached from the midpoints
  // 464 / 61440 upwards.  The test is made on the quotient before a bf16 row rounds it (steps of 2 / 256 up there), so the limit
  // of bf16 rows lies half a step lower: anything below it rounds to the bf16 number under the midpoint at most.
  if (c.subnormals && e_bits == 4 && m_bits == 3) { c.hw = 1; c.hw_lim = BF ? 463.0f : 464.0f; }
  if (c.subnormals && e_bits == 5 && m_bits == 2) { c.hw = 2; c.hw_lim = BF ? 61312.0f : 61440.0f; }
  return c;
}

// FloatQuantizer.dequant on stored fp32 codes: out = (q - 0) * s in fp32
template <int BF>
__global__ __launch_bounds__(256) void dequant_fp_kernel(const float* __restrict__ q, int64_t rows, int64_t cols,
                                                         const void* __restrict__ scales, float* __restrict__ out,
                                                         int scalar_qp) {
  const int64_t n = rows * cols;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (int64_t)gridDim.x * 256) {
    const float s = load_scalar<BF>(scales, scalar_qp ? 0 : e / cols);
    out[e] = (q[e] - 0.0f) * s;
  }
}


// ---- FloatQuantizer without qtorch: per-element power-of-two-ish steps -------------------------
// get_float_qparams + quant + dequant, quant.py:1004-1026, 1042-1080, as one pass.  Per row
//   maxval = max(max, -min);  bias = 2^e - log2(maxval) + log2(2 - 2^-m) - 1
// and per element
//   xc = min(max(x, -maxval), maxval)
//   ls = clamp(floor(log2|xc| + bias), min=1);  s = 2^(ls - m - bias);  s == 0 -> 1
//   q = round(xc / s + 0);  dq = (q - 0) * s
// with a rounding to the row dtype after every operation (bf16 rows), as torch evaluates it.
// log2 and 2^x as torch's GPU kernels compute them: the device math library's log2f, and pow(2, x) for `2.0 ** x`
// (not exp2f, which differs from it in the last place).  With these the fp32 rows agree with torch on the GPU bit for
// bit; torch's CPU kernels use another library and differ from both in the last place of the bias of about a quarter
// of the rows.  bf16 rows round every intermediate to 8 bits and agree with both.
#define LCQ_EMU_LOG2(x) log2f(x)
#define LCQ_EMU_EXP2(x) powf(2.0f, x)
struct EmuArgs {
  const void* x; const void* mn; const void* mx; const void* s_in;
  void* xc; void* s_out; void* q; void* dq;
  int64_t rows, cols;
  float two_e, m_bits;
  int is_static, scalar_qp, row_qp, q_fp8, e_bits;
};

template <int BF>
__global__ __launch_bounds__(256) void fp_emu_kernel(EmuArgs a) {
  constexpr int N = Vec<BF>::N;
  const int64_t cpr = a.cols / N;                          // chunks per row (host guarantees cols % N == 0)
  const int64_t nchunks = a.rows * cpr;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < nchunks; c += (int64_t)gridDim.x * 256) {
    const int64_t row = c / cpr, e0 = c * N;
    float v[N], xc[N], sc[N], q[N], dq[N];
    unpack<BF>(((const u32x4*)a.x)[c], v);
    float maxval = 0.0f, bias = 0.0f;
    if (!a.is_static) {
      const float mn = load_scalar<BF>(a.mn, row), mx = load_scalar<BF>(a.mx, row);
      maxval = nan_max(mx, -mn);
      // log2(2 - 2^-m) is a 0-dim fp32 tensor in the reference: where it is added to the 16-bit rows torch rounds it
      // to their type first (on both platforms: a sum)
      bias = rnd<BF>(a.two_e - rnd<BF>(LCQ_EMU_LOG2(maxval)));
      bias = rnd<BF>(bias + rnd<BF>(LCQ_EMU_LOG2(2.0f - LCQ_EMU_EXP2(-a.m_bits))));
      bias = rnd<BF>(bias - 1.0f);
    }
    #pragma unroll
    for (int i = 0; i < N; ++i) {
      float s;
      if (a.is_static) {
        xc[i] = v[i];
        s = load_scalar<BF>(a.s_in, a.scalar_qp ? 0 : (a.row_qp ? row : e0 + i));
      } else {
        xc[i] = nan_min(nan_max(v[i], -maxval), maxval);
        float l = rnd<BF>(LCQ_EMU_LOG2(fabsf(xc[i])));
        l = rnd<BF>(l + bias);
        l = __builtin_floorf(l);
        l = clamp_min_nan(l, 1.0f);
        float ex = rnd<BF>(l - a.m_bits);
        ex = rnd<BF>(ex - bias);
        s = rnd<BF>(LCQ_EMU_EXP2(ex));
      }
      if (s == 0.0f) s = 1.0f;                             // scales[scales == 0] = 1, quant.py:1061
      sc[i] = s;
      float t = rnd<BF>(xc[i] / s);
      t = t + 0.0f;
      q[i] = __builtin_rintf(t);
      dq[i] = rnd<BF>((q[i] - 0.0f) * s);
    }
    if (a.xc) ((u32x4*)a.xc)[c] = pack<BF>(xc);
    if (a.s_out) ((u32x4*)a.s_out)[c] = pack<BF>(sc);
    if (a.dq) ((u32x4*)a.dq)[c] = pack<BF>(dq);
    if (a.q) {
      if (a.q_fp8) {
        // |q| <= 2^(m+1) - 1 is an integer, exact in float8; written with the e4m3fn / e5m2 encoder
        FpOp<BF> enc; enc.e_bits = a.e_bits;
        #pragma unroll
        for (int i = 0; i < N; ++i) ((uint8_t*)a.q)[e0 + i] = (uint8_t)enc.byte(q[i]);
      } else ((u32x4*)a.q)[c] = pack<BF>(q);
    }
  }
}

}  // namespace

extern "C" {

int lcq_quant_fp(const void* x, int dtype, int64_t rows, int64_t cols, int e_bits, int m_bits, float qmax, int flags,
                 void* dq, void* codes, int code_dtype, void* scales, void* stream) {
  if (!x || rows < 0 || cols <= 0 || !scales) return LCQ_EINVAL;
  if (rows == 0) return LCQ_OK;
  if (e_bits < 2 || e_bits > 5 || m_bits < 1 || m_bits > 10 || !(qmax > 0.0f)) return LCQ_EINVAL;
  if (codes) {
    if (code_dtype == LCQ_CODE_FP8) {
      if (!((e_bits == 4 && m_bits == 3) || (e_bits == 5 && m_bits == 2))) return LCQ_EDTYPE;
    } else if (code_dtype != LCQ_CODE_F32) return LCQ_EDTYPE;
  } else code_dtype = LCQ_CODE_NONE;
  if ((flags & LCQ_FLAG_SCALAR_QP) && !(flags & LCQ_FLAG_STATIC)) return LCQ_EINVAL;
  if ((flags & LCQ_FLAG_SCALE_F32) && !(flags & LCQ_FLAG_STATIC)) return LCQ_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (dtype == LCQ_F32)
    rc = dispatch_rows(x, rows, cols, dq, codes, scales, (void*)nullptr, make_op<false>(e_bits, m_bits, qmax, flags, code_dtype), false, st);
  else if (dtype == LCQ_BF16)
    rc = dispatch_rows(x, rows, cols, dq, codes, scales, (void*)nullptr, make_op<true>(e_bits, m_bits, qmax, flags, code_dtype), false, st);
  else if (dtype == LCQ_F16)                               // fp16 rows: the element-wise kernel (correct to the bit, not tuned)
    rc = dispatch_rows(x, rows, cols, dq, codes, scales, (void*)nullptr, make_op<ROW_F16>(e_bits, m_bits, qmax, flags, code_dtype), true, st);
  else return LCQ_EDTYPE;
  if (rc != LCQ_OK) return rc;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_dequant_fp(const float* q, int64_t rows, int64_t cols, const void* scales, int scale_dtype, int flags,
                   float* out, void* stream) {
  if (!q || !scales || !out || rows < 0 || cols <= 0) return LCQ_EINVAL;
  if (rows == 0) return LCQ_OK;
  const int scalar_qp = (flags & LCQ_FLAG_SCALAR_QP) != 0;
  int64_t grid = (rows * cols + 255) / 256;
  if (grid > 65536) grid = 65536;
  hipStream_t st = (hipStream_t)stream;
  if (scale_dtype == LCQ_F32) dequant_fp_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>(q, rows, cols, scales, out, scalar_qp);
  else if (scale_dtype == LCQ_BF16) dequant_fp_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>(q, rows, cols, scales, out, scalar_qp);
  else if (scale_dtype == LCQ_F16) dequant_fp_kernel<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(q, rows, cols, scales, out, scalar_qp);
  else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_quant_fp_emu(const void* x, int dtype, int64_t rows, int64_t cols, int e_bits, int m_bits, int flags,
                     const void* min_in, const void* max_in, const void* scales_in, void* xc, void* scales_out,
                     void* q, int code_dtype, void* dq, void* stream) {
  if (!x || rows < 0 || cols <= 0) return LCQ_EINVAL;
  if (rows == 0) return LCQ_OK;
  if (e_bits < 2 || e_bits > 5 || m_bits < 1 || m_bits > 10) return LCQ_EINVAL;
  const int is_static = (flags & LCQ_FLAG_STATIC) != 0;
  if (is_static ? !scales_in : (!min_in || !max_in)) return LCQ_EINVAL;
  if ((flags & (LCQ_FLAG_SCALAR_QP | LCQ_FLAG_ROW_QP)) && !is_static) return LCQ_EINVAL;
  if (dtype != LCQ_F32 && dtype != LCQ_BF16 && dtype != LCQ_F16) return LCQ_EDTYPE;
  const int n = (dtype == LCQ_F32) ? 4 : 8;
  if (cols % n != 0) return LCQ_EINVAL;
  int q_fp8 = 0;
  if (q) {
    if (code_dtype == LCQ_CODE_FP8) {
      if (!((e_bits == 4 && m_bits == 3) || (e_bits == 5 && m_bits == 2))) return LCQ_EDTYPE;
      q_fp8 = 1;
    } else if (code_dtype != LCQ_CODE_SAME) return LCQ_EDTYPE;
  }
  const void* al[] = {x, xc, scales_out, dq, (q && !q_fp8) ? q : nullptr, (is_static && !(flags & (LCQ_FLAG_SCALAR_QP | LCQ_FLAG_ROW_QP))) ? scales_in : nullptr};
  for (const void* p : al) if (p && ((uintptr_t)p % 16) != 0) return LCQ_EALIGN;
  EmuArgs a;
  a.x = x; a.mn = min_in; a.mx = max_in; a.s_in = scales_in; a.xc = xc; a.s_out = scales_out; a.q = q; a.dq = dq;
  a.rows = rows; a.cols = cols;
  a.two_e = (float)(1 << e_bits);
  a.m_bits = (float)m_bits;
  a.is_static = is_static; a.scalar_qp = (flags & LCQ_FLAG_SCALAR_QP) != 0; a.row_qp = (flags & LCQ_FLAG_ROW_QP) != 0;
  a.q_fp8 = q_fp8; a.e_bits = e_bits;
  int64_t grid = (rows * (cols / n) + 255) / 256;
  if (grid > 262144) grid = 262144;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LCQ_BF16) fp_emu_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>(a);
  else if (dtype == LCQ_F16) fp_emu_kernel<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(a);
  else fp_emu_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>(a);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
