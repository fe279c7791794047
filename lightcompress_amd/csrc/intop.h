// Integer quantizer arithmetic shared by the row kernels (quant_int.hip) and the AWQ clip search
// (awq_clip.hip): per-row parameters (get_qparams, quant.py:544-558) and per-element quantize /
// dequantize (quant.py:698-716) with the exactness rules described in quant_int.hip.
#pragma once
#include "rowquant.h"

namespace lcq {

struct IntRow {
  float s, z, r, sdq;
  float lo, hi;      // qmin - z, qmax - z: clamp bounds of the code minus the zero point
  int fast;          // x * (1/s) + guard may replace x / s
  int zint;          // zero point is a small integer: rint(t) + z and q - z are exact
  // nibble packing (zint rows): bit patterns of 1.5 * 2^23 + (qmin - z) and + (qmax - z), and the sum over the
  // eight nibble positions of the pattern that stands for code -8
  int clo, chi;
  uint32_t nib0;
};

// 1.5 * 2^23: x + RINT_BIAS rounds x to the nearest integer, ties to even (the constant is even), and leaves
// that integer in the low mantissa bits, for |x| < 2^22
constexpr float RINT_BIAS = 12582912.0f;
constexpr int RINT_BIAS_BITS = 0x4B400000;

// FAST: round_zp and |qmin|,qmax <= 256 (every stock configuration).
template <int BF_, bool FAST, bool PRESCALE = false, int CD_ = -1>
struct IntOp {
  static constexpr int BF = BF_;          // row type: 0 fp32, 1 bf16, 2 fp16 (element-wise forms only: FAST is false)
  static constexpr bool HAS_PRESCALE = PRESCALE;
  static constexpr bool HAS_FUSED_DQ = FAST;
  static constexpr bool HAS_CUSTOM_EMIT = false;
  static constexpr bool ABS_ONLY = false;
  static constexpr int CD = CD_;
  using Row = IntRow;
  float qmin, qmax, qrange, osf;
  float rqmax, rqrange;         // 1 / qmax, 1 / qrange (fp32-rounded)
  int sym, round_zp, is_static, scalar_qp, dq_f32, code_dtype, range_bf16, range_f16, scale_f32;
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
    // caller-given zero points need not be integers; a row whose scale is infinite or NaN (an infinite or NaN weight)
    // takes the element-wise form too, which hands NaN codes on like torch.clamp does
    p.zint = (z == rintf(z)) && (fabsf(z) <= 512.0f) && (a < __builtin_inff());
    p.sdq = rnd<BF>(s * osf);
    p.lo = qmin - z; p.hi = qmax - z;                       // exact: small integers
    p.clo = RINT_BIAS_BITS + (int)p.lo; p.chi = RINT_BIAS_BITS + (int)p.hi;
    p.nib0 = (uint32_t)(RINT_BIAS_BITS - ((int)z + 8)) * 0x11111111u;
    return p;
  }

  // a / c for a per-launch constant c (rc = 1/c rounded to fp32), rounded to the row type.  bf16 rows:
  // the product a * rc stands for the quotient unless it lies within 8 ulp of a bf16 rounding
  // midpoint; fp32 rows need the correctly rounded quotient itself.
  __device__ __forceinline__ float div_const(float a, float c, float rc) const {
    if constexpr (BF == ROW_BF16) {
      float q = a * rc;
      if (__builtin_expect(((f2u(q) & 0xffffu) - 0x7ff8u) <= 0x10u, 0)) q = a / c;
      return rnd<BF>(q);
    } else {
      return rnd<BF>(a / c);                                 // fp32: the quotient itself; fp16: the quotient, rounded
    }
  }

  // get_qparams, quant.py:544-558
  __device__ __forceinline__ Row make(float mn, float mx) const {
    // clamp(min=1e-5) in the range dtype: 1e-5 rounds to the same number in bf16 (1.3125 * 2^-17) and fp16 (168 * 2^-24)
    const float cmin = (BF || range_bf16 || range_f16) ? 1.0013580322265625e-05f : 1e-5f;
    float s, z;
    if (sym) {
      float a = nan_max(fabsf(mx), fabsf(mn));
      a = clamp_min_nan(a, cmin);
      s = div_const(a, qmax, rqmax);
      z = 0.0f;
    } else {
      float d = rnd<BF>(mx - mn);
      if (range_bf16) d = bf16_round(d);
      if (range_f16) d = f16_round(d);
      d = clamp_min_nan(d, cmin);
      s = div_const(d, qrange, rqrange);
      // mn / s through the reciprocal, with the same exactness guards as the per-element quotients
      float t = mn * __builtin_amdgcn_rcpf(s);
      const float as = fabsf(s);
      bool ok = (as > 8.6736174e-19f) && (as < 1.1529215e18f);
      if constexpr (BF == ROW_F16) {
        ok = false;                                          // fp16 rows: always the division
      } else if constexpr (BF == ROW_BF16) {
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
    if (scale_f32) {
      // 0-dim fp32 parameters next to a 16-bit tensor: torch on a GPU converts a 0-dim tensor operand to the type of
      // the result before every operation, so the quotient, the sums and the product see the parameters rounded to
      // the row type, and scales * output_scale_factor (0-dim fp32 times a number) is rounded where it meets the rows
      const float s32 = ((const float*)scales)[i];
      Row p = finish(rnd<BF>(s32), zeros ? rnd<BF>(((const float*)zeros)[i]) : 0.0f);
      p.sdq = rnd<BF>(s32 * osf);
      return p;
    }
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
      const float lo = BF == ROW_F16 ? 0.0f : (BF ? 1.00044417e-09f : 1e-9f);   // scales.clamp_min(1e-9): the bound in the row type (0 in fp16)
      const float t = rnd<BF>(x / clamp_min_nan(p.s, lo));
      q = rintf(rnd<BF>(t + p.z));
    }
    if (q != q) return q;                                    // torch.clamp hands a NaN on (inf / inf of an infinite weight)
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
      ok = ok && nearest.x > 0x10 && nearest.y > 0x10;
    } else {
      #pragma unroll
      for (int i = 0; i < N; ++i) {
        t[i] = x[i] * p.r;
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

  // Eight 4-bit codes of one bf16 chunk as a compressed-tensors word (code + 8 in nibble i), FAST rows with an
  // integer zero point.  t + RINT_BIAS holds rint(t) in its low mantissa bits; clamped as an integer pattern (any
  // NaN or infinity lands on a bound), shifted to its nibble and added up, the eight patterns differ from the
  // eight nibbles by a per-row constant (arithmetic modulo 2^32 is linear, so the high bits cancel too).
  __device__ __forceinline__ uint32_t ct4_word(const float* x, const Row& p) const {
    float t[8];
    quotients<8>(x, t, p);
    uint32_t acc = 0;
    #pragma unroll
    for (int i = 0; i < 8; ++i) {
      int b = (int)f2u(t[i] + RINT_BIAS), c;
      asm("v_med3_i32 %0, %1, %2, %3" : "=v"(c) : "v"(b), "v"(p.clo), "v"(p.chi));
      acc = ((uint32_t)c << (4 * i)) + acc;
    }
    return acc - p.nib0;
  }

  // fake quant without the codes (FAST only): (clamp(rint(t) + z, qmin, qmax) - z) * s equals
  // clamp(rint(t), qmin - z, qmax - z) * s when z is a small integer (all terms exact); the "+ 0" of the
  // fused multiply-add (one rounding, that of the product) turns the -0 that rint(-0.3) leaves into the +0
  // that (q - z) gives.  The products are left unrounded: the caller rounds to the row type while packing.
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
    for (int i = 0; i < N; ++i) d[i] = __builtin_fmaf(__builtin_amdgcn_fmed3f(rintf(t[i]), p.lo, p.hi), p.sdq, 0.0f);
  }

  // dequant, quant.py:709-711 (scale already multiplied by output_scale_factor)
  __device__ __forceinline__ float deq_raw(float q, const Row& p) const {   // before the rounding to the row type
    float d = q - p.z;                                       // exact for small integer codes
    if constexpr (BF != 0) { if (!FAST || !p.zint) d = rnd<BF>(d); }
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
  c.range_f16 = (flags & LCQ_FLAG_RANGE_F16) != 0;
  c.scale_f32 = (flags & LCQ_FLAG_SCALE_F32) != 0;
  c.colscale = nullptr; c.wrow_cols = 1;
  c.code_dtype = code_dtype;
  return c;
}

}  // namespace lcq
