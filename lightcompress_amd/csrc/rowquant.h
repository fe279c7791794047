// Row-wise fused quantizer skeleton for gfx950, shared by the integer and the
// minifloat quantizers.  One pass over HBM: load a row (16-byte chunks per
// lane), reduce min/max across the lanes that share the row (DPP /
// ds_swizzle butterflies), derive the row's parameters, emit codes and/or
// dequantized values.
//
// An Op policy supplies the arithmetic:
//   static constexpr int BF             row type: 0 fp32, 1 bf16, 2 fp16 (a bool reads as 0 / 1)
//   struct Row                          per-row parameters
//   Row  make(mn, mx)                   dynamic parameters from the row range
//   Row  load(scales, zeros, row)       static parameters
//   void store_qp(scales, zeros, row, Row)
//   float code(x, Row)                  quantized value as a float
//   void codes<N>(x[N], q[N], Row)      the same for one 16-byte chunk (lets the op share work)
//   float deq(q, Row)                   dequantized value (already rounded to the output type)
//   uint32_t byte(q)                    1-byte storage of a code (U8 / I8 / FP8)
//   uint32_t pack4(q[4])                four of them in one word
//   bool is_static, dq_f32; int code_dtype
//   static constexpr int CD             code storage fixed at compile time, or -1 (use code_dtype)
//   static constexpr bool ABS_ONLY      make() uses max |x| only: min is not reduced (mn == mx == max |x| then)
//   static constexpr bool HAS_PRESCALE; if set, prescale(chunk,row,ch,nchunks) / prescale1(x,row,col,cols)
//   multiply the input by a per-column factor (rounded to the row type) before anything else
#pragma once
#include "common.h"
#include "lcq_internal.h"

namespace lcq {

// BF: the row type.  0 = fp32, 1 = bf16, 2 = fp16 (a bool argument reads as 0 / 1).  The fast kernels exist for fp32
// and bf16; fp16 rows go through the element-wise kernel (row_scalar_kernel) and the element-wise forms of the ops.
constexpr int ROW_F32 = 0, ROW_BF16 = 1, ROW_F16 = 2;
template <int BF> struct Vec { static constexpr int N = BF ? 8 : 4; };
typedef unsigned short lcq_u16x2 __attribute__((ext_vector_type(2)));

template <int BF> __device__ __forceinline__ float rnd(float v) {
  if constexpr (BF == ROW_F16) {
    // torch rounds twice: the fp32 result of the operation, then the conversion to fp16.  The empty asm keeps the
    // compiler from folding an fp32 multiply into a mixed-precision instruction that rounds the exact product once
    // (v_fma_mixlo_f16): the two differ when the fp32 rounding lands on an fp16 tie (x * 1.7 does, often).
    asm("" : "+v"(v));
    return (float)(_Float16)v;
  }
  else if constexpr (BF) return (float)(__bf16)v;
  else return v;
}
// per-element rounding: hardware RNE convert (v_cvt_pk_bf16_f32 / v_cvt_f16_f32)
template <int BF> __device__ __forceinline__ float rnd_e(float v) { return rnd<BF>(v); }
__device__ __forceinline__ float clamp_min_nan(float v, float lo) { return nan_max(v, lo); }

// two fp32 values -> one dword of two bf16 (RNE), a single v_cvt_pk_bf16_f32
typedef float lcq_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 lcq_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 lcq_f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf16_pack_rne(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(lcq_f32x2{a, b}, lcq_bf16x2));
}
__device__ __forceinline__ uint32_t f16_pack_rne(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(lcq_f32x2{a, b}, lcq_f16x2));
}
__device__ __forceinline__ float f16_lo(uint32_t w) { return (float)__builtin_bit_cast(lcq_f16x2, w).x; }
__device__ __forceinline__ float f16_hi(uint32_t w) { return (float)__builtin_bit_cast(lcq_f16x2, w).y; }
// round a pair to the row type in place (bf16: one convert + two unpack ops for two elements)
template <int BF> __device__ __forceinline__ void rnd_pair(float& a, float& b) {
  if constexpr (BF == ROW_F16) {
    a = rnd<BF>(a); b = rnd<BF>(b);
  } else if constexpr (BF) {
    const uint32_t u = bf16_pack_rne(a, b);
    a = u2f(u << 16);
    b = u2f(u & 0xffff0000u);
  }
}

template <int BF>
__device__ __forceinline__ void unpack(const u32x4& raw, float* v) {
  if constexpr (BF == ROW_F16) {
    #pragma unroll
    for (int i = 0; i < 4; ++i) { v[2 * i] = f16_lo(raw[i]); v[2 * i + 1] = f16_hi(raw[i]); }
  } else if constexpr (BF) {
    #pragma unroll
    for (int i = 0; i < 4; ++i) { v[2 * i] = bf16_lo(raw[i]); v[2 * i + 1] = bf16_hi(raw[i]); }
  } else {
    #pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = u2f(raw[i]);
  }
}
// values already exact in the row type -> one 16-byte chunk
template <int BF>
__device__ __forceinline__ u32x4 pack(const float* v) {
  u32x4 raw;
  if constexpr (BF == ROW_F16) {
    #pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = f16_pack_rne(v[2 * i], v[2 * i + 1]);
  } else if constexpr (BF) {
    #pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = bf16_pack(v[2 * i], v[2 * i + 1]);
  } else {
    #pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = f2u(v[i]);
  }
  return raw;
}

template <int BF>
__device__ __forceinline__ float load_scalar(const void* p, int64_t i) {
  if constexpr (BF == ROW_F16) return (float)((const _Float16*)p)[i];
  else if constexpr (BF) return u2f((uint32_t)((const uint16_t*)p)[i] << 16);
  else return ((const float*)p)[i];
}
// v is exact in the row type
template <int BF>
__device__ __forceinline__ void store_scalar(void* p, int64_t i, float v) {
  if constexpr (BF == ROW_F16) ((_Float16*)p)[i] = (_Float16)v;
  else if constexpr (BF) ((uint16_t*)p)[i] = (uint16_t)(f2u(v) >> 16);
  else ((float*)p)[i] = v;
}

// values NOT yet rounded to the row type -> one 16-byte chunk, rounding (RNE) while packing
template <int BF>
__device__ __forceinline__ u32x4 pack_rne(const float* v) {
  u32x4 raw;
  if constexpr (BF == ROW_F16) {
    #pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = f16_pack_rne(v[2 * i], v[2 * i + 1]);
  } else if constexpr (BF) {
    #pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = bf16_pack_rne(v[2 * i], v[2 * i + 1]);
  } else {
    #pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = f2u(v[i]);
  }
  return raw;
}

// N codes of one 16-byte input chunk -> storage
template <class Op>
__device__ __forceinline__ void store_codes(const Op& op, void* codes, int64_t elem0, const float* q) {
  constexpr int BF = Op::BF;
  constexpr int N = Vec<BF>::N;
  const int cd = (Op::CD >= 0) ? Op::CD : op.code_dtype;       // compile-time when the op pins it
  if (cd == LCQ_CODE_I32) {
    int32_t* p = (int32_t*)codes + elem0;
    #pragma unroll
    for (int i = 0; i < N; i += 4) {
      u32x4 w;
      #pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = (uint32_t)(int32_t)q[i + j];
      *(u32x4*)(p + i) = w;
    }
  } else if (cd == LCQ_CODE_F32) {
    float* p = (float*)codes + elem0;
    #pragma unroll
    for (int i = 0; i < N; i += 4) {
      u32x4 w;
      #pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = f2u(q[i + j]);
      *(u32x4*)(p + i) = w;
    }
  } else if (cd == LCQ_CODE_U8 || cd == LCQ_CODE_I8 || cd == LCQ_CODE_FP8) {
    uint8_t* p = (uint8_t*)codes + elem0;
    #pragma unroll
    for (int i = 0; i < N; i += 4) {
      *(uint32_t*)(p + i) = op.pack4(q + i);
    }
  } else if (cd == LCQ_CODE_SAME) {
    *((u32x4*)codes + elem0 / N) = pack<BF>(q);
  } else if (cd == LCQ_CODE_CT4) {
    // compressed-tensors nibbles: 8 codes per int32 word, a 4-element chunk fills half a word
    uint32_t w = 0;
    #pragma unroll
    for (int i = 0; i < N; ++i) w |= (((uint32_t)(int32_t)q[i] + 8u) & 0xfu) << (4 * i);
    if constexpr (N == 8) ((uint32_t*)codes)[elem0 / 8] = w;
    else ((uint16_t*)codes)[elem0 / 4] = (uint16_t)w;
  }
}
template <class Op>
__device__ __forceinline__ void store_code1(const Op& op, void* codes, int64_t e, float q) {
  const int cd = op.code_dtype;
  if (cd == LCQ_CODE_I32) ((int32_t*)codes)[e] = (int32_t)q;
  else if (cd == LCQ_CODE_F32) ((float*)codes)[e] = q;
  else if (cd == LCQ_CODE_U8 || cd == LCQ_CODE_I8 || cd == LCQ_CODE_FP8) ((uint8_t*)codes)[e] = (uint8_t)op.byte(q);
  else if (cd == LCQ_CODE_SAME) store_scalar<Op::BF>(codes, e, q);
}

// codes + dq of one chunk, generic form: op.codes -> storage, op.deq_raw -> storage
template <class Op>
__device__ __forceinline__ void emit_chunk_generic(const Op& op, const typename Op::Row& p, const float* v_in, int64_t cidx,
                                                   void* dq, void* codes) {
  constexpr int BF = Op::BF;
  constexpr int N = Vec<BF>::N;
  float v[N], q[N];
  #pragma unroll
  for (int i = 0; i < N; ++i) v[i] = v_in[i];
  if constexpr (Op::CD == LCQ_CODE_CT4 && N == 8 && Op::HAS_FUSED_DQ) {
    if (codes && !dq && p.zint && p.fast) {                  // nibbles straight from the quotients
      ((uint32_t*)codes)[cidx] = op.ct4_word(v, p);
      return;
    }
  }
  op.template codes<N>(v, q, p);
  if (codes) store_codes(op, codes, cidx * N, q);
  if (dq) {
    #pragma unroll
    for (int i = 0; i < N; ++i) v[i] = op.deq_raw(q[i], p);   // rounded to the row type by the packing below
    if (op.dq_f32) {
      #pragma unroll
      for (int i = 0; i < N; i += 4) {
        u32x4 w;
        #pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = f2u(v[i + j]);
        __builtin_nontemporal_store(w, (u32x4*)dq + (cidx * N + i) / 4);
      }
    } else {
      __builtin_nontemporal_store(pack_rne<BF>(v), (u32x4*)dq + cidx);
    }
  }
}
// Returns false when the op's fast path declined the chunk (HAS_CUSTOM_EMIT only): the caller
// then runs emit_chunk_slow on it, from ONE rolled loop, so the long generic code exists once per
// kernel instead of once per unrolled chunk (and stays out of the instruction cache).
template <class Op>
__device__ __forceinline__ bool emit_chunk(const Op& op, const typename Op::Row& p, const u32x4& r, int64_t cidx,
                                           void* dq, void* codes) {
  constexpr int BF = Op::BF;
  constexpr int N = Vec<BF>::N;
  float v[N], q[N];
  unpack<BF>(r, v);
  if constexpr (Op::HAS_CUSTOM_EMIT) {
    return op.template emit_fast<N>(v, p, cidx, dq, codes);
  } else {
    if constexpr (Op::HAS_FUSED_DQ) {
      if (!codes) {                                          // fake quant: no detour through the codes
        if (dq) {
          op.template fused_dq<N>(v, q, p);
          __builtin_nontemporal_store(pack_rne<BF>(q), (u32x4*)dq + cidx);
        }
        return true;
      }
    }
    emit_chunk_generic(op, p, v, cidx, dq, codes);
    return true;
  }
}
template <class Op>
__device__ __forceinline__ void emit_chunk_slow(const Op& op, const typename Op::Row& p, const u32x4& r, int64_t cidx,
                                                void* dq, void* codes) {
  float v[Vec<Op::BF>::N];
  unpack<Op::BF>(r, v);
  emit_chunk_generic(op, p, v, cidx, dq, codes);
}

// running min / max of a chunk; NaN-propagating like torch.amax / amin (v_minimum3 / v_maximum3)
template <class Op>
__device__ __forceinline__ void chunk_minmax(const u32x4& r, float& mn, float& mx) {
  constexpr int N = Vec<Op::BF>::N;
  float v[N];
  unpack<Op::BF>(r, v);
  if constexpr (Op::ABS_ONLY) {                              // the op wants max |x| only: mx carries it, mn is unused
    #pragma unroll
    for (int i = 0; i < N; i += 2) mx = nan_max(nan_max(mx, __builtin_fabsf(v[i])), __builtin_fabsf(v[i + 1]));
  } else {
    #pragma unroll
    for (int i = 0; i < N; i += 2) {
      mn = nan_min(nan_min(mn, v[i]), v[i + 1]);
      mx = nan_max(nan_max(mx, v[i]), v[i + 1]);
    }
  }
}
// range of a row from the per-lane partials
template <int TEAM, bool ABS_ONLY = false>
__device__ __forceinline__ void team_range(float& mn, float& mx) {
  mx = team_reduce<TEAM, true>(mx);
  if constexpr (ABS_ONLY) mn = mx; else mn = team_reduce<TEAM, false>(mn);
}

// ---------------------------------------------------------------------------
// short rows: TEAM lanes per row, ITERS chunks per lane, UNR row batches per wave
// ---------------------------------------------------------------------------
// FULL: every row of the grid exists and every lane owns exactly ITERS chunks (no predicates).
template <class Op, int TEAM, int ITERS, int UNR, bool FULL>
__global__ __launch_bounds__(256) void row_team_kernel(
    const u32x4* __restrict__ x, void* __restrict__ dq, void* __restrict__ codes,
    void* __restrict__ scales, void* __restrict__ zeros, int64_t rows, int nchunks, Op op) {
  constexpr int RPW = LCQ_WAVE / TEAM;                      // rows per wave per batch
  constexpr int N = Vec<Op::BF>::N;
  // one-byte codes of a full grid whose lanes each produce exactly 16 bytes of them
  constexpr bool STAGED = FULL && !Op::HAS_CUSTOM_EMIT && (Op::CD == LCQ_CODE_U8 || Op::CD == LCQ_CODE_I8) && ITERS * N == 16;
  __shared__ uint32_t stage[STAGED ? 4 * RPW * TEAM * 4 : 1];
  const int lane = threadIdx.x & 63;
  const int t = lane & (TEAM - 1);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int64_t row0 = wave * (RPW * UNR) + (lane / TEAM);

  u32x4 raw[UNR][ITERS];
  #pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int64_t row = row0 + (int64_t)u * RPW;
    #pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int ch = t + it * TEAM;
      if (FULL || (row < rows && ch < nchunks)) {
        raw[u][it] = __builtin_nontemporal_load(x + row * nchunks + ch);
        if constexpr (Op::HAS_PRESCALE) raw[u][it] = op.prescale(raw[u][it], row, ch, nchunks);
      } else raw[u][it] = u32x4{0, 0, 0, 0};
    }
  }

  #pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const int64_t row = row0 + (int64_t)u * RPW;
    const bool row_ok = FULL || row < rows;
    typename Op::Row p;
    if (!op.is_static) {
      float mn = __builtin_inff(), mx = -__builtin_inff();
      #pragma unroll
      for (int it = 0; it < ITERS; ++it)
        if (FULL || t + it * TEAM < nchunks) chunk_minmax<Op>(raw[u][it], mn, mx);
      team_range<TEAM, Op::ABS_ONLY>(mn, mx);
      p = op.make(mn, mx);
      if (row_ok && t == 0) op.store_qp(scales, zeros, row, p);
    } else {
      p = op.load(scales, zeros, row_ok ? row : 0);
    }
    if constexpr (STAGED) {
      if (codes) {
        // byte codes: a lane's chunks are 8*TEAM.. elements apart, so direct stores would write 4-8 byte
        // pieces of every line; the words take a detour through LDS (same wave: no barrier) and
        // leave as ONE 16-byte store per lane, a full line per row
        uint32_t* const wrow = stage + (threadIdx.x >> 6) * (RPW * TEAM * 4) + (lane / TEAM) * (TEAM * 4);
        #pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          float v[N], q[N];
          unpack<Op::BF>(raw[u][it], v);
          op.template codes<N>(v, q, p);
          #pragma unroll
          for (int k = 0; k < N / 4; ++k) wrow[(t + it * TEAM) * (N / 4) + k] = op.pack4(q + 4 * k);
          if (dq) {
            #pragma unroll
            for (int i = 0; i < N; ++i) v[i] = op.deq_raw(q[i], p);
            __builtin_nontemporal_store(pack_rne<Op::BF>(v), (u32x4*)dq + (row * nchunks + t + it * TEAM));
          }
        }
        const u32x4 w = *(const u32x4*)(wrow + t * 4);
        *((u32x4*)((uint8_t*)codes + row * (int64_t)(TEAM * 16)) + t) = w;
        continue;
      }
    }
    uint32_t redo = 0;
    #pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int ch = t + it * TEAM;
      if (FULL || (row_ok && ch < nchunks))
        if (!emit_chunk(op, p, raw[u][it], row * nchunks + ch, dq, codes)) redo |= 1u << it;
    }
    if constexpr (Op::HAS_CUSTOM_EMIT) {
      #pragma unroll 1
      for (int it = 0; redo; ++it, redo >>= 1)
        if (redo & 1u) {
          const int ch = t + it * TEAM;
          u32x4 r = x[row * nchunks + ch];
          if constexpr (Op::HAS_PRESCALE) r = op.prescale(r, row, ch, nchunks);
          emit_chunk_slow(op, p, r, row * nchunks + ch, dq, codes);
        }
    }
  }
}

// ---------------------------------------------------------------------------
// long rows: one 256-thread workgroup per row, first CACHE chunks per thread
// stay in registers, the rest is re-read (L2 resident: a row is a few 10 KB)
// ---------------------------------------------------------------------------
template <bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float* sm) {
  v = team_reduce<64, IS_MAX>(v);
  const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sm[w] = v;
  __syncthreads();
  float r = sm[0];
  for (int i = 1; i < nw; ++i) r = IS_MAX ? nan_max(r, sm[i]) : nan_min(r, sm[i]);
  return r;
}

// min and max of a workgroup in one round: two barriers instead of four
template <bool ABS_ONLY = false>
__device__ __forceinline__ void block_range(float& mn, float& mx, float* sm) {
  if constexpr (!ABS_ONLY) mn = team_reduce<64, false>(mn);
  mx = team_reduce<64, true>(mx);
  const int w = threadIdx.x >> 6;
  __syncthreads();                                           // previous readers of sm are done
  if ((threadIdx.x & 63) == 0) { if constexpr (!ABS_ONLY) sm[w] = mn; sm[4 + w] = mx; }
  __syncthreads();
  mx = nan_max(nan_max(sm[4], sm[5]), nan_max(sm[6], sm[7]));
  if constexpr (ABS_ONLY) mn = mx; else mn = nan_min(nan_min(sm[0], sm[1]), nan_min(sm[2], sm[3]));
}

template <class Op, int CACHE>
__global__ __launch_bounds__(256) void row_block_kernel(
    const u32x4* __restrict__ x, void* __restrict__ dq, void* __restrict__ codes,
    void* __restrict__ scales, void* __restrict__ zeros, int64_t rows, int nchunks, Op op) {
  __shared__ float sm[8];
  const int64_t row = blockIdx.x;
  const u32x4* xr = x + row * nchunks;
  u32x4 raw[CACHE];
  #pragma unroll
  for (int k = 0; k < CACHE; ++k) {
    const int ch = threadIdx.x + k * 256;
    raw[k] = (ch < nchunks) ? __builtin_nontemporal_load(xr + ch) : u32x4{0, 0, 0, 0};
    if constexpr (Op::HAS_PRESCALE) if (ch < nchunks) raw[k] = op.prescale(raw[k], row, ch, nchunks);
  }
  typename Op::Row p;
  if (!op.is_static) {
    float mn = __builtin_inff(), mx = -__builtin_inff();
    #pragma unroll
    for (int k = 0; k < CACHE; ++k)
      if ((int)threadIdx.x + k * 256 < nchunks) chunk_minmax<Op>(raw[k], mn, mx);
    for (int ch = threadIdx.x + CACHE * 256; ch < nchunks; ch += 256) {
      u32x4 r = xr[ch];
      if constexpr (Op::HAS_PRESCALE) r = op.prescale(r, row, ch, nchunks);
      chunk_minmax<Op>(r, mn, mx);
    }
    block_range<Op::ABS_ONLY>(mn, mx, sm);
    p = op.make(mn, mx);
    if (threadIdx.x == 0) op.store_qp(scales, zeros, row, p);
  } else {
    p = op.load(scales, zeros, row);
  }
  // chunks the fast path declines are redone by the generic code in the rolled loop at the end
  bool redo = false;
  #pragma unroll
  for (int k = 0; k < CACHE; ++k) {
    const int ch = threadIdx.x + k * 256;
    if (ch < nchunks) redo = !emit_chunk(op, p, raw[k], row * nchunks + ch, dq, codes) || redo;
  }
  for (int ch = threadIdx.x + CACHE * 256; ch < nchunks; ch += 256) {
    u32x4 r = xr[ch];
    if constexpr (Op::HAS_PRESCALE) r = op.prescale(r, row, ch, nchunks);
    redo = !emit_chunk(op, p, r, row * nchunks + ch, dq, codes) || redo;
  }
  if constexpr (Op::HAS_CUSTOM_EMIT) {
    if (__builtin_expect(redo, 0)) {
      // rare: redo every chunk of this lane with the generic code (same results where the fast path ran)
      #pragma unroll 1
      for (int ch = threadIdx.x; ch < nchunks; ch += 256) {
        u32x4 r = xr[ch];
        if constexpr (Op::HAS_PRESCALE) r = op.prescale(r, row, ch, nchunks);
        emit_chunk_slow(op, p, r, row * nchunks + ch, dq, codes);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// any row length / alignment: one wave per row, one element per lane-step
// ---------------------------------------------------------------------------
template <class Op>
__global__ __launch_bounds__(256) void row_scalar_kernel(
    const void* __restrict__ x, void* __restrict__ dq, void* __restrict__ codes,
    void* __restrict__ scales, void* __restrict__ zeros, int64_t rows, int64_t cols, Op op) {
  constexpr int BF = Op::BF;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= rows) return;                                   // whole wave leaves together
  typename Op::Row p;
  if (!op.is_static) {
    float mn = __builtin_inff(), mx = -__builtin_inff();
    for (int64_t j = lane; j < cols; j += 64) {
      float v = load_scalar<BF>(x, row * cols + j);
      if constexpr (Op::HAS_PRESCALE) v = op.prescale1(v, row, j, cols);
      mn = nan_min(mn, v); mx = nan_max(mx, v);
    }
    mn = team_reduce<64, false>(mn);
    mx = team_reduce<64, true>(mx);
    p = op.make(mn, mx);
    if (lane == 0) op.store_qp(scales, zeros, row, p);
  } else {
    p = op.load(scales, zeros, row);
  }
  for (int64_t j = lane; j < cols; j += 64) {
    const int64_t e = row * cols + j;
    float xv = load_scalar<BF>(x, e);
    if constexpr (Op::HAS_PRESCALE) xv = op.prescale1(xv, row, j, cols);
    const float q = op.code(xv, p);
    if (codes) store_code1(op, codes, e, q);
    if (dq) {
      const float d = op.deq(q, p);
      if (op.dq_f32) ((float*)dq)[e] = d; else store_scalar<BF>(dq, e, d);
    }
  }
}

// ---------------------------------------------------------------------------
// host-side dispatch.  Each lane takes up to four 16-byte chunks of its row
// so the per-row parameter arithmetic (IEEE divisions) is amortised over
// 16..32 elements.
// ---------------------------------------------------------------------------
template <class Op, int TEAM, int ITERS, int UNR>
void launch_team(const void* x, void* dq, void* codes, void* scales, void* zeros, int64_t rows, int nchunks,
                 const Op& op, hipStream_t st) {
  constexpr int RPW = LCQ_WAVE / TEAM;
  const int64_t rows_per_block = (int64_t)RPW * UNR * 4;
  const int64_t grid = (rows + rows_per_block - 1) / rows_per_block;
  if (rows % rows_per_block == 0 && nchunks == TEAM * ITERS)
    row_team_kernel<Op, TEAM, ITERS, UNR, true><<<dim3((unsigned)grid), dim3(256), 0, st>>>(
        (const u32x4*)x, dq, codes, scales, zeros, rows, nchunks, op);
  else
    row_team_kernel<Op, TEAM, ITERS, UNR, false><<<dim3((unsigned)grid), dim3(256), 0, st>>>(
        (const u32x4*)x, dq, codes, scales, zeros, rows, nchunks, op);
}

template <class Op>
int dispatch_rows(const void* x, int64_t rows, int64_t cols, void* dq, void* codes, void* scales, void* zeros,
                  const Op& op, bool force_scalar, hipStream_t st) {
  constexpr int N = Vec<Op::BF>::N;
  if (rows > 0x7fffffff) return LCQ_EINVAL;
  const bool aligned = (cols % N == 0) && (((uintptr_t)x | (uintptr_t)dq) % 16 == 0) &&
                       ((uintptr_t)codes % (Op::CD == LCQ_CODE_CT4 ? 4 : 16) == 0);
  if (!aligned || force_scalar) {
    const int64_t grid = (rows + 3) / 4;
    row_scalar_kernel<Op><<<dim3((unsigned)grid), dim3(256), 0, st>>>(x, dq, codes, scales, zeros, rows, cols, op);
    return LCQ_OK;
  }
  const int64_t nch64 = cols / N;
  if (nch64 > 0x7fffffff) return LCQ_EINVAL;
  const int nchunks = (int)nch64;
  #define LCQ_TEAM(T, I, U) launch_team<Op, T, I, U>(x, dq, codes, scales, zeros, rows, nchunks, op, st)
  if (nchunks <= 1) LCQ_TEAM(1, 1, 4);
  else if (nchunks <= 2) LCQ_TEAM(1, 2, 2);
  else if (nchunks <= 4) LCQ_TEAM(1, 4, 1);
  else if (nchunks <= 8) LCQ_TEAM(2, 4, 1);
  else if (nchunks <= 16) LCQ_TEAM(8, 2, 1);       // 8 lanes x 16 B: whole 128-byte lines per row and instruction
  else if (nchunks <= 32) { if constexpr (Op::BF) LCQ_TEAM(8, 4, 1); else LCQ_TEAM(8, 4, 2); }   // fp32 rows of 512 bytes: two rows per team in flight (25.6 -> 23.9 us on 4096 x 4096; four are slower again)
  else if (nchunks <= 64) LCQ_TEAM(16, 4, 1);
  else if (nchunks <= 128) LCQ_TEAM(32, 4, 1);
  else if (nchunks <= 256) LCQ_TEAM(64, 4, 1);
  else {
    row_block_kernel<Op, 4><<<dim3((unsigned)rows), dim3(256), 0, st>>>(
        (const u32x4*)x, dq, codes, scales, zeros, rows, nchunks, op);
  }
  #undef LCQ_TEAM
  return LCQ_OK;
}

}  // namespace lcq
