// GPTQ lazy-batch column loop for gfx950.
//
// Replaces GPTQ.weight_transform (llmc/compression/quantization/gptq.py:198-244)
// together with search_column_qparams (:358-366):
//   for each block of `blocksize` columns:
//     for each column i:  (group boundary -> refresh scale/zero from W[:, i:i+g])
//        q = quant_dequant(w);  tmp[:, i] = w;  Losses[:, i] = (w-q)^2 / (2 d^2)
//        err = (w-q)/d;  W1[:, i:] -= err (x) Hinv1[i, i:];  Err1[:, i] = err
//     W[:, i2:] -= Err1 @ Hinv[i1:i2, i2:]
// The reference issues >= 5 tiny launches per column; here one launch runs the
// 128 sequential columns of a block and fp32-MFMA launches apply the deferred
// update.  The update entry point takes any (contraction range, column range),
// so the host can defer a second time: update only the next few blocks after
// every block and everything behind them once per 1024 columns, which reads
// and writes the bulk of W eight times less often.
//
// Block kernel layout: 16 lanes share one weight row, lane t starts with columns 8t..8t+7 of the
// block in registers; a wave therefore carries 4 rows and a 256-thread workgroup 16.  Every lane
// evaluates the quantizer on its own register (same instruction stream), the owner's error is
// broadcast inside the 16-lane team, and all lanes apply the rank-1 update to their 8 columns from
// the Hinv block held in LDS.  Per-group min/max are 16-lane DPP butterflies.
//
// With R = 4096 rows the kernel has one wave per SIMD on the whole chip, so its run time is the
// length of the per-column dependency chain times 128.  That chain is kept to about ten VALU
// operations:
//  * the quotient w/s goes through the group's reciprocal; an octet (8 columns) in which an owner
//    comes within 2^-11 of a rounding boundary is replayed with true divisions;
//  * (w-q)/d goes through a reciprocal of the diagonal prepared in LDS (at most one ulp from the
//    quotient; it only perturbs later columns, never the rounding of this one);
//  * the registers rotate by one lane after every octet, so the owner is always lane 0 and the
//    broadcast of the error is a DPP row_share:0 instead of an LDS permute, while the loop over
//    octets stays rolled (fully unrolled it is 126 KB of straight-line code that runs at
//    instruction-fetch speed);
//  * the octet's rows of U are fetched from LDS ahead of the chain, and because U is stored zero
//    below the diagonal no update needs a mask;
//  * tmp / (w-q) / err rotate along and are stored once at the end, 32 bytes per lane: a store
//    inside the loop would make every later wait on a load cover it too.
#include <type_traits>

#include "gemm_f32.h"
#include "lcq_internal.h"

namespace {
using namespace lcq;

constexpr int BS = 128;          // columns per block (lazy batch)
// Hinv1 in LDS: a row holds, for each of the 16 lanes of a team, the first four of the lane's eight columns at
// float 4 t and the other four at UH + 4 t, so the two 16-byte reads of a team are each one contiguous run (no bank
// conflicts); the second half starts 4 floats past a multiple of 64 so that a wave's 16-byte stores, which alternate
// between the halves while the block is loaded, do not collide either.
constexpr int UH = 68;           // offset of the second halves inside a row
constexpr int UP = 136;          // row pitch (floats)
__device__ __forceinline__ int us_col(int c) { return ((c & 4) ? UH : 0) + 4 * (c >> 3) + (c & 3); }

struct LoopArgs {
  float* W; float* tmp; float* Losses; float* Err; const float* U;
  const float* W0;      // the weights before the loop, or null: Err then receives q - W0 instead of the errors (see lcq_chol_block_factor)
  float* scales; float* zeros; const int* gidx;
  long long R; int K, Kq, i1, count, g, G, ldErr;      // Kq: columns that are quantized (K unless outlier columns are kept)
  float qmin, qmax;
  int sym, is_static, aligned;
  int nrz;              // round_zp=False: un-rounded zero point inside the rounding, scale clamped at 1e-9 (quant.py:556-557, 702-706)
};

// DPP moves inside every 16-lane row: the value of lane 0, and the value of the next lane (rotation by one)
__device__ __forceinline__ float row16_first(float v) {
  return u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(v), 0x150, 0xf, 0xf, true));          // row_share:0
}
__device__ __forceinline__ float row16_next(float v) {
  return u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(v), 0x12F, 0xf, 0xf, true));          // row_ror:15
}

struct ColQ {           // quantizer of the column being processed
  float s, z, r;        // scale, zero point, 1/s
  float lo, hi;         // qmin - z, qmax - z: clamp(round(t) + z, qmin, qmax) - z == clamp(round(t), lo, hi) for integral z
  bool fast;            // x * r may stand for x / s (guarded) and lo / hi are exact
};
__device__ __forceinline__ ColQ make_colq(float s, float z, float qmin, float qmax, bool nrz = false) {
  ColQ q;
  q.s = s; q.z = z;
  q.r = __builtin_amdgcn_rcpf(s);
  q.lo = qmin - z; q.hi = qmax - z;
  const float a = fabsf(s);
  q.fast = (a > 8.6736174e-19f) & (a < 1.1529215e18f) & (rintf(z) == z) & (fabsf(z) <= 512.0f) & (fabsf(qmin) <= 512.0f) &
           (fabsf(qmax) <= 512.0f) & !nrz;
  return q;
}

// A group opens at column idx: scale and zero point from the range of W[row, idx : min(idx+g, K)] as it is in
// memory now -- trailing updates of earlier blocks applied, this block's own updates not (gptq.py:216-222 reads
// W, not W1).
// `held`: the team's registers when they are exactly that range (group = block, nothing updated yet).
__device__ __forceinline__ ColQ open_group(const LoopArgs& a, int idx, int lane, long long row, bool row_ok, long long rbase,
                                           const float (&held)[8], bool use_held) {
  const int end = min(idx + a.g, a.Kq);
  float mn = __builtin_inff(), mx = -__builtin_inff();
  if (use_held) {
    #pragma unroll
    for (int c = 0; c < 8; ++c) { mn = nan_min(mn, held[c]); mx = nan_max(mx, held[c]); }      // NaN-propagating like torch.amin / amax
  } else {
    for (int col = idx + lane; col < end; col += 16) {
      const float v = a.W[rbase + col];
      mn = nan_min(mn, v); mx = nan_max(mx, v);
    }
  }
  mn = team_reduce<16, false>(mn);
  mx = team_reduce<16, true>(mx);
  float s, z;
  if (a.sym) {
    s = fmaxf(fmaxf(fabsf(mx), fabsf(mn)), 1e-5f) / a.qmax;
    z = 0.0f;
  } else {
    s = fmaxf(mx - mn, 1e-5f) / (a.qmax - a.qmin);
    z = a.nrz ? a.qmin - mn / s : fminf(fmaxf(a.qmin - rintf(mn / s), a.qmin), a.qmax);
  }
  if (row_ok && lane == 0) {
    a.scales[row * a.G + idx / a.g] = s;
    if (!a.sym) a.zeros[row * a.G + idx / a.g] = z;
  }
  return make_colq(s, z, a.qmin, a.qmax, a.nrz);
}

// STATIC: scales / zero points are given (per group, or per column through gidx).  OCT: every group starts on
// a multiple of 8 columns, so groups open only between octets and the 8 columns of an octet are straight-line code.
// RW rows per workgroup (16 lanes each): 16, or 32 for launches of many rows (one copy of Hinv1 in LDS then serves
// eight waves, and two such workgroups put four waves on every SIMD instead of two).
template <bool STATIC, bool OCT, int RW>
__global__ __launch_bounds__(16 * RW) void gptq_block_kernel(LoopArgs a) {
  constexpr int NT = 16 * RW;                    // threads
  constexpr int ROWS_PER_WG = RW;
  constexpr int NP = OCT ? 16 : BS;              // parameter slots of a row: one per octet, or one per column
  __shared__ float Us[BS * UP];                  // Hinv1 = U[i1:i2, i1:i2] above the diagonal, zero everywhere else (us_col layout)
  __shared__ float Rd[BS];                       // 1 / U[i, i]
  __shared__ float Dg[BS];                       // U[i, i]
  __shared__ float Ps[STATIC ? 1 : ROWS_PER_WG * NP], Pz[STATIC ? 1 : ROWS_PER_WG * NP];   // scale, zero point in force
  const int tid = threadIdx.x;
  // full block and 16-byte aligned rows (the entry point checks the base pointers): vector loads and stores
  const bool vec = (a.count == BS) && (a.K % 4 == 0) && (a.i1 % 4 == 0) && a.aligned;
  // The diagonal is zero in LDS as well: a column's own update would only turn it into its quantized value, which
  // nothing reads.  Left alone, the register of a finished column keeps the weight as it was when the column was
  // quantized, which is the `tmp` output, and (w - q), err and the loss are recomputed from it once, after the loop.
  if (vec) {
    // all 16 loads of the thread in flight at once: one after the other they are 16 memory latencies,
    // which used to be most of the kernel's run time
    constexpr int NL = BS * BS / 4 / NT;
    f32x4 v[NL];
    #pragma unroll
    for (int j = 0; j < NL; ++j) {
      const int e = tid + NT * j, r = e >> 5, c = (e & 31) * 4;
      v[j] = *(const f32x4*)(a.U + (long long)(a.i1 + r) * a.K + a.i1 + c);
    }
    #pragma unroll
    for (int j = 0; j < NL; ++j) {
      const int e = tid + NT * j, r = e >> 5, c = (e & 31) * 4;
      #pragma unroll
      for (int k = 0; k < 4; ++k) if (c + k <= r) v[j][k] = 0.0f;
      *(f32x4*)(Us + r * UP + us_col(c)) = v[j];
    }
  } else {
    for (int e = tid; e < BS * BS / 4; e += NT) {
      const int r = (e * 4) / BS, c = (e * 4) % BS;
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (r < a.count) {
        const float* p = a.U + (long long)(a.i1 + r) * a.K + a.i1 + c;
        #pragma unroll
        for (int k = 0; k < 4; ++k) if (c + k < a.count && c + k > r) v[k] = p[k];
      }
      *(f32x4*)(Us + r * UP + us_col(c)) = v;
    }
  }
  if (tid < BS) {
    const float d = (tid < a.count) ? a.U[(long long)(a.i1 + tid) * a.K + a.i1 + tid] : 1.0f;
    Dg[tid] = d;
    Rd[tid] = (tid < a.count) ? 1.0f / d : 0.0f;
  }

  const int lane = tid & 15;                     // physical lane inside the row's team
  const int prow = tid >> 4;                     // the team's row inside the workgroup
  const long long row = (long long)blockIdx.x * ROWS_PER_WG + prow;
  const bool row_ok = row < a.R;
  const long long rbase = (row_ok ? row : 0) * a.K;

  // lane t starts with columns 8t..8t+7 (and, for static groups, their scales and zero points)
  float w[8], ss[8], zz[8];
  if (vec) {                                     // rows of W / tmp / Losses are 16-byte aligned at the block's columns
    const f32x4 lo4 = *(const f32x4*)(a.W + rbase + a.i1 + 8 * lane), hi4 = *(const f32x4*)(a.W + rbase + a.i1 + 8 * lane + 4);
    #pragma unroll
    for (int k = 0; k < 4; ++k) { w[k] = row_ok ? lo4[k] : 0.0f; w[4 + k] = row_ok ? hi4[k] : 0.0f; }
  }
  #pragma unroll
  for (int c = 0; c < 8; ++c) {
    const int col = 8 * lane + c;
    if (!vec) w[c] = (row_ok && col < a.count) ? a.W[rbase + a.i1 + col] : 0.0f;
    ss[c] = 1.0f; zz[c] = 0.0f;
    if (STATIC && col < a.count) {
      const int idx = a.i1 + col;
      const int gi = a.gidx ? a.gidx[idx] : (a.g > 0 ? idx / a.g : 0);
      ss[c] = a.scales[(row_ok ? row : 0) * a.G + gi];
      zz[c] = a.sym ? 0.0f : a.zeros[(row_ok ? row : 0) * a.G + gi];
    }
  }
  ColQ q = make_colq(1.0f, 0.0f, a.qmin, a.qmax);
  int nextb = 0x7fffffff;
  if (!STATIC) {
    nextb = (a.i1 + a.g - 1) / a.g * a.g;
    if (a.i1 % a.g != 0)                         // the block starts inside a group opened by an earlier block
      q = make_colq(a.scales[(row_ok ? row : 0) * a.G + a.i1 / a.g], a.sym ? 0.0f : a.zeros[(row_ok ? row : 0) * a.G + a.i1 / a.g], a.qmin, a.qmax,
                    a.nrz);
  }
  __syncthreads();

  // Octet `to` = columns 8*to .. 8*to+7.  After every octet the registers rotate by one lane inside the team, so
  // the owner of the current octet is always lane 0 (a constant DPP source) and lane p holds the columns of
  // team member (p + to) mod 16.  After the last octet lane p therefore holds the finished columns of octet
  // (p + n_oct) mod 16, eight consecutive columns, and stores them once.  (Stores inside the loop would make every
  // later wait on a load wait for them too.)
  // A lone wave per SIMD issues about one instruction every ten cycles whatever the instruction is, so the run time
  // is the number of instructions per column, not the length of the dependency chain: the loop body holds the
  // chain, the eight fused multiply-adds of the rank-1 update and nothing else.
  const bool first = lane == 0;
  int n_oct = 0;
  for (int to = 0; to < 16; ++to) {
    if (8 * to >= a.count) break;
    ++n_oct;
    // the octet's 8 rows of U (this lane's 8 columns of each) and reciprocal diagonals, fetched ahead of the
    // dependency chain; rows past `count` are zero in LDS, so the 8 columns need no bound check
    const float* ucol = Us + (8 * to) * UP + 4 * ((lane + to) & 15);
    f32x4 u0[8], u1[8];
    #pragma unroll
    for (int c = 0; c < 8; ++c) {
      u0[c] = *(const f32x4*)(ucol + c * UP);
      u1[c] = *(const f32x4*)(ucol + c * UP + UH);
    }
    const f32x4 rda = *(const f32x4*)(Rd + 8 * to), rdb = *(const f32x4*)(Rd + 8 * to + 4);
    const float rd[8] = {rda[0], rda[1], rda[2], rda[3], rdb[0], rdb[1], rdb[2], rdb[3]};
    if (!STATIC && OCT) {
      if (a.i1 + 8 * to == nextb) {
        nextb += a.g;
        q = open_group(a, a.i1 + 8 * to, lane, row, row_ok, rbase, w, to == 0 && a.g == BS && a.count == BS);
      }
      if (first) { Ps[prow * NP + to] = q.s; Pz[prow * NP + to] = q.z; }
    }
    // 8 columns.  Each: quantize-dequantize like clamp(round(w / s) + z, qmin, qmax), (q - z) * s in fp32 (only
    // lane 0's result is used), err = (w - q) / d, rank-1 update of the lane's 8 columns.  U is strictly upper
    // triangular in LDS, so the column itself and the columns left of it see a zero factor and need no mask.
    // The first pass takes the quotient through the reciprocal and only notes how close an owner's product came to
    // a rounding boundary: within 2^-11 product and quotient may round apart, and the wave runs the octet again
    // from the saved registers with true divisions.  (Beyond +-1024 both round outside the clamp range, which
    // make_colq keeps within +-1024 for `fast` parameters; an infinite or NaN product makes the distance NaN.)
    // That keeps every branch out of the chain.
    auto octet = [&](auto exact_tag) -> bool {
      constexpr bool EXACT = decltype(exact_tag)::value;
      float margin = 0.5f;                                  // smallest distance of a product from a rounding boundary
      #pragma unroll
      for (int c = 0; c < 8; ++c) {
        if (STATIC) {
          q = make_colq(ss[c], zz[c], a.qmin, a.qmax, a.nrz);               // lane 0: the parameters of this column
          if (!EXACT) margin = q.fast ? margin : 0.0f;
        } else if (!OCT) {
          if (a.i1 + 8 * to + c == nextb && 8 * to + c < a.count) {
            nextb += a.g;
            q = open_group(a, a.i1 + 8 * to + c, lane, row, row_ok, rbase, w, false);
          }
          if (first) { Ps[prow * NP + 8 * to + c] = q.s; Pz[prow * NP + 8 * to + c] = q.z; }
        }
        const float wv = w[c];
        float diff;
        if (EXACT) {
          const float code = a.nrz ? rintf(wv / fmaxf(q.s, 1e-9f) + q.z) : rintf(wv / q.s) + q.z;
          diff = wv - (__builtin_amdgcn_fmed3f(code, a.qmin, a.qmax) - q.z) * q.s;
        } else {
          const float t = wv * q.r, rt = rintf(t);
          margin = nan_min(margin, fabsf(fabsf(t - rt) - 0.5f));
          diff = wv - __builtin_amdgcn_fmed3f(rt, q.lo, q.hi) * q.s;
        }
        const float eb = row16_first(diff * rd[c]);
        #pragma unroll
        for (int k = 0; k < 4; ++k) {
          w[k] = __builtin_fmaf(-eb, u0[c][k], w[k]);
          w[4 + k] = __builtin_fmaf(-eb, u1[c][k], w[4 + k]);
        }
      }
      if (EXACT) return false;
      return first & !((margin > 4.8828125e-04f) & (STATIC || q.fast));
    };
    if (STATIC || OCT) {
      float saved[8];
      #pragma unroll
      for (int c = 0; c < 8; ++c) saved[c] = w[c];
      const bool unsure = octet(std::false_type{});
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(unsure) != 0, 0)) {
        #pragma unroll
        for (int c = 0; c < 8; ++c) w[c] = saved[c];
        octet(std::true_type{});
      }
    } else {
      octet(std::true_type{});          // groups may open inside the octet: no replay, divide throughout
    }
    #pragma unroll
    for (int c = 0; c < 8; ++c) {
      w[c] = row16_next(w[c]);
      if (STATIC) { ss[c] = row16_next(ss[c]); zz[c] = row16_next(zz[c]); }
    }
  }

  // Outputs of the lane's eight finished columns.  w still holds each column as it was when it was quantized; the
  // quantized value, with true divisions, is the one the loop used (its reciprocal form is only taken where it
  // rounds like the division), and err = (w - q) * (1 / d) as in the loop.
  const int oct = (lane + n_oct) & 15;                      // the octet whose columns this lane holds now
  if (row_ok && 8 * oct < a.count) {
    float o_err[8], loss[8];
    #pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int col = 8 * oct + c;
      float s_, z_;
      if (STATIC) { s_ = ss[c]; z_ = zz[c]; }
      else { s_ = Ps[prow * NP + (OCT ? oct : col)]; z_ = Pz[prow * NP + (OCT ? oct : col)]; }
      if (col >= a.count) { s_ = 1.0f; z_ = 0.0f; }
      const float wv = w[c];
      const float code = a.nrz ? rintf(wv / fmaxf(s_, 1e-9f) + z_) : rintf(wv / s_) + z_;
      const float qdq = (__builtin_amdgcn_fmed3f(code, a.qmin, a.qmax) - z_) * s_;
      const float diff = wv - qdq;
      o_err[c] = diff * Rd[col];
      if (a.W0) o_err[c] = (col < a.count) ? qdq - a.W0[rbase + a.i1 + col] : 0.0f;
      const float d = Dg[col];
      loss[c] = (diff * diff) / (2.0f * (d * d));
    }
    if (vec) {
      float* pt = a.tmp + rbase + a.i1 + 8 * oct;
      float* pl = a.Losses + rbase + a.i1 + 8 * oct;
      *(f32x4*)pt = f32x4{w[0], w[1], w[2], w[3]};
      *(f32x4*)(pt + 4) = f32x4{w[4], w[5], w[6], w[7]};
      *(f32x4*)pl = f32x4{loss[0], loss[1], loss[2], loss[3]};
      *(f32x4*)(pl + 4) = f32x4{loss[4], loss[5], loss[6], loss[7]};
    }
    float* pe = a.Err + row * a.ldErr + 8 * oct;
    if (vec && a.ldErr % 4 == 0 && (reinterpret_cast<uintptr_t>(a.Err) & 15) == 0) {
      *(f32x4*)pe = f32x4{o_err[0], o_err[1], o_err[2], o_err[3]};
      *(f32x4*)(pe + 4) = f32x4{o_err[4], o_err[5], o_err[6], o_err[7]};
    } else {
      #pragma unroll
      for (int c = 0; c < 8; ++c) if (8 * oct + c < a.count) pe[c] = o_err[c];
    }
    if (!vec) {
      #pragma unroll
      for (int c = 0; c < 8; ++c) {
        const int col = 8 * oct + c;
        if (col < a.count) {
          a.tmp[rbase + a.i1 + col] = w[c];
          a.Losses[rbase + a.i1 + col] = loss[c];
        }
      }
    }
  }
}

}  // namespace

extern "C" {

int lcq_gptq_block(float* W, float* tmp, float* Losses, float* Err, int64_t ldErr, const float* U, const float* W0, int64_t R,
                   int64_t K, int64_t n_quant, int64_t i1, int count, int group_size, float qmin, float qmax, int flags, float* scales, float* zeros,
                   const int32_t* gidx, int64_t G, void* stream) {
  if (!W || !tmp || !Losses || !Err || !U || !scales || ldErr < count || ldErr > 0x7fffffff) return LCQ_EINVAL;
  if (R <= 0 || K <= 0 || K > 0x7fffffff || i1 < 0 || count <= 0 || count > BS) return LCQ_EINVAL;
  if (n_quant <= 0 || n_quant > K || i1 + count > n_quant) return LCQ_EINVAL;
  if (!(qmax > qmin) || G <= 0) return LCQ_EINVAL;
  const int is_static = (flags & LCQ_FLAG_STATIC) != 0;
  const int sym = (flags & LCQ_FLAG_SYM) != 0;
  if (!is_static && (group_size <= 0 || G < (n_quant + group_size - 1) / group_size)) return LCQ_EINVAL;
  if (!sym && !zeros) return LCQ_EINVAL;
  LoopArgs a;
  a.W = W; a.tmp = tmp; a.Losses = Losses; a.Err = Err; a.U = U; a.W0 = W0;
  a.scales = scales; a.zeros = zeros; a.gidx = gidx;
  a.R = R; a.K = (int)K; a.Kq = (int)n_quant; a.i1 = (int)i1; a.count = count; a.g = group_size; a.G = (int)G;
  a.qmin = qmin; a.qmax = qmax; a.sym = sym; a.is_static = is_static; a.ldErr = (int)ldErr;
  a.nrz = (flags & LCQ_FLAG_NO_ROUND_ZP) != 0;
  a.aligned = ((reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(tmp) | reinterpret_cast<uintptr_t>(Losses) |
                reinterpret_cast<uintptr_t>(U)) & 15) == 0;
  const bool oct = !is_static && group_size % 8 == 0 && i1 % 8 == 0;
  hipStream_t st = (hipStream_t)stream;
  // From 6144 rows on, 32 rows per workgroup: one copy of Hinv1 in LDS (70 KB) per eight waves, so that the two
  // workgroups a CU holds put four waves on every SIMD (R = 28672: 57 -> 48 us per block, 14336: 35 -> 29, 6144:
  // 20 -> 19; at 4096 rows, one workgroup per CU either way, the smaller workgroup is faster, 17 against 19 us).
  // The rows do not interact: the results are the same bit for bit.
  if (R >= 6144 && (is_static || oct) && !(flags & LCQ_FLAG_ROWS16)) {
    const unsigned grid = (unsigned)((R + 31) / 32);
    if (is_static) gptq_block_kernel<true, true, 32><<<dim3(grid), dim3(512), 0, st>>>(a);
    else gptq_block_kernel<false, true, 32><<<dim3(grid), dim3(512), 0, st>>>(a);
  } else {
    const unsigned grid = (unsigned)((R + 15) / 16);
    if (is_static) gptq_block_kernel<true, true, 16><<<dim3(grid), dim3(256), 0, st>>>(a);
    else if (oct) gptq_block_kernel<false, true, 16><<<dim3(grid), dim3(256), 0, st>>>(a);
    else gptq_block_kernel<false, false, 16><<<dim3(grid), dim3(256), 0, st>>>(a);
  }
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_gptq_trailing(float* W, const float* Err, int64_t ldErr, const float* U, int64_t R, int64_t K, int64_t k1,
                      int64_t k2, int64_t j1, int64_t j2, void* stream) {
  if (!W || !Err || !U || R <= 0 || K <= 0 || K > 0x7fffffff || R > 0x7fffffff) return LCQ_EINVAL;
  if (k1 < 0 || k2 <= k1 || k2 > K || j1 < k2 || j2 < j1 || j2 > K || ldErr < k2 - k1 || ldErr > 0x7fffffff) return LCQ_EINVAL;
  if (j1 == j2) return LCQ_OK;
  // W[:, j1:j2] -= Err[:, :k2-k1] @ U[k1:k2, j1:j2]
  GemmProblem g{Err, U + k1 * K + j1, W + j1, (int)R, (int)(j2 - j1), (int)(k2 - k1), (int)ldErr, (int)K, (int)K};
  launch_gemm<false>(g, -1.0f, 1.0f, 0, (hipStream_t)stream);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
