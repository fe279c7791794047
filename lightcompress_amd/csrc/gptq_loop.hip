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
// Block kernel layout: 16 lanes share one weight row, lane t keeps columns
// 8t..8t+7 of the block in registers; a wave therefore carries 4 rows and a
// 256-thread workgroup 16.  Column i lives on lane i/8: every lane evaluates
// the quantizer on its own register (same instruction stream), the owner's
// error is broadcast inside the 16-lane team with ds_bpermute, and all lanes
// apply the rank-1 update to their 8 columns from the Hinv block held in LDS.
// Per-group min/max are 16-lane DPP butterflies.  tmp / Losses / Err are kept
// in registers and written once, 32 bytes per lane.
#include "gemm_f32.h"
#include "lcq_internal.h"

namespace {
using namespace lcq;

constexpr int BS = 128;          // columns per block (lazy batch)
constexpr int ROWS_PER_WG = 16;

struct LoopArgs {
  float* W; float* tmp; float* Losses; float* Err; const float* U;
  float* scales; float* zeros; const int* gidx;
  long long R; int K, i1, count, g, G, ldErr;
  float qmin, qmax;
  int sym, is_static;
};

__device__ __forceinline__ float team16_bcast(float v, int src) {   // value of lane (lane & ~15) | src
  return u2f((uint32_t)__builtin_amdgcn_ds_bpermute((int)(((threadIdx.x & ~15) | src) << 2), (int)f2u(v)));
}

__global__ __launch_bounds__(256) void gptq_block_kernel(LoopArgs a) {
  __shared__ float Us[BS * BS];                  // Hinv1 = U[i1:i2, i1:i2]
  const int tid = threadIdx.x;
  for (int e = tid; e < BS * BS / 4; e += 256) {
    const int r = (e * 4) / BS, c = (e * 4) % BS;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (r < a.count) {
      const float* p = a.U + (long long)(a.i1 + r) * a.K + a.i1 + c;
      #pragma unroll
      for (int k = 0; k < 4; ++k) if (c + k < a.count) v[k] = p[k];
    }
    *(f32x4*)(Us + e * 4) = v;
  }

  const int t = tid & 15;
  const long long row = (long long)blockIdx.x * ROWS_PER_WG + (tid >> 4);
  const bool row_ok = row < a.R;
  const long long rbase = (row_ok ? row : 0) * a.K;

  float w[8], otmp[8], oloss[8], oerr[8];
  #pragma unroll
  for (int c = 0; c < 8; ++c) {
    const int col = 8 * t + c;
    w[c] = (row_ok && col < a.count) ? a.W[rbase + a.i1 + col] : 0.0f;
    otmp[c] = 0.0f; oloss[c] = 0.0f; oerr[c] = 0.0f;
  }
  __syncthreads();

  float s = 1.0f, z = 0.0f;
  const float qrange = a.qmax - a.qmin;
  for (int to = 0; to < 16; ++to) {              // owner lane of columns 8*to .. 8*to+7
    if (8 * to >= a.count) break;
    #pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int i = 8 * to + c;
      const int idx = a.i1 + i;
      if (i < a.count) {
        // ---- per-group parameters (uniform branch: idx is the same for every lane) ----
        if (a.is_static) {
          const int gi = a.gidx ? a.gidx[idx] : (a.g > 0 ? idx / a.g : 0);
          if (i == 0 || a.gidx || (a.g > 0 && idx % a.g == 0)) {
            s = a.scales[(row_ok ? row : 0) * a.G + gi];
            z = a.sym ? 0.0f : a.zeros[(row_ok ? row : 0) * a.G + gi];
          }
        } else if (idx % a.g == 0) {
          // range of W[row, idx : min(idx+g, K)] as it is in memory now: trailing updates of
          // earlier blocks applied, this block's own updates not (gptq.py:216-222 reads W, not W1)
          const int end = min(idx + a.g, a.K);
          float mn = __builtin_inff(), mx = -__builtin_inff();
          for (int col = idx + t; col < end; col += 16) {
            const float v = a.W[rbase + col];
            mn = fminf(mn, v); mx = fmaxf(mx, v);
          }
          mn = team_reduce<16, false>(mn);
          mx = team_reduce<16, true>(mx);
          if (a.sym) {
            s = fmaxf(fmaxf(fabsf(mx), fabsf(mn)), 1e-5f) / a.qmax;
            z = 0.0f;
          } else {
            s = fmaxf(mx - mn, 1e-5f) / qrange;
            z = fminf(fmaxf(a.qmin - rintf(mn / s), a.qmin), a.qmax);
          }
          if (row_ok && t == 0) {
            a.scales[row * a.G + idx / a.g] = s;
            if (!a.sym) a.zeros[row * a.G + idx / a.g] = z;
          }
        } else if (i == 0) {
          // the block starts inside a group opened by an earlier block
          s = a.scales[(row_ok ? row : 0) * a.G + idx / a.g];
          z = a.sym ? 0.0f : a.zeros[(row_ok ? row : 0) * a.G + idx / a.g];
        }
        // ---- quantize this lane's register c (meaningful on the owner lane) ----
        const float d = Us[i * BS + i];
        const float wv = w[c];
        float q = rintf(wv / s) + z;
        q = fminf(fmaxf(q, a.qmin), a.qmax);
        const float dq = (q - z) * s;
        const float diff = wv - dq;
        const float err = diff / d;
        if (t == to) {
          otmp[c] = wv;
          oloss[c] = (diff * diff) / (2.0f * (d * d));
          oerr[c] = err;
        }
        const float eb = team16_bcast(err, to);
        // ---- rank-1 update of the remaining columns of the block ----
        const f32x4 u0 = *(const f32x4*)(Us + i * BS + 8 * t);
        const f32x4 u1 = *(const f32x4*)(Us + i * BS + 8 * t + 4);
        #pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (8 * t + k > i) w[k] -= eb * u0[k];
          if (8 * t + 4 + k > i) w[4 + k] -= eb * u1[k];
        }
      }
    }
  }

  if (row_ok) {
    #pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int col = 8 * t + c;
      if (col < a.count) {
        a.tmp[rbase + a.i1 + col] = otmp[c];
        a.Losses[rbase + a.i1 + col] = oloss[c];
        a.Err[row * a.ldErr + col] = oerr[c];
      }
    }
  }
}

}  // namespace

extern "C" {

int lcq_gptq_block(float* W, float* tmp, float* Losses, float* Err, int64_t ldErr, const float* U, int64_t R, int64_t K,
                   int64_t i1, int count, int group_size, float qmin, float qmax, int flags, float* scales, float* zeros,
                   const int32_t* gidx, int64_t G, void* stream) {
  if (!W || !tmp || !Losses || !Err || !U || !scales || ldErr < count || ldErr > 0x7fffffff) return LCQ_EINVAL;
  if (R <= 0 || K <= 0 || K > 0x7fffffff || i1 < 0 || count <= 0 || count > BS || i1 + count > K) return LCQ_EINVAL;
  if (!(qmax > qmin) || G <= 0) return LCQ_EINVAL;
  const int is_static = (flags & LCQ_FLAG_STATIC) != 0;
  const int sym = (flags & LCQ_FLAG_SYM) != 0;
  if (!is_static && (group_size <= 0 || G < (K + group_size - 1) / group_size)) return LCQ_EINVAL;
  if (!sym && !zeros) return LCQ_EINVAL;
  LoopArgs a;
  a.W = W; a.tmp = tmp; a.Losses = Losses; a.Err = Err; a.U = U;
  a.scales = scales; a.zeros = zeros; a.gidx = gidx;
  a.R = R; a.K = (int)K; a.i1 = (int)i1; a.count = count; a.g = group_size; a.G = (int)G;
  a.qmin = qmin; a.qmax = qmax; a.sym = sym; a.is_static = is_static; a.ldErr = (int)ldErr;
  const unsigned grid = (unsigned)((R + ROWS_PER_WG - 1) / ROWS_PER_WG);
  gptq_block_kernel<<<dim3(grid), dim3(256), 0, (hipStream_t)stream>>>(a);
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
