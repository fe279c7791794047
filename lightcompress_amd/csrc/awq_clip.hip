// AWQ weight-clip search for gfx950.
//
// Replaces AutoClipper.auto_clip_layer / fake_quantize_weight (clip_version v1, weight-only;
// llmc/compression/quantization/auto_clip.py:83-191, 258-262) and apply_clip v1 (:194-211).
// For every (output row r, group g) the reference tries n_steps shrunken ranges
//   max_i = org_max * (1 - i/n_grid),  min_i = org_min * (1 - i/n_grid)      (or -max_i)
// fake-quantizes clamp(w, min_i, max_i) and keeps the range whose per-group partial outputs
//   out[r, t, g] = sum_j x[t, g, j] * w_q[r, g, j]
// are closest (mean over the sampled tokens t of the squared difference) to those of the
// original weights.  It materialises [256, T, G, 128] products per shrink step; here a wave keeps
// 32 rows of one group in registers, derives the bf16 weight DIFFERENCE of every step there and
// multiplies it with the group's token tile (LDS) on bf16 MFMA:
//   err_i[r] = mean_t ( sum_j x[t, j] * (fq_i(w) - w)[r, j] )^2
// The reference rounds both dot products to bf16 before subtracting them; that rounding noise
// (2^-9 of the outputs) is not reproduced, the decision rule is: errors are rounded to bf16 and
// compared with <, so the first minimum wins exactly as `err_mean < min_errs` does.
//
// GEMM shape per wave and step: tokens (M, from LDS) x 32 weight rows (N, registers) x 128 (K).
// With v_mfma_f32_32x32x16_bf16 lane (h = lane/32, c = lane%32) supplies token c / weight row c
// and k = 16 ks + 8 h .. +7 of k-step ks; accumulator register r holds token 8(r/4)+4h+r%4 of
// weight row c, so the sum over tokens is a sum over a lane's registers plus its partner lane.
#include "intop.h"

namespace {
using namespace lcq;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int CG = 128;                  // group size
constexpr int TS = 512;                  // tokens per LDS pass
constexpr int PITCH = CG * 2 + 16;       // bytes per token row in LDS (16-byte skew against bank conflicts)
constexpr int ROWS_PER_WG = 256;         // 8 waves x 32 rows

__global__ __launch_bounds__(512, 1) void awq_clip_kernel(const uint16_t* __restrict__ w, const uint16_t* __restrict__ x,
                                                          int R, int K, int T, int n_grid, int n_steps, int clip_sym,
                                                          IntOp<true, true> op, uint16_t* __restrict__ best_max,
                                                          uint16_t* __restrict__ best_min, float* __restrict__ errs) {
  __shared__ __attribute__((aligned(16))) char lds[TS * PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = lane >> 5, c = lane & 31;
  const int gi = blockIdx.y, G = K / CG;
  const int row = blockIdx.x * ROWS_PER_WG + wave * 32 + c;
  const bool row_ok = row < R;
  const int npass = (T + TS - 1) / TS;

  auto load_tokens = [&](int t0) {                          // tokens t0 .. t0+TS of group gi -> LDS, zero past T
    const int c16 = tid & 15, tr = tid >> 4;
    #pragma unroll 4
    for (int it = 0; it < TS / 32; ++it) {
      const int t = it * 32 + tr;
      u32x4 v = {0, 0, 0, 0};
      if (t0 + t < T) v = *(const u32x4*)(x + (int64_t)(t0 + t) * K + gi * CG + c16 * 8);
      *(u32x4*)(lds + t * PITCH + c16 * 16) = v;
    }
  };

  // this lane's 64 weights of row `row`: j = 16 ks + 8 h + i
  u32x4 wf[8];
  #pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    wf[ks] = u32x4{0, 0, 0, 0};
    if (row_ok) wf[ks] = *(const u32x4*)(w + (int64_t)row * K + gi * CG + 16 * ks + 8 * h);
  }
  float mn = __builtin_inff(), mx = -__builtin_inff();
  #pragma unroll
  for (int ks = 0; ks < 8; ++ks) chunk_minmax<IntOp<true, true>>(wf[ks], mn, mx);
  mn = nan_min(mn, __shfl_xor(mn, 32));
  mx = nan_max(mx, __shfl_xor(mx, 32));
  const float org_min = mn;
  const float org_max = clip_sym ? nan_max(fabsf(mn), fabsf(mx)) : mx;       // w.abs().amax when clip_sym

  if (npass == 1) { load_tokens(0); __syncthreads(); }

  float best = 999817216.0f;                                // bf16(1e9), min_errs = ones_like * 1e9
  float bmax = org_max, bmin = org_min;
  for (int s = 0; s < n_steps; ++s) {
    const float fs = (float)(1.0 - (double)s / (double)n_grid);
    const float max_s = rnd<true>(org_max * fs);
    const float min_s = clip_sym ? -max_s : rnd<true>(org_min * fs);
    // range of the clamped group = clamped range (clamp is monotone)
    const IntRow p = op.make(fminf(fmaxf(mn, min_s), max_s), fminf(fmaxf(mx, min_s), max_s));
    u32x4 bfrag[8];
    #pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      float wv[8], cv[8], d[8];
      unpack<true>(wf[ks], wv);
      #pragma unroll
      for (int i = 0; i < 8; ++i) cv[i] = fminf(fmaxf(wv[i], min_s), max_s);
      op.template fused_dq<8>(cv, d, p);
      #pragma unroll
      for (int i = 0; i < 8; i += 2) rnd_pair<true>(d[i], d[i + 1]);           // fake-quantized weight (bf16)
      #pragma unroll
      for (int i = 0; i < 8; ++i) d[i] -= wv[i];                               // exact in fp32
      bfrag[ks] = pack_rne<true>(d);
    }
    float e = 0.0f;
    for (int ps = 0; ps < npass; ++ps) {
      if (npass > 1) { __syncthreads(); load_tokens(ps * TS); __syncthreads(); }
      const int nt = min(TS, T - ps * TS);
      for (int tb = 0; tb * 32 < nt; ++tb) {
        f32x16 acc;
        #pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
        const char* a0 = lds + (tb * 32 + c) * PITCH + 16 * h;
        #pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          const u32x4 a = *(const u32x4*)(a0 + 32 * ks);
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, bfrag[ks]),
                                                        acc, 0, 0, 0);
        }
        #pragma unroll
        for (int r = 0; r < 16; ++r) e = __builtin_fmaf(acc[r], acc[r], e);
      }
    }
    e += __shfl_xor(e, 32);
    const float mean = e * (1.0f / (float)T);       // torch's GPU mean: the sum times an fp32 factor
    if (errs && row_ok && h == 0) errs[((int64_t)row * G + gi) * n_steps + s] = mean;
    const float eb = rnd<true>(mean);
    if (eb < best) { best = eb; bmax = max_s; bmin = min_s; }
  }
  if (row_ok && h == 0) {
    best_max[(int64_t)row * G + gi] = (uint16_t)(f2u(bmax) >> 16);
    best_min[(int64_t)row * G + gi] = (uint16_t)(f2u(bmin) >> 16);
  }
}

template <int BF>
__global__ __launch_bounds__(256) void clamp_groups_kernel(const u32x4* __restrict__ w, int64_t nchunks, int cpg,
                                                           const void* __restrict__ lo, const void* __restrict__ hi,
                                                           u32x4* __restrict__ out) {
  constexpr int N = Vec<BF>::N;
  for (int64_t ch = (int64_t)blockIdx.x * 256 + threadIdx.x; ch < nchunks; ch += (int64_t)gridDim.x * 256) {
    const int64_t grp = ch / cpg;
    const float l = load_scalar<BF>(lo, grp), u = load_scalar<BF>(hi, grp);
    float v[N];
    unpack<BF>(w[ch], v);
    #pragma unroll
    for (int i = 0; i < N; ++i) v[i] = nan_min(nan_max(v[i], l), u);          // torch.clamp: min(max(x, lo), hi)
    out[ch] = pack<BF>(v);
  }
}

// the same clamp element by element, for group sizes that do not fill 16-byte chunks
template <int BF>
__global__ __launch_bounds__(256) void clamp_groups_scalar_kernel(const void* __restrict__ w, int64_t n, int gs,
                                                                  const void* __restrict__ lo, const void* __restrict__ hi,
                                                                  void* __restrict__ out) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t grp = i / gs;
    store_scalar<BF>(out, i, nan_min(nan_max(load_scalar<BF>(w, i), load_scalar<BF>(lo, grp)), load_scalar<BF>(hi, grp)));
  }
}

// out[r, g, t] = round( sum_j round(x[t, g*gs + j] * w[r, g*gs + j]) ): the reference's (x * w).sum(dim=-1) of
// auto_clip.py:141,160 on x [1, T, G, gs] and w [R, 1, G, gs] - the product tensor is materialised in the tensors'
// type there (every product rounded), the sum accumulates in fp32 and rounds once.  General in the group size, the
// element type and which tensors are multiplied, so it serves every configuration the MFMA search kernel leaves out
// (activation fake-quant, learnable ranges, other group sizes) and reproduces the reference's rounding sequence.
// With `org` (the same sums for the original weights) the sums are not stored; the kernel goes on to
//   err[r, g] = round( mean_t round( round(out - org)^2 ) )                    (auto_clip.py:163)
// One workgroup: 64 rows x one group, looping over 64-token tiles and 128-column chunks staged in LDS as fp32; thread
// (ty, tx) = (tid / 16, tid % 16) owns rows ty + 16 a and tokens tx + 16 b (a, b = 0..3): 8 LDS reads per 16 products.
constexpr int GD_J = 128, GD_P = GD_J + 1, GD_M = 64;
template <int BF>
__device__ __forceinline__ void gd_stage(float (*S)[GD_P], const void* __restrict__ src, int row0, int nrows, int K,
                                         int64_t col0, int nj, bool vec, int tid) {
  constexpr int N = Vec<BF>::N;
  if (vec) {                                                // 16-byte pieces: K, the group offset and nj are multiples of N
    for (int e = tid; e < GD_M * (GD_J / N); e += 256) {
      const int rr = e / (GD_J / N), c = (e % (GD_J / N)) * N;
      float v[N];
      #pragma unroll
      for (int i = 0; i < N; ++i) v[i] = 0.0f;
      if (rr + row0 < nrows && c < nj) {
        const char* p = (const char*)src + ((int64_t)(row0 + rr) * K + col0 + c) * (BF ? 2 : 4);
        unpack<BF>(*(const u32x4*)p, v);
      }
      #pragma unroll
      for (int i = 0; i < N; ++i) S[rr][c + i] = v[i];
    }
  } else {
    for (int e = tid; e < GD_M * GD_J; e += 256) {
      const int rr = e / GD_J, j = e % GD_J;
      S[rr][j] = (j < nj && row0 + rr < nrows) ? load_scalar<BF>(src, (int64_t)(row0 + rr) * K + col0 + j) : 0.0f;
    }
  }
}

template <int BF>
__global__ __launch_bounds__(256) void group_dots_kernel(const void* __restrict__ x, const void* __restrict__ w, int R, int K,
                                                         int T, int gs, int vec, void* __restrict__ out,
                                                         const void* __restrict__ org, void* __restrict__ err) {
  __shared__ float Xs[GD_M][GD_P], Ws[GD_M][GD_P];
  const int tid = threadIdx.x, G = K / gs, g = blockIdx.y;
  const int r0 = blockIdx.x * GD_M, ty = tid >> 4, tx = tid & 15;
  const bool one_chunk = gs <= GD_J;
  float esum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (one_chunk) gd_stage<BF>(Ws, w, r0, R, K, (int64_t)g * gs, gs, vec, tid);
  for (int t0 = 0; t0 < T; t0 += GD_M) {
    float acc[4][4];
    #pragma unroll
    for (int a = 0; a < 4; ++a)
      #pragma unroll
      for (int b = 0; b < 4; ++b) acc[a][b] = 0.0f;
    for (int j0 = 0; j0 < gs; j0 += GD_J) {
      const int nj = min(GD_J, gs - j0);
      __syncthreads();
      gd_stage<BF>(Xs, x, t0, T, K, (int64_t)g * gs + j0, nj, vec, tid);
      if (!one_chunk) gd_stage<BF>(Ws, w, r0, R, K, (int64_t)g * gs + j0, nj, vec, tid);
      __syncthreads();
      for (int j = 0; j < nj; ++j) {
        float wv[4], xv[4];
        #pragma unroll
        for (int a = 0; a < 4; ++a) wv[a] = Ws[ty + 16 * a][j];
        #pragma unroll
        for (int b = 0; b < 4; ++b) xv[b] = Xs[tx + 16 * b][j];
        #pragma unroll
        for (int a = 0; a < 4; ++a)
          #pragma unroll
          for (int b = 0; b < 4; b += 2) {
            float p0 = xv[b] * wv[a], p1 = xv[b + 1] * wv[a];
            rnd_pair<BF>(p0, p1);
            acc[a][b] += p0;
            acc[a][b + 1] += p1;
          }
      }
    }
    #pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int r = r0 + ty + 16 * a;
      #pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int t = t0 + tx + 16 * b;
        if (r < R && t < T) {
          const int64_t at = ((int64_t)r * G + g) * T + t;
          const float v = rnd_e<BF>(acc[a][b]);
          if (org) {
            const float d = rnd_e<BF>(v - load_scalar<BF>(org, at));
            esum[a] += rnd_e<BF>(d * d);
          } else {
            store_scalar<BF>(out, at, v);
          }
        }
      }
    }
  }
  if (org) {
    #pragma unroll
    for (int a = 0; a < 4; ++a) {
      const float s = team_sum<16>(esum[a]);
      const int r = r0 + ty + 16 * a;
      if (tx == 0 && r < R) store_scalar<BF>(err, (int64_t)r * G + g, rnd_e<BF>(s * (1.0f / (float)T)));
    }
  }
}

}  // namespace

extern "C" {

int lcq_group_dots(const void* x, const void* w, int dtype, int64_t R, int64_t K, int64_t T, int group_size, void* out,
                   const void* org, void* err, void* stream) {
  if (!x || !w || R <= 0 || K <= 0 || T <= 0 || group_size <= 0 || K % group_size != 0) return LCQ_EINVAL;
  if ((org && !err) || (!org && !out)) return LCQ_EINVAL;
  if (R > 0x7fffffff || K > 0x7fffffff || T > 0x7fffffff || K / group_size > 65535) return LCQ_EINVAL;
  if (dtype != LCQ_BF16 && dtype != LCQ_F32 && dtype != LCQ_F16) return LCQ_EDTYPE;
  const int n = dtype == LCQ_F32 ? 4 : 8;
  const int vec = (K % n == 0 && group_size % n == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0) ? 1 : 0;
  const dim3 grid((unsigned)((R + GD_M - 1) / GD_M), (unsigned)(K / group_size));
  hipStream_t st = (hipStream_t)stream;
  if (dtype == LCQ_BF16)
    group_dots_kernel<true><<<grid, dim3(256), 0, st>>>(x, w, (int)R, (int)K, (int)T, group_size, vec, out, org, err);
  else if (dtype == LCQ_F16)
    group_dots_kernel<ROW_F16><<<grid, dim3(256), 0, st>>>(x, w, (int)R, (int)K, (int)T, group_size, vec, out, org, err);
  else
    group_dots_kernel<false><<<grid, dim3(256), 0, st>>>(x, w, (int)R, (int)K, (int)T, group_size, vec, out, org, err);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_awq_clip_search(const void* w, const void* x, int64_t R, int64_t K, int64_t T, int n_grid, int n_steps,
                        int clip_sym, float qmin, float qmax, int flags, void* best_max, void* best_min, float* errs,
                        void* stream) {
  if (!w || !x || !best_max || !best_min || R <= 0 || K <= 0 || T <= 0) return LCQ_EINVAL;
  if (K % CG != 0 || K > 0x7fffffff / 2 || R > 0x7fffffff || T > 0x7fffffff) return LCQ_EINVAL;
  if (n_grid <= 0 || n_steps <= 0 || n_steps > n_grid) return LCQ_EINVAL;
  if (!(qmax > qmin) || qmax > 256.0f || qmin < -256.0f || (flags & (LCQ_FLAG_STATIC | LCQ_FLAG_NO_ROUND_ZP))) return LCQ_EINVAL;
  if ((((uintptr_t)w | (uintptr_t)x) % 16) != 0) return LCQ_EALIGN;
  IntOp<true, true> op;
  op.qmin = qmin; op.qmax = qmax; op.qrange = qmax - qmin; op.osf = 1.0f;
  op.rqmax = (float)(1.0 / (double)qmax); op.rqrange = (float)(1.0 / (double)(qmax - qmin));
  op.sym = (flags & LCQ_FLAG_SYM) != 0; op.round_zp = 1; op.is_static = 0; op.scalar_qp = 0; op.dq_f32 = 0;
  op.range_bf16 = 0; op.range_f16 = 0; op.scale_f32 = 0; op.colscale = nullptr; op.wrow_cols = 1; op.code_dtype = LCQ_CODE_NONE;
  const dim3 grid((unsigned)((R + ROWS_PER_WG - 1) / ROWS_PER_WG), (unsigned)(K / CG));
  awq_clip_kernel<<<grid, dim3(512), 0, (hipStream_t)stream>>>((const uint16_t*)w, (const uint16_t*)x, (int)R, (int)K,
                                                               (int)T, n_grid, n_steps, clip_sym, op, (uint16_t*)best_max,
                                                               (uint16_t*)best_min, errs);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_clamp_groups(const void* w, int dtype, int64_t R, int64_t K, int group_size, const void* lo, const void* hi,
                     void* out, void* stream) {
  if (!w || !lo || !hi || !out || R <= 0 || K <= 0 || group_size <= 0 || K % group_size != 0) return LCQ_EINVAL;
  if (dtype != LCQ_F32 && dtype != LCQ_BF16 && dtype != LCQ_F16) return LCQ_EDTYPE;
  const int n = dtype == LCQ_F32 ? 4 : 8;
  hipStream_t st = (hipStream_t)stream;
  if (group_size % n != 0 || (((uintptr_t)w | (uintptr_t)out) % 16) != 0) {
    int64_t grid = (R * K + 255) / 256;
    if (grid > 262144) grid = 262144;
    if (dtype == LCQ_BF16) clamp_groups_scalar_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>(w, R * K, group_size, lo, hi, out);
    else if (dtype == LCQ_F16) clamp_groups_scalar_kernel<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(w, R * K, group_size, lo, hi, out);
    else clamp_groups_scalar_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>(w, R * K, group_size, lo, hi, out);
    LCQ_CHECK_LAUNCH();
    return LCQ_OK;
  }
  const int64_t nchunks = R * K / n;
  int64_t grid = (nchunks + 255) / 256;
  if (grid > 262144) grid = 262144;
  if (dtype == LCQ_BF16) clamp_groups_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)w, nchunks, group_size / n, lo, hi, (u32x4*)out);
  else if (dtype == LCQ_F16) clamp_groups_kernel<ROW_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)w, nchunks, group_size / n, lo, hi, (u32x4*)out);
  else clamp_groups_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, st>>>((const u32x4*)w, nchunks, group_size / n, lo, hi, (u32x4*)out);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
