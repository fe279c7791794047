// Damped Cholesky chain of GPTQ for gfx950.
//
// Replaces, in GPTQ.process_hessian_and_weights (gptq.py:139-141, 150-153, 169-174):
//   dead = diag(H) == 0; H[dead, dead] = 1; W[:, dead] = 0
//   H = H[perm][:, perm]
//   H += percdamp * mean(diag(H)) * I
//   H = cholesky(H); H = cholesky_inverse(H); H = cholesky(H, upper=True)
// The result U is upper triangular with U^T U = (H + damp I)^-1.
//
// Instead of three factorizations (4/3 K^3 flop) the chain is computed as
//   J H J = L L^T  (J = index reversal, L lower)   ->   U = J L^-1 J,
// one Cholesky plus one triangular inverse (2/3 K^3 flop): L^-1 lower with a
// positive diagonal, reversed on both axes, is upper triangular and
// (J L^-1 J)^T (J L^-1 J) = J (L L^T)^-1 J = H^-1, so it IS the unique upper
// Cholesky factor of H^-1.
//
// Kernels
//   diag_prep      diagonal scan: dead columns, mean(diag) -> damp
//   build          gather  A[a][b] = H[p(K-1-a)][p(K-1-b)] (+damp on the diagonal), a >= b
//   potrf_diag     128x128 diagonal block in LDS: L11 and L11^-1 (one workgroup)
//   gemm_f32       fp32 MFMA: panel solve  A21 <- A21 L11^-T  and trailing  A22 -= A21 A21^T
//   (batched)      triangular inverse by pairwise merging of inverted diagonal
//                  blocks: [[A,0],[B,C]]^-1 = [[A^-1,0],[-C^-1 B A^-1, C^-1]]
//   scatter        U[i][j] = Linv[K-1-i][K-1-j], j >= i; zeros below the diagonal
#include "gemm_f32.h"
#include "lcq_internal.h"

namespace {
using namespace lcq;

constexpr int NB = 128;

struct PrepScalars {
  float damp;
  int status;      // 0 ok, 1 non-positive pivot met
};

// one workgroup: dead-column fix on the diagonal, damp = percdamp * mean(diag)
__global__ __launch_bounds__(1024) void diag_prep_kernel(float* __restrict__ H, int K, float percdamp,
                                                         uint8_t* __restrict__ dead, PrepScalars* sc) {
  __shared__ float part[16];
  float s = 0.0f;
  for (int j = threadIdx.x; j < K; j += 1024) {
    float d = H[(long long)j * K + j];
    const bool is_dead = (d == 0.0f);
    if (is_dead) { d = 1.0f; H[(long long)j * K + j] = 1.0f; }
    dead[j] = is_dead;
    s += d;
  }
  s = team_sum<64>(s);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.0f;
    for (int i = 0; i < 16; ++i) t += part[i];
    sc->damp = percdamp * (t / (float)K);
    sc->status = 0;
  }
}

// W[:, dead] = 0
__global__ __launch_bounds__(256) void apply_dead_kernel(float* __restrict__ W, long long R, int K,
                                                         const uint8_t* __restrict__ dead) {
  const long long n = R * K;
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < n; e += (long long)gridDim.x * 256)
    if (dead[e % K]) W[e] = 0.0f;
}

// W[r, j] = dead[c] ? 0 : float(w[r, c]),  c = perm ? perm[j] : j   -- the weight clone, fp32 cast, dead-column
// zeroing and act-order gather of process_hessian_and_weights (gptq.py:133-141, 150-151) in one pass.  A workgroup
// takes 4 rows; reads are gathers inside a row (it stays in cache), writes are coalesced.
template <int DT>
__global__ __launch_bounds__(256) void prepare_w_kernel(const void* __restrict__ w, long long R, int K,
                                                        const long long* __restrict__ perm,
                                                        const uint8_t* __restrict__ dead, float* __restrict__ out) {
  for (long long row = (long long)blockIdx.x * 4; row < R && row < (long long)blockIdx.x * 4 + 4; ++row) {
    for (int j = threadIdx.x; j < K; j += 256) {
      const long long c = perm ? perm[j] : j;
      float v;
      if (DT == LCQ_F32) v = ((const float*)w)[row * K + c];
      else if (DT == LCQ_BF16) v = u2f((uint32_t)((const uint16_t*)w)[row * K + c] << 16);
      else v = (float)((const _Float16*)w)[row * K + c];
      if (dead && dead[c]) v = 0.0f;
      out[row * K + j] = v;
    }
  }
}

// A (lower triangle, reversed + permuted + damped); strict upper triangle zeroed
__global__ __launch_bounds__(256) void build_kernel(const float* __restrict__ H, int K, const long long* __restrict__ perm,
                                                    const PrepScalars* __restrict__ sc, float* __restrict__ A) {
  const int a = blockIdx.y;
  const int b = blockIdx.x * 256 + threadIdx.x;
  if (b >= K) return;
  float v = 0.0f;
  if (b <= a) {
    long long i = K - 1 - a, j = K - 1 - b;
    if (perm) { i = perm[i]; j = perm[j]; }
    const long long lo = i < j ? i : j, hi = i < j ? j : i;     // H is valid on and above the diagonal
    v = H[lo * K + hi];
    if (a == b) v += sc->damp;
  }
  A[(long long)a * K + b] = v;
}

// Diagonal block: Cholesky factor L11 and its inverse in one elimination sweep.
// 256 threads hold the 128x128 block of A and of B (= I, turning into L11^-1) in registers, 8x8 each,
// dealt out cyclically: thread (ty, tx) owns rows ty + 16 ii and columns tx + 16 cc.  The elimination
// front therefore shrinks on every thread alike -- during columns 16P .. 16P+15 ("phase" P) a thread
// updates (8-P)(9-P)/2 elements of A and (8-P)(P+1) of B per step, whichever thread it is -- where a
// blocked layout leaves the last wave with 128 FMAs per step to the end while the first idles.
// Step j:
//   barrier; every thread reads the UNSCALED column j of A, row j of B and the pivot from LDS (double
//   buffered; entries that must not take part are published as zeros, so no update needs a mask),
//   derives 1/sqrt(a_jj) itself and applies
//     a[i][k] -= l_ij l_kj  (i, k > j)      b[i][:] -= l_ij x_j[:]  (i > j)
//   starting with the two register columns of A and rows of B that can hold column / row j+1, which
//   their owners publish at once; the rest of the update then overlaps the next barrier.
// The right-looking Cholesky update and the forward substitution L X = I share the broadcast.
constexpr int lds_slot(int r) { return (r & 15) * 8 + (r >> 4); }   // a thread's 8 rows (columns) are contiguous

template <int P>
__device__ __forceinline__ void potrf_phase(float (&a)[8][8], float (&x)[8][8], float (*colbuf)[NB], float (*rowbuf)[NB],
                                            float* pivbuf, int ty, int tx, bool& bad) {
  #pragma clang fp contract(fast)   // a -= l*l as one FMA; nothing here needs op-by-op rounding
  constexpr int P1 = (P < 7) ? P + 1 : 7;
  #pragma unroll 1
  for (int jl = 0; jl < 16; ++jl) {
    const int j = 16 * P + jl, pb = j & 1;
    __syncthreads();
    const float pv = pivbuf[pb];
    const f32x4 r0 = *(const f32x4*)(colbuf[pb] + 8 * ty), r1 = *(const f32x4*)(colbuf[pb] + 8 * ty + 4);
    const f32x4 c0 = *(const f32x4*)(colbuf[pb] + 8 * tx), c1 = *(const f32x4*)(colbuf[pb] + 8 * tx + 4);
    const f32x4 x0 = *(const f32x4*)(rowbuf[pb] + 8 * tx), x1 = *(const f32x4*)(rowbuf[pb] + 8 * tx + 4);
    bad = bad || !(pv > 0.0f);
    float rinv = __builtin_amdgcn_rsqf(pv);           // 1/sqrt(pivot), one Newton step to full precision
    rinv = rinv * (1.5f - 0.5f * pv * rinv * rinv);
    float lr[8], lc[8], xr[8];
    #pragma unroll
    for (int k = 0; k < 4; ++k) {
      lr[k] = r0[k] * rinv; lr[4 + k] = r1[k] * rinv;
      lc[k] = c0[k] * rinv; lc[4 + k] = c1[k] * rinv;
      xr[k] = x0[k] * rinv; xr[4 + k] = x1[k] * rinv;
    }
    // ---- first: what column j+1 of A and row j+1 of B can depend on ----
    #pragma unroll
    for (int ii = P; ii < 8; ++ii) {
      a[ii][P] -= lr[ii] * lc[P];
      if (P1 != P && P1 <= ii) a[ii][P1] -= lr[ii] * lc[P1];
    }
    #pragma unroll
    for (int cc = 0; cc <= P; ++cc) {
      x[P][cc] -= lr[P] * xr[cc];
      if (P1 != P) x[P1][cc] -= lr[P1] * xr[cc];
    }
    // owners keep the scaled column j of L and row j of X (the published zeros left their own entries alone)
    if (tx == jl) {
      #pragma unroll
      for (int ii = P; ii < 8; ++ii) {
        const int r = ty + 16 * ii;
        if (r > j) a[ii][P] = lr[ii];
        else if (r == j) a[ii][P] = pv * rinv;
      }
    }
    if (ty == jl) {
      #pragma unroll
      for (int cc = 0; cc <= P; ++cc) x[P][cc] = xr[cc];
    }
    // ---- publish column j+1 / row j+1 for the next step ----
    if (j + 1 < NB) {
      const int jn = j + 1, tn = jn & 15;
      const bool nextphase = (jl == 15);
      if (tx == tn) {
        f32x4 v0, v1;
        #pragma unroll
        for (int ii = 0; ii < 8; ++ii) {
          const float v = (ty + 16 * ii > jn) ? (nextphase ? a[ii][P1] : a[ii][P]) : 0.0f;
          if (ii < 4) v0[ii] = v; else v1[ii - 4] = v;
        }
        *(f32x4*)(colbuf[pb ^ 1] + 8 * ty) = v0;
        *(f32x4*)(colbuf[pb ^ 1] + 8 * ty + 4) = v1;
        if (ty == tn) pivbuf[pb ^ 1] = nextphase ? a[P1][P1] : a[P][P];
      }
      if (ty == tn) {
        f32x4 v0, v1;
        #pragma unroll
        for (int cc = 0; cc < 8; ++cc) {
          const float v = (tx + 16 * cc <= jn) ? (nextphase ? x[P1][cc] : x[P][cc]) : 0.0f;
          if (cc < 4) v0[cc] = v; else v1[cc - 4] = v;
        }
        *(f32x4*)(rowbuf[pb ^ 1] + 8 * tx) = v0;
        *(f32x4*)(rowbuf[pb ^ 1] + 8 * tx + 4) = v1;
      }
    }
    // ---- the rest of the update ----
    #pragma unroll
    for (int ii = P + 2; ii < 8; ++ii)
      #pragma unroll
      for (int cc = P + 2; cc <= ii; ++cc) a[ii][cc] -= lr[ii] * lc[cc];
    #pragma unroll
    for (int ii = P + 2; ii < 8; ++ii)
      #pragma unroll
      for (int cc = 0; cc <= P; ++cc) x[ii][cc] -= lr[ii] * xr[cc];
  }
}

__global__ __launch_bounds__(256) void potrf_diag_kernel(float* __restrict__ Ablk, int lda, int nb,
                                                         float* __restrict__ Dinv, PrepScalars* sc) {
  __shared__ __align__(16) float colbuf[2][NB];  // unscaled column j of A strictly below the diagonal, zero elsewhere
  __shared__ __align__(16) float rowbuf[2][NB];  // unscaled row j of B up to the diagonal, zero elsewhere
  __shared__ float pivbuf[2];                    // a_jj
  const int tid = threadIdx.x;
  const int ty = tid >> 4, tx = tid & 15;
  float a[8][8], x[8][8];
  #pragma unroll
  for (int ii = 0; ii < 8; ++ii)
    #pragma unroll
    for (int cc = 0; cc < 8; ++cc) {
      const int r = ty + 16 * ii, c = tx + 16 * cc;
      a[ii][cc] = (r < nb && c <= r) ? Ablk[(long long)r * lda + c] : ((r == c) ? 1.0f : 0.0f);   // pad with identity
      x[ii][cc] = (r == c) ? 1.0f : 0.0f;
    }
  // column 0 / row 0
  if (tx == 0) {
    #pragma unroll
    for (int ii = 0; ii < 8; ++ii) colbuf[0][8 * ty + ii] = (ty + 16 * ii > 0) ? a[ii][0] : 0.0f;
    if (ty == 0) pivbuf[0] = a[0][0];
  }
  if (ty == 0) {
    #pragma unroll
    for (int cc = 0; cc < 8; ++cc) rowbuf[0][8 * tx + cc] = (tx + 16 * cc <= 0) ? x[0][cc] : 0.0f;
  }
  bool bad = false;
  potrf_phase<0>(a, x, colbuf, rowbuf, pivbuf, ty, tx, bad);
  if (nb > 16) potrf_phase<1>(a, x, colbuf, rowbuf, pivbuf, ty, tx, bad);
  if (nb > 32) potrf_phase<2>(a, x, colbuf, rowbuf, pivbuf, ty, tx, bad);
  if (nb > 48) potrf_phase<3>(a, x, colbuf, rowbuf, pivbuf, ty, tx, bad);
  if (nb > 64) potrf_phase<4>(a, x, colbuf, rowbuf, pivbuf, ty, tx, bad);
  if (nb > 80) potrf_phase<5>(a, x, colbuf, rowbuf, pivbuf, ty, tx, bad);
  if (nb > 96) potrf_phase<6>(a, x, colbuf, rowbuf, pivbuf, ty, tx, bad);
  if (nb > 112) potrf_phase<7>(a, x, colbuf, rowbuf, pivbuf, ty, tx, bad);
  if (bad && tid == 0) sc->status = 1;
  #pragma unroll
  for (int ii = 0; ii < 8; ++ii)
    #pragma unroll
    for (int cc = 0; cc < 8; ++cc) {
      const int r = ty + 16 * ii, c = tx + 16 * cc;
      if (r < nb && c < nb) Ablk[(long long)r * lda + c] = (c <= r) ? a[ii][cc] : 0.0f;
      Dinv[r * NB + c] = (r < nb && c <= r && c < nb) ? x[ii][cc] : 0.0f;
    }
}

// copy the inverted diagonal blocks into place
__global__ __launch_bounds__(256) void place_diag_kernel(float* __restrict__ A, int K, const float* __restrict__ Dinv) {
  const int blk = blockIdx.x, k0 = blk * NB;
  const int nb = min(NB, K - k0);
  const float* D = Dinv + (long long)blk * NB * NB;
  for (int e = threadIdx.x; e < NB * NB; e += 256) {
    const int r = e / NB, c = e % NB;
    if (r < nb && c < nb) A[(long long)(k0 + r) * K + k0 + c] = D[e];
  }
}

__global__ __launch_bounds__(256) void scatter_kernel(const float* __restrict__ Linv, int K, float* __restrict__ U) {
  const int i = blockIdx.y;
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= K) return;
  U[(long long)i * K + j] = (j >= i) ? Linv[(long long)(K - 1 - i) * K + (K - 1 - j)] : 0.0f;
}

}  // namespace

extern "C" {

int64_t lcq_chol_inv_upper_workspace_bytes(int64_t K) {
  const int64_t nblk = (K + NB - 1) / NB;
  return K * K * 4 + nblk * NB * NB * 4 + ((K + 255) / 256) * 256 + 256;
}

int lcq_gptq_prepare_weights(const void* w, int dtype, int64_t R, int64_t K, const int64_t* perm, const uint8_t* dead,
                             float* out, void* stream) {
  if (!w || !out || R <= 0 || K <= 0 || K > 0x7fffffff || (const void*)out == w) return LCQ_EINVAL;
  const int64_t grid = (R + 3) / 4;
  if (grid > 0x7fffffff) return LCQ_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  const long long* p = (const long long*)perm;
  if (dtype == LCQ_F32) prepare_w_kernel<LCQ_F32><<<dim3((unsigned)grid), dim3(256), 0, st>>>(w, R, (int)K, p, dead, out);
  else if (dtype == LCQ_BF16) prepare_w_kernel<LCQ_BF16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(w, R, (int)K, p, dead, out);
  else if (dtype == LCQ_F16) prepare_w_kernel<LCQ_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(w, R, (int)K, p, dead, out);
  else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_chol_inv_upper(float* H, int64_t K64, const int64_t* perm, float percdamp, float* W, int64_t R, float* U,
                       void* workspace, int64_t workspace_bytes, int* status, void* stream) {
  if (!H || !U || !workspace || K64 <= 0 || K64 > 65536 || R < 0) return LCQ_EINVAL;
  if (workspace_bytes < lcq_chol_inv_upper_workspace_bytes(K64)) return LCQ_EWORKSPACE;
  if (((uintptr_t)workspace % 16) != 0) return LCQ_EALIGN;
  const int K = (int)K64;
  const int nblk = (K + NB - 1) / NB;
  hipStream_t st = (hipStream_t)stream;
  float* A = (float*)workspace;
  float* Dinv = A + (long long)K * K;
  uint8_t* dead = (uint8_t*)(Dinv + (long long)nblk * NB * NB);
  PrepScalars* sc = (PrepScalars*)(dead + ((K + 255) / 256) * 256);

  diag_prep_kernel<<<dim3(1), dim3(1024), 0, st>>>(H, K, percdamp, dead, sc);
  if (W && R > 0) {
    long long g = ((long long)R * K + 255) / 256;
    if (g > 65536) g = 65536;
    apply_dead_kernel<<<dim3((unsigned)g), dim3(256), 0, st>>>(W, R, K, dead);
  }
  build_kernel<<<dim3((unsigned)((K + 255) / 256), (unsigned)K), dim3(256), 0, st>>>(H, K, (const long long*)perm, sc, A);

  // Blocked right-looking Cholesky with two block sizes: 128-column panels are factored one by
  // one, but their trailing update is applied only inside the current 512-column super-panel;
  // the rest of the matrix is updated once per super-panel with a 512-deep contraction, which
  // cuts the read-modify-write traffic on the trailing matrix fourfold.
  constexpr int NBO = 4 * NB;
  for (int o0 = 0; o0 < K; o0 += NBO) {
    const int o1 = (o0 + NBO < K) ? (o0 + NBO) : K;
    for (int k0 = o0; k0 < o1; k0 += NB) {
      const int b = k0 / NB, nb = (K - k0 < NB) ? (K - k0) : NB;
      float* Akk = A + (long long)k0 * K + k0;
      float* Db = Dinv + (long long)b * NB * NB;
      potrf_diag_kernel<<<dim3(1), dim3(256), 0, st>>>(Akk, K, nb, Db, sc);
      const int k1 = k0 + nb, M = K - k1;
      if (M > 0) {
        float* A21 = A + (long long)k1 * K + k0;
        launch_gemm<true>(GemmProblem{A21, Db, A21, M, nb, nb, K, NB, K}, 1.0f, 0.0f, 0, st);       // A21 L11^-T
        if (o1 > k1)                                                                              // inside the super-panel
          launch_gemm<true>(GemmProblem{A21, A21, A + (long long)k1 * K + k1, M, o1 - k1, nb, K, K, K}, -1.0f, 1.0f,
                            GEMM_LOWER_TILES, st);
      }
    }
    if (o1 < K) {                                                                                 // everything behind it
      const float* P = A + (long long)o1 * K + o0;
      launch_gemm<true>(GemmProblem{P, P, A + (long long)o1 * K + o1, K - o1, K - o1, o1 - o0, K, K, K}, -1.0f, 1.0f,
                        GEMM_LOWER_TILES, st);
    }
  }

  // triangular inverse: inverted diagonal blocks, then pairwise merges
  place_diag_kernel<<<dim3((unsigned)nblk), dim3(256), 0, st>>>(A, K, Dinv);
  int nseg = nblk;
  int seg_start[512], seg_size[512];
  if (nblk > 512) return LCQ_EINVAL;
  for (int b = 0; b < nblk; ++b) { seg_start[b] = b * NB; seg_size[b] = (K - b * NB < NB) ? (K - b * NB) : NB; }
  float* T = U;                                  // scratch until the final scatter
  while (nseg > 1) {
    const int npairs = nseg / 2;
    for (int p0 = 0; p0 < npairs; p0 += GEMM_MAX_BATCH) {
      const int np = (npairs - p0 < GEMM_MAX_BATCH) ? (npairs - p0) : GEMM_MAX_BATCH;
      GemmBatch b1, b2;
      int maxM = 0, maxN = 0;
      for (int q = 0; q < np; ++q) {
        const int sa = seg_start[2 * (p0 + q)], na = seg_size[2 * (p0 + q)];
        const int sc_ = seg_start[2 * (p0 + q) + 1], nc = seg_size[2 * (p0 + q) + 1];
        const long long offBlk = (long long)sc_ * K + sa;          // B block (rows of C-part, cols of A-part)
        // T1 = B * Ainv
        b1.offA[q] = offBlk; b1.offB[q] = (long long)sa * K + sa; b1.offC[q] = offBlk;
        b1.M[q] = nc; b1.N[q] = na; b1.Kc[q] = na;
        // X = -Cinv * T1
        b2.offA[q] = (long long)sc_ * K + sc_; b2.offB[q] = offBlk; b2.offC[q] = offBlk;
        b2.M[q] = nc; b2.N[q] = na; b2.Kc[q] = nc;
        if (nc > maxM) maxM = nc;
        if (na > maxN) maxN = na;
      }
      const dim3 grid((unsigned)((maxN + GT - 1) / GT), (unsigned)((maxM + GT - 1) / GT), (unsigned)np);
      gemm_f32_batched_kernel<false><<<grid, dim3(256), 0, st>>>(A, K, A, K, T, K, b1, 1.0f, 0.0f, GEMM_K_FROM_N);
      gemm_f32_batched_kernel<false><<<grid, dim3(256), 0, st>>>(A, K, T, K, A, K, b2, -1.0f, 0.0f, GEMM_K_TO_M);
    }
    int w = 0;
    for (int p = 0; p < npairs; ++p) {
      seg_start[w] = seg_start[2 * p];
      seg_size[w] = seg_size[2 * p] + seg_size[2 * p + 1];
      ++w;
    }
    if (nseg & 1) { seg_start[w] = seg_start[nseg - 1]; seg_size[w] = seg_size[nseg - 1]; ++w; }
    nseg = w;
  }

  scatter_kernel<<<dim3((unsigned)((K + 255) / 256), (unsigned)K), dim3(256), 0, st>>>(A, K, U);
  if (status)
    (void)hipMemcpyAsync(status, &sc->status, sizeof(int), hipMemcpyDeviceToDevice, st);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
