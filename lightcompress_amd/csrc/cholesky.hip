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
#include <mutex>
#include "gemm_f32.h"
#include "lcq_internal.h"

namespace lcq {
std::atomic<int> g_gemm_split{1};
}

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
    sc->damp = percdamp * (t * (1.0f / (float)K));     // torch.mean on the GPU: the sum times an fp32 factor
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
// takes 4 rows; without a permutation reads and writes are both coalesced.
template <int DT>
__device__ __forceinline__ float load_w(const void* w, long long i) {
  if (DT == LCQ_F32) return ((const float*)w)[i];
  if (DT == LCQ_BF16) return u2f((uint32_t)((const uint16_t*)w)[i] << 16);
  return (float)((const _Float16*)w)[i];
}
template <int DT>
__global__ __launch_bounds__(256) void prepare_w_kernel(const void* __restrict__ w, long long R, int K,
                                                        const long long* __restrict__ perm,
                                                        const uint8_t* __restrict__ dead, float* __restrict__ out) {
  for (long long row = (long long)blockIdx.x * 4; row < R && row < (long long)blockIdx.x * 4 + 4; ++row) {
    for (int j = threadIdx.x; j < K; j += 256) {
      const long long c = perm ? perm[j] : j;
      float v = load_w<DT>(w, row * K + c);
      if (dead && dead[c]) v = 0.0f;
      out[row * K + j] = v;
    }
  }
}
// The same with a permutation: a gather inside every row.  From memory that is one 64-byte sector per element; here
// the workgroup's rows (`rows` of them, as many as fit 64 KB) come in as they lie, 16 bytes per lane, and the gather
// reads LDS.  The permutation is read once per workgroup and column.
template <int DT>
__global__ __launch_bounds__(256) void prepare_w_gather_kernel(const void* __restrict__ w, long long R, int K, int rows,
                                                               const long long* __restrict__ perm,
                                                               const uint8_t* __restrict__ dead, float* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char staged[];
  constexpr int ES = DT == LCQ_F32 ? 4 : 2;
  const long long row0 = (long long)blockIdx.x * rows;
  const int n = (int)((R - row0 < rows) ? (R - row0) : rows);
  const long long nbytes = (long long)n * K * ES;
  const unsigned char* src = (const unsigned char*)w + row0 * K * ES;
  if ((((uintptr_t)src) & 15) == 0) {
    const long long n16 = nbytes >> 4;
    for (long long i = threadIdx.x; i < n16; i += 256) ((u32x4*)staged)[i] = ((const u32x4*)src)[i];
    for (long long i = (n16 << 4) + threadIdx.x; i < nbytes; i += 256) staged[i] = src[i];
  } else {
    for (long long i = threadIdx.x; i < nbytes; i += 256) staged[i] = src[i];
  }
  __syncthreads();
  for (int j = threadIdx.x; j < K; j += 256) {
    const long long c = perm[j];
    const bool dz = dead && dead[c];
    for (int r = 0; r < n; ++r) {
      const float v = load_w<DT>(staged, (long long)r * K + c);
      out[(row0 + r) * K + j] = dz ? 0.0f : v;
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

// The same from a fully symmetric H and with a permutation: row a of A draws on row perm[K-1-a] of H only, which
// comes in as it lies (16 bytes per lane) and is gathered from LDS.  (Picking H[min][max] from memory, as build_kernel
// does, walks down a column of H for half of the entries: one 64-byte sector per element.)
__global__ __launch_bounds__(256) void build_gather_kernel(const float* __restrict__ H, int K, const long long* __restrict__ perm,
                                                           const PrepScalars* __restrict__ sc, float* __restrict__ A) {
  extern __shared__ __align__(16) float hrow[];
  const int a = blockIdx.x;
  const float* src = H + perm[K - 1 - a] * (long long)K;
  if ((((uintptr_t)src) & 15) == 0 && (K & 3) == 0) {
    for (int i = threadIdx.x; i < (K >> 2); i += 256) ((f32x4*)hrow)[i] = ((const f32x4*)src)[i];
  } else {
    for (int i = threadIdx.x; i < K; i += 256) hrow[i] = src[i];
  }
  __syncthreads();
  const float damp = sc->damp;
  for (int b = threadIdx.x; b < K; b += 256) {
    float v = 0.0f;
    if (b <= a) {
      v = hrow[perm[K - 1 - b]];
      if (a == b) v += damp;
    }
    A[(long long)a * K + b] = v;
  }
}

// Diagonal block: Cholesky factor L11 of a 128x128 block and its inverse, one workgroup of 8 waves.
// A wave that is alone on its SIMD issues about one instruction per 8 cycles, and a column-by-column sweep with a
// barrier per column executes ~150 instructions per column in every wave: 70 us per block, none of it arithmetic.
// Here the 128 columns are 8 panels of 16, and the serial part of a panel runs in ONE wave without barriers:
//   * waves 0-3 ("update waves") hold the lower triangle in registers, 8x8 per thread, dealt out cyclically (thread
//     (ty, tx) owns rows ty + 16 ii and columns tx + 16 cc);
//   * wave 4 (the "panel wave") takes the current 16-column panel from LDS with one or two rows per lane and factors
//     it in registers: pivot and multipliers travel by v_readlane, 3 instructions per (column, later column) pair;
//     it leaves the scaled panel in LDS;
//   * the update waves apply a finished panel first to the next panel's columns, hand those to the panel wave, and
//     apply it to the rest of their registers while the panel wave is already factoring (a right-looking update
//     with look-ahead); two barriers per panel;
//   * wave 5 inverts the 16x16 diagonal block of the previous panel meanwhile (forward substitution in registers);
//   * afterwards all 8 waves merge the inverted diagonal blocks pairwise, 16 -> 32 -> 64 -> 128,
//     [[A,0],[B,C]]^-1 = [[A^-1,0],[-C^-1 B A^-1, C^-1]], from LDS.
// Row (column) r of the block lives at float `lds_slot(r)` of an LDS row.  Thread t of the 16 x 16 update grid owns rows
// t + 16 ii, ii < 8: the first four sit at 4 t .. 4 t + 3 and the other four at 64 + 4 t .., so both 16-byte pieces of
// a thread are contiguous with its neighbours' (no bank conflicts for 16-byte accesses), and 16 consecutive rows are 16
// bytes apart (none for the 4-byte accesses of the panel wave and of the matrix-pipe operand reads either).
constexpr int lds_slot(int r) { return ((r >> 4) < 4) ? 4 * (r & 15) + (r >> 4) : 64 + 4 * (r & 15) + (r >> 4) - 4; }
constexpr int LP = NB + 4;       // row pitch of the LDS matrices (16-byte aligned rows, 4-bank skew)

struct PotrfLds {
  float L[8][16][LP];    // L[P][k][lds_slot(r)] = L(r, 16 P + k); zero above the diagonal inside the panel's own 16 rows
  float X[NB][LP];       // L^-1, row-major
  float Pn[16][LP];      // the panel on its way to the panel wave, same layout as L[P], unscaled (padded rows: the 16
                         // rows a publishing wave writes at once fall into different banks)
  float T[64 * 64];      // products of the inverse merges
};

__device__ __forceinline__ float rdlane(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}

// panel P: columns 16 P .. +15, rows 16 P .. 127; lane l owns row 16 P + l and (TWO) row 16 P + 64 + l
template <bool TWO>
__device__ __forceinline__ void potrf_panel(PotrfLds& s, int P, int lane, bool& bad) {
  #pragma clang fp contract(fast)   // a -= l*l as one FMA; nothing here needs op-by-op rounding
  const int c0 = 16 * P;
  const int rA = c0 + lane, rB = c0 + 64 + lane;
  const bool okA = rA < NB, okB = TWO && rB < NB;
  const int sA = lds_slot(okA ? rA : 0), sB = lds_slot(okB ? rB : 0);
  float a0[16], a1[16];
  #pragma unroll
  for (int k = 0; k < 16; ++k) {
    a0[k] = okA ? s.Pn[k][sA] : 0.0f;
    a1[k] = okB ? s.Pn[k][sB] : 0.0f;
  }
  #pragma unroll
  for (int j = 0; j < 16; ++j) {
    const float piv = rdlane(a0[j], j);
    bad = bad || !(piv > 0.0f);
    float rinv = __builtin_amdgcn_rsqf(piv);          // 1/sqrt(pivot), one Newton step to full precision
    rinv = rinv * (1.5f - 0.5f * piv * rinv * rinv);
    a0[j] *= rinv;                                    // the diagonal entry becomes sqrt(pivot); rows above it hold zeros
    if (TWO) a1[j] *= rinv;
    #pragma unroll
    for (int c = j + 1; c < 16; ++c) {
      const float m = rdlane(a0[j], c);               // L(16 P + c, 16 P + j)
      a0[c] -= a0[j] * m;                             // (entries above the diagonal pick up garbage; never read, masked below)
      if (TWO) a1[c] -= a1[j] * m;
    }
  }
  #pragma unroll
  for (int k = 0; k < 16; ++k) {
    if (okA) s.L[P][k][sA] = (lane >= k) ? a0[k] : 0.0f;
    if (okB) s.L[P][k][sB] = a1[k];
  }
}

// X_QQ = L_QQ^-1 for the 16x16 diagonal block Q: lane c (mod 16) carries column c of the inverse
__device__ __forceinline__ void potrf_diag_inv(PotrfLds& s, int Q, int lane) {
  #pragma clang fp contract(fast)
  const int c0 = 16 * Q, l16 = lane & 15;
  const int sl = lds_slot(c0 + l16);
  float t[16], x[16];
  #pragma unroll
  for (int k = 0; k < 16; ++k) t[k] = s.L[Q][k][sl];          // lane j: row j of the block
  #pragma unroll
  for (int j = 0; j < 16; ++j) {
    float acc = (l16 == j) ? 1.0f : 0.0f;
    #pragma unroll
    for (int k = 0; k < j; ++k) acc -= rdlane(t[k], j) * x[k];
    const float d = rdlane(t[j], j);
    float r = __builtin_amdgcn_rcpf(d);
    r = r * (2.0f - d * r);
    x[j] = acc * r;
  }
  if (lane < 16) {
    #pragma unroll
    for (int j = 0; j < 16; ++j) s.X[c0 + j][c0 + lane] = (lane <= j) ? x[j] : 0.0f;
  }
}

// a[ii][cc] -= sum_k L(row, 16 PL + k) L(col, 16 PL + k) for the register columns CC_LO .. 7 (rows ii >= cc), or for
// the single column CC_LO (ONE).  Compile-time ranges: a run-time range costs a branch per register column and
// panel column, and a wave here pays ~10 cycles for every instruction it issues.
template <int PL, int CC_LO, bool ONE>
__device__ __forceinline__ void potrf_update(const PotrfLds& s, float (&a)[8][8], int ty, int tx) {
  #pragma clang fp contract(fast)
  if constexpr (CC_LO < 8) {
    #pragma unroll 2
    for (int k = 0; k < 16; ++k) {
      const f32x4 r0 = *(const f32x4*)(s.L[PL][k] + 4 * ty), r1 = *(const f32x4*)(s.L[PL][k] + 64 + 4 * ty);
      const float lr[8] = {r0[0], r0[1], r0[2], r0[3], r1[0], r1[1], r1[2], r1[3]};
      if constexpr (ONE) {
        const float lc = s.L[PL][k][(CC_LO < 4 ? 4 * tx + CC_LO : 64 + 4 * tx + CC_LO - 4)];
        #pragma unroll
        for (int ii = CC_LO; ii < 8; ++ii) a[ii][CC_LO] -= lr[ii] * lc;
      } else {
        const f32x4 c0 = *(const f32x4*)(s.L[PL][k] + 4 * tx), c1 = *(const f32x4*)(s.L[PL][k] + 64 + 4 * tx);
        const float lc[8] = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
        #pragma unroll
        for (int cc = CC_LO; cc < 8; ++cc)
          #pragma unroll
          for (int ii = cc; ii < 8; ++ii) a[ii][cc] -= lr[ii] * lc[cc];
      }
    }
  }
}

// register column PC (columns tx + 16 PC) -> Pn, zero above the diagonal
template <int PC>
__device__ __forceinline__ void potrf_publish(PotrfLds& s, const float (&a)[8][8], int ty, int tx) {
  float v[8];
  #pragma unroll
  for (int ii = 0; ii < 8; ++ii) v[ii] = (ty + 16 * ii >= tx + 16 * PC) ? a[ii][PC] : 0.0f;
  *(f32x4*)(s.Pn[tx] + 4 * ty) = f32x4{v[0], v[1], v[2], v[3]};
  *(f32x4*)(s.Pn[tx] + 64 + 4 * ty) = f32x4{v[4], v[5], v[6], v[7]};
}

// panel P of the sweep, all 8 waves
template <int P>
__device__ __forceinline__ void potrf_phase(PotrfLds& s, float (&a)[8][8], int wave, int lane, bool upd, int ty, int tx, bool& bad) {
  __syncthreads();                                   // Pn holds panel P; L[P - 1] is complete
  if (wave == 4) {
    potrf_panel<(16 * P + 64 < NB)>(s, P, lane, bad);
  } else if (wave == 5) {
    if constexpr (P > 0) potrf_diag_inv(s, P - 1, lane);
  } else if (upd) {
    if constexpr (P > 0) potrf_update<P - 1, P + 1, false>(s, a, ty, tx);     // panel P - 1 on everything behind panel P
  }
  __syncthreads();                                   // L[P] is complete
  if constexpr (P < 7) {
    if (upd) {
      potrf_update<P, P + 1, true>(s, a, ty, tx);      // panel P on the next panel's columns, handed over at once
      potrf_publish<P + 1>(s, a, ty, tx);
    }
  }
}

// One level of the inverse: the blocks of size S on the diagonal of X are inverted already, the block below each even
// one follows as X21 = -X22 (L21 X11), two products on the fp32 matrix pipe with operands straight from LDS.
// v_mfma_f32_32x32x2f32: lane l supplies A(row l % 32, k = l / 32) and B(k = l / 32, column l % 32); accumulator
// register r holds row 8 (r / 4) + 4 (l / 32) + r % 4 of column l % 32.  v_mfma_f32_16x16x4f32: A(row l % 16,
// k = l / 16), B(k = l / 16, column l % 16), register r holds row 4 (l / 16) + r of column l % 16.
// One wave per 32x32 (16x16) output tile; both triangular operands are cut at tile granularity and read zeros above
// their diagonals (X is cleared at the start).
typedef __attribute__((ext_vector_type(16))) float potrf_f32x16;

template <int S>
__device__ __forceinline__ void potrf_merge(PotrfLds& s, int wave, int lane) {
  if constexpr (S >= 32) {
    constexpr int TS = S / 32, TPP = TS * TS, NT = (NB / (2 * S)) * TPP;
    const int p = wave / TPP, t = wave % TPP, ti = t / TS, tj = t % TS;
    const int o = 2 * S * p, lm = lane & 31, lk = lane >> 5;
    const bool on = wave < NT;
    if (on) {
      potrf_f32x16 acc;
      #pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
      const int rs = lds_slot(o + S + 32 * ti + lm);
      for (int k = 32 * tj; k < S; k += 2) {             // X11(k, j) = 0 for k < j
        const int kk = o + k + lk;
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(s.L[kk >> 4][kk & 15][rs], s.X[kk][o + 32 * tj + lm], acc, 0, 0, 0);
      }
      #pragma unroll
      for (int r = 0; r < 16; ++r)
        s.T[(p * S + 32 * ti + 8 * (r >> 2) + 4 * lk + (r & 3)) * S + 32 * tj + lm] = acc[r];
    }
    __syncthreads();
    if (on) {
      potrf_f32x16 acc;
      #pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
      for (int k = 0; k < 32 * (ti + 1); k += 2) {       // X22(i, k) = 0 for k > i
        const int kk = k + lk;
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(s.X[o + S + 32 * ti + lm][o + S + kk], s.T[(p * S + kk) * S + 32 * tj + lm],
                                                   acc, 0, 0, 0);
      }
      #pragma unroll
      for (int r = 0; r < 16; ++r)
        s.X[o + S + 32 * ti + 8 * (r >> 2) + 4 * lk + (r & 3)][o + 32 * tj + lm] = -acc[r];
    }
    __syncthreads();
  } else {
    static_assert(S == 16, "block sizes 16, 32, 64");
    const int p = wave, o = 32 * p, lm = lane & 15, lk = lane >> 4;
    const bool on = wave < NB / 32;
    if (on) {
      f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
      const int rs = lds_slot(o + 16 + lm);
      #pragma unroll
      for (int k = 0; k < 16; k += 4) {
        const int kk = o + k + lk;
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(s.L[kk >> 4][kk & 15][rs], s.X[kk][o + lm], acc, 0, 0, 0);
      }
      #pragma unroll
      for (int r = 0; r < 4; ++r) s.T[(p * 16 + 4 * lk + r) * 16 + lm] = acc[r];
    }
    __syncthreads();
    if (on) {
      f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
      #pragma unroll
      for (int k = 0; k < 16; k += 4) {
        const int kk = k + lk;
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(s.X[o + 16 + lm][o + 16 + kk], s.T[(p * 16 + kk) * 16 + lm], acc, 0, 0, 0);
      }
      #pragma unroll
      for (int r = 0; r < 4; ++r) s.X[o + 16 + 4 * lk + r][o + lm] = -acc[r];
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(512) void potrf_diag_kernel(float* __restrict__ Ablk, int lda, int nb,
                                                         float* __restrict__ Dinv, PrepScalars* sc) {
  __shared__ __align__(16) PotrfLds s;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ty = (tid >> 4) & 15, tx = tid & 15;
  const bool upd = tid < 256;
  for (int e = tid; e < NB * LP / 4; e += 512) ((f32x4*)&s.X[0][0])[e] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  float a[8][8];
  if (upd) {
    #pragma unroll
    for (int ii = 0; ii < 8; ++ii)
      #pragma unroll
      for (int cc = 0; cc < 8; ++cc) {
        const int r = ty + 16 * ii, c = tx + 16 * cc;
        a[ii][cc] = (r < nb && c <= r) ? Ablk[(long long)r * lda + c] : ((r == c) ? 1.0f : 0.0f);   // pad with identity
      }
    potrf_publish<0>(s, a, ty, tx);
  }
  bool bad = false;
  potrf_phase<0>(s, a, wave, lane, upd, ty, tx, bad);
  potrf_phase<1>(s, a, wave, lane, upd, ty, tx, bad);
  potrf_phase<2>(s, a, wave, lane, upd, ty, tx, bad);
  potrf_phase<3>(s, a, wave, lane, upd, ty, tx, bad);
  potrf_phase<4>(s, a, wave, lane, upd, ty, tx, bad);
  potrf_phase<5>(s, a, wave, lane, upd, ty, tx, bad);
  potrf_phase<6>(s, a, wave, lane, upd, ty, tx, bad);
  potrf_phase<7>(s, a, wave, lane, upd, ty, tx, bad);
  __syncthreads();
  if (wave == 5) potrf_diag_inv(s, 7, lane);
  if (wave == 4 && bad && lane == 0) sc->status = 1;
  __syncthreads();
  potrf_merge<16>(s, wave, lane);
  potrf_merge<32>(s, wave, lane);
  potrf_merge<64>(s, wave, lane);
  for (int v = tid; v < NB * NB / 4; v += 512) {            // L^-1, row-major, zeros above the diagonal and in the padding
    const int r = v >> 5, c4 = (v & 31) * 4;
    f32x4 x = *(const f32x4*)(&s.X[r][c4]);
    #pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = (r < nb && c4 + e <= r) ? x[e] : 0.0f;
    *(f32x4*)(Dinv + r * NB + c4) = x;
  }
  // (L itself is not written back: everything after this kernel works with the inverse, the solved panels and the
  // blocks behind them; place_diag_kernel puts the inverse where the block was.)
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

int lcq_set_gemm_split(int on) {
  return g_gemm_split.exchange(on ? 1 : 0);
}

int lcq_gptq_prepare_weights(const void* w, int dtype, int64_t R, int64_t K, const int64_t* perm, const uint8_t* dead,
                             float* out, void* stream) {
  if (!w || !out || R <= 0 || K <= 0 || K > 0x7fffffff || (const void*)out == w) return LCQ_EINVAL;
  const int64_t grid = (R + 3) / 4;
  if (grid > 0x7fffffff) return LCQ_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  const long long* p = (const long long*)perm;
  const int es = dtype == LCQ_F32 ? 4 : 2;
  if (p && K * es <= 65536 && (dtype == LCQ_F32 || dtype == LCQ_BF16 || dtype == LCQ_F16)) {   // gather through LDS
    int rows = (int)(65536 / (K * es));
    if (rows > 8) rows = 8;
    const int64_t g = (R + rows - 1) / rows;
    if (g > 0x7fffffff) return LCQ_EINVAL;
    const size_t lds = (size_t)rows * K * es;
    if (dtype == LCQ_F32) prepare_w_gather_kernel<LCQ_F32><<<dim3((unsigned)g), dim3(256), lds, st>>>(w, R, (int)K, rows, p, dead, out);
    else if (dtype == LCQ_BF16) prepare_w_gather_kernel<LCQ_BF16><<<dim3((unsigned)g), dim3(256), lds, st>>>(w, R, (int)K, rows, p, dead, out);
    else prepare_w_gather_kernel<LCQ_F16><<<dim3((unsigned)g), dim3(256), lds, st>>>(w, R, (int)K, rows, p, dead, out);
  }
  else if (dtype == LCQ_F32) prepare_w_kernel<LCQ_F32><<<dim3((unsigned)grid), dim3(256), 0, st>>>(w, R, (int)K, p, dead, out);
  else if (dtype == LCQ_BF16) prepare_w_kernel<LCQ_BF16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(w, R, (int)K, p, dead, out);
  else if (dtype == LCQ_F16) prepare_w_kernel<LCQ_F16><<<dim3((unsigned)grid), dim3(256), 0, st>>>(w, R, (int)K, p, dead, out);
  else return LCQ_EDTYPE;
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

// A second stream per (device, caller's stream) for the deep trailing updates of long chains, with the two events that
// order it against the caller's stream.  Created on first use, kept until the process ends.
struct SideLane { int dev; hipStream_t caller; hipStream_t side; hipEvent_t fork, join; };
static SideLane g_lanes[16];
static int g_nlanes = 0;
static std::mutex g_lane_mu;
static std::atomic<int> g_lookahead{1};
static SideLane* side_lane(hipStream_t st) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(g_lane_mu);
  for (int i = 0; i < g_nlanes; ++i)
    if (g_lanes[i].dev == dev && g_lanes[i].caller == st) return &g_lanes[i];
  if (g_nlanes == 16) return nullptr;
  SideLane l{dev, st, nullptr, nullptr, nullptr};
  if (hipStreamCreateWithFlags(&l.side, hipStreamNonBlocking) != hipSuccess) return nullptr;       // default priority
  if (hipEventCreateWithFlags(&l.fork, hipEventDisableTiming) != hipSuccess ||
      hipEventCreateWithFlags(&l.join, hipEventDisableTiming) != hipSuccess) return nullptr;
  g_lanes[g_nlanes] = l;
  return &g_lanes[g_nlanes++];
}

// The chain behind lcq_chol_inv_upper (blocks_only = false) and lcq_chol_block_factor (true).
static int chol_chain(float* H, int64_t K64, const int64_t* perm, float percdamp, float* W, int64_t R, float* U,
                      void* workspace, int64_t workspace_bytes, int* status, void* stream, bool blocks_only) {
  if (!H || !U || !workspace || K64 <= 0 || K64 > 65536 || R < 0) return LCQ_EINVAL;
  if (blocks_only && K64 % NB != 0) return LCQ_EINVAL;     // the blocks of the reversed matrix must be the loop's blocks
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
  if (perm && K <= 16384) {                       // a row of H fits the 64 KB of LDS a workgroup may ask for
    if (lcq_symmetrize(H, K, stream) != LCQ_OK) return LCQ_ELAUNCH;
    build_gather_kernel<<<dim3((unsigned)K), dim3(256), (size_t)K * 4, st>>>(H, K, (const long long*)perm, sc, A);
  } else {
    build_kernel<<<dim3((unsigned)((K + 255) / 256), (unsigned)K), dim3(256), 0, st>>>(H, K, (const long long*)perm, sc, A);
  }

  // Blocked right-looking Cholesky with two block sizes: 128-column panels are factored one by
  // one, but their trailing update is applied only inside the current 512-column super-panel;
  // the rest of the matrix is updated once per super-panel with a 512-deep contraction, which
  // cuts the read-modify-write traffic on the trailing matrix fourfold.
  constexpr int NBO = 4 * NB;
  // Long chains: the deep update behind a super-panel is split into the columns of the NEXT super-panel (on the
  // caller's stream, the panels that follow need it) and everything behind those (on the side stream, beside those
  // panels: a few narrow launches that leave the chip to it).  The next deep update touches that region again and
  // waits for it.
  SideLane* lane = (g_lookahead.load() && K >= 8192) ? side_lane(st) : nullptr;
  bool pending = false;
  for (int o0 = 0; o0 < K; o0 += NBO) {
    const int o1 = (o0 + NBO < K) ? (o0 + NBO) : K;
    for (int k0 = o0; k0 < o1; k0 += NB) {
      const int b = k0 / NB, nb = (K - k0 < NB) ? (K - k0) : NB;
      float* Akk = A + (long long)k0 * K + k0;
      float* Db = Dinv + (long long)b * NB * NB;
      potrf_diag_kernel<<<dim3(1), dim3(512), 0, st>>>(Akk, K, nb, Db, sc);
      const int k1 = k0 + nb, M = K - k1;
      if (M > 0) {
        float* A21 = A + (long long)k1 * K + k0;
        launch_gemm<true>(GemmProblem{A21, Db, A21, M, nb, nb, K, NB, K}, 1.0f, 0.0f, 0, st);       // A21 L11^-T
        if (o1 > k1)                                                                              // inside the super-panel
          launch_gemm<true>(GemmProblem{A21, A21, A + (long long)k1 * K + k1, M, o1 - k1, nb, K, K, K}, -1.0f, 1.0f,
                            GEMM_LOWER_TILES, st);
      }
    }
    if (o1 < K && lane) {
      const int o2 = (o1 + NBO < K) ? (o1 + NBO) : K;
      const float* P = A + (long long)o1 * K + o0;
      if (pending && hipStreamWaitEvent(st, lane->join, 0) != hipSuccess) return LCQ_ELAUNCH;
      pending = false;
      if (hipEventRecord(lane->fork, st) != hipSuccess) return LCQ_ELAUNCH;           // the panels of this super-panel
      launch_gemm<true>(GemmProblem{P, P, A + (long long)o1 * K + o1, K - o1, o2 - o1, o1 - o0, K, K, K}, -1.0f, 1.0f,
                        GEMM_LOWER_TILES, st);
      if (o2 < K) {
        const float* P2 = A + (long long)o2 * K + o0;
        if (hipStreamWaitEvent(lane->side, lane->fork, 0) != hipSuccess) return LCQ_ELAUNCH;
        launch_gemm<true>(GemmProblem{P2, P2, A + (long long)o2 * K + o2, K - o2, K - o2, o1 - o0, K, K, K}, -1.0f, 1.0f,
                          GEMM_LOWER_TILES, lane->side);
        if (hipEventRecord(lane->join, lane->side) != hipSuccess) return LCQ_ELAUNCH;
        pending = true;
      }
    } else if (o1 < K) {                                                                          // everything behind it
      const float* P = A + (long long)o1 * K + o0;
      launch_gemm<true>(GemmProblem{P, P, A + (long long)o1 * K + o1, K - o1, K - o1, o1 - o0, K, K, K}, -1.0f, 1.0f,
                        GEMM_LOWER_TILES, st);
    }
  }
  if (pending && hipStreamWaitEvent(st, lane->join, 0) != hipSuccess) return LCQ_ELAUNCH;

  if (blocks_only) {
    // No triangular inverse.  With M = J L J (H_d = M M^T, M upper triangular; J reverses the order) the inverse
    // factor is U = M^-1, and the column loop needs of it only (a) the diagonal blocks U_bb = (M_bb)^-1, which drive
    // the recurrence inside a block, and (b) something that carries a block's effect to the columns behind it.  From
    // E U = W - Q (E the loop's errors, Q the quantized weights, W the weights before the loop) follows
    //   W[:, b] as the loop finds it at block b  =  W0[:, b] + sum_{p<b} (W0 - Q)[:, p] M[p, b] U_bb,
    // so with P[p, b] = M[p, b] U_bb above the diagonal blocks and P[b, b] = U_bb the loop runs unchanged on P if a
    // block hands (Q - W0) instead of its errors to the deferred update.  In the reversed order that is every
    // sub-diagonal panel of L times the inverse of its diagonal block, which the factorization has already: one
    // batched product instead of the log2(K/128) merge levels of the inverse (K^3/3 flop).
    for (int b0 = 0; b0 + 1 < nblk; b0 += GEMM_MAX_BATCH) {
      const int np = (nblk - 1 - b0 < GEMM_MAX_BATCH) ? (nblk - 1 - b0) : GEMM_MAX_BATCH;
      GemmBatch bt;
      int maxM = 0;
      for (int q = 0; q < np; ++q) {
        const int b = b0 + q, k0 = b * NB, k1 = k0 + NB;
        bt.offA[q] = (long long)k1 * K + k0; bt.offB[q] = (long long)b * NB * NB; bt.offC[q] = bt.offA[q];
        bt.M[q] = K - k1; bt.N[q] = NB; bt.Kc[q] = NB;
        if (K - k1 > maxM) maxM = K - k1;
      }
      const dim3 grid(1, (unsigned)((maxM + GT - 1) / GT), (unsigned)np);
      gemm_f32_batched_kernel<false><<<grid, dim3(256), 0, st>>>(A, K, Dinv, NB, A, K, bt, 1.0f, 0.0f, 0);
    }
    place_diag_kernel<<<dim3((unsigned)nblk), dim3(256), 0, st>>>(A, K, Dinv);
    scatter_kernel<<<dim3((unsigned)((K + 255) / 256), (unsigned)K), dim3(256), 0, st>>>(A, K, U);
    if (status)
      (void)hipMemcpyAsync(status, &sc->status, sizeof(int), hipMemcpyDeviceToDevice, st);
    LCQ_CHECK_LAUNCH();
    return LCQ_OK;
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
      if (g_gemm_split.load() && ((long long)grid.x * grid.y * grid.z > 256 || maxN >= 256)) {      // long contractions
        gemm_s3_batched_kernel<false><<<grid, dim3(256), 0, st>>>(A, K, A, K, T, K, b1, 1.0f, 0.0f, GEMM_K_FROM_N);
        gemm_s3_batched_kernel<false><<<grid, dim3(256), 0, st>>>(A, K, T, K, A, K, b2, -1.0f, 0.0f, GEMM_K_TO_M);
      } else {
        gemm_f32_batched_kernel<false><<<grid, dim3(256), 0, st>>>(A, K, A, K, T, K, b1, 1.0f, 0.0f, GEMM_K_FROM_N);
        gemm_f32_batched_kernel<false><<<grid, dim3(256), 0, st>>>(A, K, T, K, A, K, b2, -1.0f, 0.0f, GEMM_K_TO_M);
      }
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

int lcq_set_chain_lookahead(int on) {
  return g_lookahead.exchange(on ? 1 : 0);
}

int lcq_chol_inv_upper(float* H, int64_t K, const int64_t* perm, float percdamp, float* W, int64_t R, float* U,
                       void* workspace, int64_t workspace_bytes, int* status, void* stream) {
  return chol_chain(H, K, perm, percdamp, W, R, U, workspace, workspace_bytes, status, stream, false);
}

int lcq_chol_block_factor(float* H, int64_t K, const int64_t* perm, float percdamp, float* W, int64_t R, float* P,
                          void* workspace, int64_t workspace_bytes, int* status, void* stream) {
  return chol_chain(H, K, perm, percdamp, W, R, P, workspace, workspace_bytes, status, stream, true);
}

}  // extern "C"
