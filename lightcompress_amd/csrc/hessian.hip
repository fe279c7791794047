// GPTQ Hessian accumulation for gfx950:  H <- alpha*H + beta * X^T X
//
// Replaces GPTQ.add_batch (llmc/compression/quantization/gptq.py:253-295):
//   H *= n/(n+b);  n += b;  H += (sqrt(2/n) X.float())^T (sqrt(2/n) X.float())
// with alpha = n/(n+b), beta = 2/(n+b).  X is the layer input [T, K] (tokens x
// in_features, row-major, bf16 or fp16), H is [K, K] fp32.
//
// bf16 x bf16 products are exact in fp32, so a bf16-in / fp32-accumulate MFMA
// GEMM differs from the reference's fp32 SGEMM only in summation order.
//
// Shape of the kernel
//  * a workgroup owns a 256 x TN tile of H, TN = 128: 4 waves (2 x 2), two
//    workgroups per CU, so one tile's barriers and epilogue overlap the other's
//    MFMAs.  (The template also covers TN = 256 - 8 waves, one workgroup
//    per CU, a third less operand traffic - which measured 5 % slower at
//    K = 14336 because nothing overlaps its barriers and epilogue.)  Each wave
//    owns 128x64 = 4x2 blocks of v_mfma_f32_32x32x16 (128 accumulator registers
//    per lane);
//  * H is symmetric: only tiles that touch the upper triangle are computed
//    (the lower triangle is filled once, when H is consumed, by lcq_symmetrize);
//  * X is streamed 32 tokens at a time through 3-4 LDS stages in its natural
//    [token][feature] layout by direct global->LDS loads
//    (global_load_lds_dwordx4): no staging registers, no LDS store
//    instructions, one barrier per 32 tokens, two slabs of loads in flight;
//  * the feature-major operand layout MFMA needs (8 consecutive tokens per
//    lane) is produced by the LDS transpose read ds_read_b64_tr_b16, so no
//    VALU shuffles are spent on the transpose;
//  * a direct load deposits a wave's 1 KiB contiguously, so LDS rows cannot be
//    padded; the four token rows a transpose read touches are kept in
//    different banks by an XOR swizzle of the 64-byte blocks of each row.
#include "common.h"
#include "lcq_internal.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int TM = 256;                   // H tile rows (A operand: 256 features)
constexpr int BT = 32;                    // tokens per LDS stage
constexpr int ROW_A = TM * 2;             // bytes per token row of the A operand in LDS (no padding)
constexpr int BYTES_A = BT * ROW_A;

// source of the 16-byte pieces that lie outside X (ragged K or T): they must read as zero
__device__ __attribute__((aligned(16))) const uint32_t zero_piece[4] = {0, 0, 0, 0};

__device__ __forceinline__ s16x4 lds_tr_read(const char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p));
}

template <bool IS_BF16>
__device__ __forceinline__ f32x16 mfma(const s16x8& a, const s16x8& b, const f32x16& c) {
  if constexpr (IS_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Workgroup -> tile map.  Tile (ti, tj) covers rows [256 ti, +256) and columns [TN tj, +TN); with
// Q = 256 / TN it is needed when it reaches the upper triangle: tj >= Q ti.  Workgroups are handed
// to the 8 XCDs round-robin (block b runs on XCD b % 8) and each XCD has its own L2, so every XCD
// gets a contiguous range of a tile order in which consecutive tiles form super-blocks of 4 tile
// rows x 4Q tile columns: the tiles an XCD works on at one time then share a handful of column
// stripes of X.  The map is evaluated by every workgroup, so it is closed-form, not a scan.
template <int Q>
__device__ __forceinline__ void decode_tile(int v, int ntr, int ntc, int& ti, int& tj) {
  constexpr int SB_R = 4, SB_C = 4 * Q;
  // super-row by bisection: the tile rows before row r0 hold r0*ntc - Q*r0*(r0-1)/2 tiles
  int lo = 0, hi = (ntr - 1) / SB_R;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1, r0 = mid * SB_R;
    if (r0 * ntc - Q * (r0 * (r0 - 1) / 2) <= v) lo = mid; else hi = mid - 1;
  }
  const int r0 = lo * SB_R, nr = min(SB_R, ntr - r0);
  v -= r0 * ntc - Q * (r0 * (r0 - 1) / 2);
  // first super-column starts on the diagonal (Q*r0 is a multiple of SB_C) and is clipped by it
  int c0 = Q * r0;
  {
    const int c1 = min(c0 + SB_C, ntc);
    for (int r = r0; r < r0 + nr; ++r) {
      const int n = max(0, c1 - Q * r);
      if (v < n) { ti = r; tj = Q * r + v; return; }
      v -= n;
    }
    c0 += SB_C;
  }
  // the other super-columns are full rectangles nr x SB_C, the last one nr x (ntc - c0)
  const int q = min(v / (nr * SB_C), (ntc - c0 - 1) / SB_C);
  v -= q * nr * SB_C;
  c0 += q * SB_C;
  const int w = min(SB_C, ntc - c0);
  ti = r0 + v / w;
  tj = c0 + v % w;
}

template <int TN> struct HessCfg {
  static constexpr int NW = 2 * TN / 64;                 // waves: 2 x TN/64
  static constexpr int ROW_B = TN * 2;                   // bytes per token row of the B operand
  static constexpr int STAGE = BYTES_A + BT * ROW_B;
  static constexpr int NSTAGE = (TN == 256) ? 4 : 3;     // 128 KiB (one workgroup per CU) / 72 KiB (two)
  static constexpr int LA = 16 / NW;                     // A wave-loads per wave and slab (2 token rows each)
  static constexpr int RB = 1024 / ROW_B;                // token rows per B wave-load
  static constexpr int LB = (BT / RB) / NW;              // B wave-loads per wave and slab
  static constexpr int NL = LA + LB;
};

// How the last round of workgroup slots is filled (lcq_hessian_accum_balanced).  Per XCD: tile slots [0, full_x) run as
// whole tiles; the rem_x tiles behind them are cut into `parts` token ranges each.  parts <= 1: nothing is split.
struct TailSplit {
  int full_x, rem_x, parts;
  float* scratch;        // 8 * rem_x * (parts - 1) tiles of TM x TN floats
};

// EDGE = false: K % 256 == 0 and T % 32 == 0, no bounds checks anywhere.
template <bool IS_BF16, bool EDGE, int TN>
__global__ __launch_bounds__(HessCfg<TN>::NW * 64, TN == 256 ? 1 : 2)
void hessian_kernel(float* __restrict__ H, int K, const uint16_t* __restrict__ X, const uint16_t* __restrict__ XB, int ldx,
                    int T, float alpha, float beta, int ntr, int ntc, int total, int slices, long long hstride, TailSplit ts) {
  using C = HessCfg<TN>;
  constexpr int ROW_B = C::ROW_B, STAGE = C::STAGE, NSTAGE = C::NSTAGE, LA = C::LA, LB = C::LB, RB = C::RB;
  __shared__ __attribute__((aligned(1024))) char lds[NSTAGE * STAGE];
  int ti = 0, tj = 0;
  int ldh = K;                                   // row pitch of the output: H, or a packed TM x TN scratch tile
  bool to_scratch = false;
  {
    const int per_xcd = (total + 7) / 8;
    int slot = blockIdx.x >> 3;
    const int xcd = blockIdx.x & 7;
    if (ts.parts > 1 && slot >= ts.full_x) {
      // The tiles of the last, partly filled round of workgroup slots: each is cut into `parts` token ranges that run
      // side by side.  Part 0 updates H like any tile; the others leave beta * (their X^T X) in scratch tiles, which
      // tail_fold_kernel adds to H afterwards in a fixed order.
      const int i = slot - ts.full_x, r = i / ts.parts, part = i - r * ts.parts;
      slot = ts.full_x + r;
      if (r >= ts.rem_x || xcd * per_xcd + slot >= total) return;
      const long long n32 = T / BT;              // EDGE launches are never split
      const int t0 = (int)(part * n32 / ts.parts) * BT, t1 = (int)((part + 1) * n32 / ts.parts) * BT;
      X += (int64_t)t0 * ldx;
      XB += (int64_t)t0 * ldx;
      T = t1 - t0;
      if (part > 0) {
        H = ts.scratch + ((int64_t)(xcd * ts.rem_x + r) * (ts.parts - 1) + (part - 1)) * (TM * TN);
        ldh = TN;
        alpha = 0.0f;
        to_scratch = true;
      }
    } else if (slot >= per_xcd) {
      return;
    }
    if (xcd * per_xcd + slot >= total) return;
    int v = xcd * per_xcd + slot;
    if (slices > 1) {
      // Token slices: `total` counts every tile once per slice.  Slice s takes an even share of the 32-token slabs,
      // [s n / S, (s + 1) n / S), and its own accumulator H + s * hstride, so a launch with too few tiles for the
      // chip (272 at K = 4096 for 512 workgroup slots) still puts two workgroups on every CU.  A slice without
      // tokens only scales its accumulator by alpha.
      const int tiles = total / slices, slice = v / tiles;
      v -= slice * tiles;
      const long long n32 = (T + BT - 1) / BT;
      const int t0 = (int)(slice * n32 / slices) * BT;
      const int t1 = min((int)((slice + 1) * n32 / slices) * BT, T);
      X += (int64_t)t0 * ldx;
      XB += (int64_t)t0 * ldx;
      H += slice * hstride;
      T = max(t1 - t0, 0);
    }
    decode_tile<TM / TN>(v, ntr, ntc, ti, tj);
  }

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave / (TN / 64), wc = wave % (TN / 64);

  // global -> LDS: direct loads (global_load_lds_dwordx4), no staging registers.  One wave
  // instruction deposits 64 x 16 bytes CONTIGUOUSLY in LDS (lane l at +16 l) from per-lane global
  // addresses: 2 token rows of a 512-byte-wide operand or 4 of a 256-byte-wide one.
  // LDS rows are unpadded; bank conflicts of the transpose reads (which touch token rows r..r+3 at
  // one 64-byte feature block) are avoided by an XOR swizzle instead: 64-byte block c of token row
  // r is stored at block c ^ (r & 3).  The swizzle is applied on the global side (which piece a
  // lane fetches), the LDS side stays contiguous.
  uint32_t gofA[LA], gofB[LB];
  bool okA[LA], okB[LB];
  int rowA[LA], rowB[LB];
  #pragma unroll
  for (int p = 0; p < LA; ++p) {
    const int r = 2 * (wave * LA + p) + (lane >> 5);
    const int col = ti * TM + (((lane & 31) ^ ((r & 3) << 2)) * 8);
    rowA[p] = r;
    gofA[p] = (uint32_t)(r * ldx + col);
    okA[p] = col < K;
  }
  #pragma unroll
  for (int p = 0; p < LB; ++p) {
    constexpr int LPR = 64 / RB;                           // lanes per token row
    const int r = RB * (wave * LB + p) + lane / LPR;
    const int col = tj * TN + (((lane % LPR) ^ ((r & 3) << 2)) * 8);
    rowB[p] = r;
    gofB[p] = (uint32_t)(r * ldx + col);
    okB[p] = col < K;
  }
  // The loads are issued from inline assembly: the compiler would otherwise wait for ALL direct
  // loads (vmcnt(0)) before any LDS read, which serialises the pipeline.  Waits are explicit below.
  const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;
  auto gload = [&](int t0, int stage) {
    const uint16_t* Xs = X + (int64_t)t0 * ldx;              // rows of H come from X ...
    const uint16_t* XsB = XB + (int64_t)t0 * ldx;            // ... columns from XB (the same matrix for X^T X)
    const uint32_t dA = lds0 + stage * STAGE + wave * LA * 1024;
    const uint32_t dB = lds0 + stage * STAGE + BYTES_A + wave * LB * 1024;
    #pragma unroll
    for (int p = 0; p < LA + LB; ++p) {
      const bool isA = p < LA;
      const uint32_t dst = isA ? dA + p * 1024 : dB + (p - LA) * 1024;
      const uint32_t gof = isA ? gofA[isA ? p : 0] : gofB[isA ? 0 : p - LA];
      if constexpr (EDGE) {
        const int r = isA ? rowA[isA ? p : 0] : rowB[isA ? 0 : p - LA];
        const bool ok = (isA ? okA[isA ? p : 0] : okB[isA ? 0 : p - LA]) && t0 + r < T;
        const uint16_t* g = ok ? (isA ? Xs : XsB) + gof : (const uint16_t*)zero_piece;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(g) : "memory");
      } else {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(gof * 2u), "s"(isA ? Xs : XsB) : "memory");
      }
    }
  };

  // transpose-read lane addressing: a group of 16 lanes reads a 4(token) x 16(feature) block;
  // lane s supplies row s/4, features 4*(s%4)..+3 and receives tokens 0..3 of feature s.
  // Every row a lane addresses has (row & 3) == L >> 2, so its swizzled block offsets are fixed.
  const int L = lane & 15, g16 = (lane >> 4) & 1, kh = lane >> 5;
  const int fcol = (g16 * 16 + (L & 3) * 4) * 2, frow = kh * 8 + (L >> 2), sw = L >> 2;
  int offA[4], offB[2];
  #pragma unroll
  for (int b = 0; b < 4; ++b) offA[b] = frow * ROW_A + (wr * 4 + (b ^ sw)) * 64 + fcol;
  #pragma unroll
  for (int j = 0; j < 2; ++j) offB[j] = BYTES_A + frow * ROW_B + ((wc * 2 + j) ^ sw) * 64 + fcol;

  f32x16 acc[4][2];
  #pragma unroll
  for (int i = 0; i < 4; ++i)
    #pragma unroll
    for (int j = 0; j < 2; ++j)
      #pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  auto compute = [&](int stage) {
    const char* const base = lds + stage * STAGE;
    #pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      s16x8 fa[4];
      #pragma unroll
      for (int b = 0; b < 4; ++b) {
        const s16x4 a0 = lds_tr_read(base + offA[b] + ks * 16 * ROW_A);
        const s16x4 a1 = lds_tr_read(base + offA[b] + ks * 16 * ROW_A + 4 * ROW_A);
        fa[b] = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
      }
      #pragma unroll
      for (int j = 0; j < 2; ++j) {
        const s16x4 b0 = lds_tr_read(base + offB[j] + ks * 16 * ROW_B);
        const s16x4 b1 = lds_tr_read(base + offB[j] + ks * 16 * ROW_B + 4 * ROW_B);
        const s16x8 fb = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
        #pragma unroll
        for (int i = 0; i < 4; ++i) acc[i][j] = mfma<IS_BF16>(fa[i], fb, acc[i][j]);
      }
    }
  };

  // NSTAGE LDS stages, one barrier per 32-token slab.  At the top of step s a wave waits for its
  // own loads of slab s (those of the NSTAGE-2 later slabs may stay in flight), the barrier then
  // makes every wave's part of slab s visible and proves that all waves are done reading slab
  // s-1, whose stage the loads of slab s+NSTAGE-1 overwrite.
  const int nsteps = (T + BT - 1) / BT;
  #pragma unroll
  for (int s = 0; s < NSTAGE - 1; ++s)
    if (s < nsteps) gload(s * BT, s);
  int cur = 0, nxt = NSTAGE - 1;
  for (int s = 0; s < nsteps; ++s) {
    const int later = min(nsteps - 1 - s, NSTAGE - 2);          // slabs that may stay in flight
    if (later >= 2) __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * C::NL));
    else if (later == 1) __builtin_amdgcn_s_waitcnt(0x0F70 | C::NL);
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (s + NSTAGE - 1 < nsteps) gload((s + NSTAGE - 1) * BT, nxt);
    __builtin_amdgcn_s_setprio(3);        // the wave that has its operands goes first: keeps the MFMA pipe fed
    compute(cur);
    __builtin_amdgcn_s_setprio(0);
    cur = (cur == NSTAGE - 1) ? 0 : cur + 1;
    nxt = (nxt == NSTAGE - 1) ? 0 : nxt + 1;
  }

  // epilogue: accumulator register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32.
  // The old values of two 32-row bands (64 per lane) are fetched before any is used so the
  // loads overlap; alpha == 0 (first batch) never reads H.
  const int row_l = 4 * (lane >> 5), col_l = lane & 31;
  const int grow = ti * TM + wr * 128 + row_l, gcol = tj * TN + wc * 64 + col_l;
  float* const Hb = to_scratch ? H + (wr * 128 + row_l) * TN + wc * 64 + col_l : H + (int64_t)grow * K + gcol;
  const bool rmw = (alpha != 0.0f);
  #pragma unroll
  for (int ih = 0; ih < 2; ++ih) {
    float old[2][2][16];
    if (rmw) {
      #pragma unroll
      for (int i2 = 0; i2 < 2; ++i2)
        #pragma unroll
        for (int j = 0; j < 2; ++j)
          #pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int dr = (ih * 2 + i2) * 32 + 8 * (r >> 2) + (r & 3), dc = j * 32;
            const bool ok = !EDGE || ((grow + dr < K) && (gcol + dc < K));
            old[i2][j][r] = ok ? Hb[(int64_t)dr * ldh + dc] : 0.0f;
          }
    }
    #pragma unroll
    for (int i2 = 0; i2 < 2; ++i2)
      #pragma unroll
      for (int j = 0; j < 2; ++j)
        #pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int dr = (ih * 2 + i2) * 32 + 8 * (r >> 2) + (r & 3), dc = j * 32;
          const bool ok = !EDGE || ((grow + dr < K) && (gcol + dc < K));
          float v = beta * acc[ih * 2 + i2][j][r];
          if (rmw) v = alpha * old[i2][j][r] + v;
          if (ok) Hb[(int64_t)dr * ldh + dc] = v;
        }
  }
}

// H tile <- ((H tile + part 1) + part 2) + ... for the tiles hessian_kernel cut into token ranges: grid (8 * rem_x, 8),
// every workgroup an eighth of a 256 x 128 tile, 16 bytes per lane and step.
template <int TN>
__global__ __launch_bounds__(256) void tail_fold_kernel(float* __restrict__ H, int K, int ntr, int ntc, int total, TailSplit ts) {
  const int per_xcd = (total + 7) / 8;
  const int xcd = blockIdx.x / ts.rem_x, r = blockIdx.x - xcd * ts.rem_x;
  const int v = xcd * per_xcd + ts.full_x + r;
  if (ts.full_x + r >= per_xcd || v >= total) return;
  int ti, tj;
  decode_tile<TM / TN>(v, ntr, ntc, ti, tj);
  const float* sc = ts.scratch + (int64_t)blockIdx.x * (ts.parts - 1) * (TM * TN);
  constexpr int PER_ROW = TN / 4;
  for (int e = blockIdx.y * 256 + threadIdx.x; e < TM * PER_ROW; e += gridDim.y * 256) {
    const int row = e / PER_ROW, c4 = (e - row * PER_ROW) * 4;
    float* hp = H + (int64_t)(ti * TM + row) * K + tj * TN + c4;
    f32x4 h = *(const f32x4*)hp;
    for (int p = 0; p < ts.parts - 1; ++p) {
      const f32x4 w = *(const f32x4*)(sc + (int64_t)p * (TM * TN) + row * TN + c4);
      h[0] += w[0]; h[1] += w[1]; h[2] += w[2]; h[3] += w[3];
    }
    *(f32x4*)hp = h;
  }
}

// H_0 <- ((H_0 + H_1) + H_2) + ..., H_s <- 0 for s >= 1: the token slices of lcq_hessian_accum_sliced back into one matrix,
// always in this order.
__global__ __launch_bounds__(256) void gather_slices_kernel(f32x4* __restrict__ H, int64_t n4, int slices, int64_t stride4) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
    f32x4 v = H[i];
    for (int s = 1; s < slices; ++s) {
      const f32x4 w = H[s * stride4 + i];
      v[0] += w[0]; v[1] += w[1]; v[2] += w[2]; v[3] += w[3];
      H[s * stride4 + i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    H[i] = v;
  }
}

// x (fp32) -> hi = bf16(x), lo = bf16(x - hi): x = hi + lo up to 2^-17 relative, and every product of two such
// halves is exact in fp32, so fp32 activations go through the bf16 matrix pipe as four products (hi/lo x hi/lo).
__global__ __launch_bounds__(256) void split_f32_kernel(const f32x4* __restrict__ x, int64_t n4, u32x2* __restrict__ hi,
                                                        u32x2* __restrict__ lo) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
    const f32x4 v = __builtin_nontemporal_load(x + i);
    float h[4], l[4];
    #pragma unroll
    for (int k = 0; k < 4; ++k) { h[k] = bf16_round(v[k]); l[k] = bf16_round(v[k] - h[k]); }
    hi[i] = u32x2{bf16_pack(h[0], h[1]), bf16_pack(h[2], h[3])};
    lo[i] = u32x2{bf16_pack(l[0], l[1]), bf16_pack(l[2], l[3])};
  }
}

// staging copy of add_batch: the caller's tokens into the fold buffer.  Streaming 16-byte accesses, every workgroup a
// contiguous 16 KiB run per step (about 1.5x the rate of the runtime's device-to-device copy at these sizes).
__global__ __launch_bounds__(256) void stage_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * 1024;
  for (int64_t base = (int64_t)blockIdx.x * 1024; base < n16; base += stride) {
    u32x4 v[4];
    #pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t i = base + k * 256 + threadIdx.x;
      if (i < n16) v[k] = __builtin_nontemporal_load(src + i);
    }
    #pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t i = base + k * 256 + threadIdx.x;
      if (i < n16) __builtin_nontemporal_store(v[k], dst + i);
    }
  }
}

// Do two byte ranges hold the same bits?  *flag = 1 if any 16-byte piece differs (never cleared here).  add_batch uses
// it for a Linear that shares another Linear's Hessian: the tokens it was handed against the copy the other Linear
// staged from the same memory a moment earlier.
__global__ __launch_bounds__(256) void compare_kernel(const u32x4* __restrict__ a, const u32x4* __restrict__ b, int64_t n16,
                                                      int* __restrict__ flag) {
  const int64_t stride = (int64_t)gridDim.x * 1024;
  uint32_t diff = 0;
  for (int64_t base = (int64_t)blockIdx.x * 1024; base < n16; base += stride) {
    u32x4 va[4], vb[4];
    #pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t i = base + k * 256 + threadIdx.x;
      if (i < n16) { va[k] = __builtin_nontemporal_load(a + i); vb[k] = __builtin_nontemporal_load(b + i); }
      else { va[k] = u32x4{0, 0, 0, 0}; vb[k] = va[k]; }
    }
    #pragma unroll
    for (int k = 0; k < 4; ++k)
      diff |= (va[k][0] ^ vb[k][0]) | (va[k][1] ^ vb[k][1]) | (va[k][2] ^ vb[k][2]) | (va[k][3] ^ vb[k][3]);
  }
  if (diff != 0) *flag = 1;                                // every writer stores the same value
}

// fill the lower triangle from the upper one: H[j][i] = H[i][j], i < j
__global__ __launch_bounds__(256) void symmetrize_kernel(float* __restrict__ H, int K) {
  __shared__ float tile[32][33];
  const int bi = blockIdx.y, bj = blockIdx.x;
  if (bj < bi) return;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int r = ty; r < 32; r += 8) {
    const int64_t i = (int64_t)bi * 32 + r, j = (int64_t)bj * 32 + tx;
    tile[r][tx] = (i < K && j < K) ? H[i * K + j] : 0.0f;
  }
  __syncthreads();
  for (int r = ty; r < 32; r += 8) {
    const int64_t j = (int64_t)bj * 32 + r, i = (int64_t)bi * 32 + tx;     // writes H[j][i]
    if (i < K && j < K && j > i) H[j * K + i] = tile[tx][r];
  }
}

}  // namespace

extern "C" {

int lcq_hessian_accum(float* H, int64_t K, const void* X, int dtype, int64_t T, int64_t ldx, float alpha, float beta,
                      void* stream) {
  return lcq_hessian_accum_sliced(H, K, X, X, dtype, T, ldx, alpha, beta, 1, 0, stream);
}

int lcq_hessian_accum_ab(float* H, int64_t K, const void* X, const void* XB, int dtype, int64_t T, int64_t ldx, float alpha,
                         float beta, void* stream) {
  return lcq_hessian_accum_sliced(H, K, X, XB, dtype, T, ldx, alpha, beta, 1, 0, stream);
}

// Workgroup slots of the device the calling thread uses: two workgroups of the Hessian kernel per CU.
static int hessian_slots() {
  static int slots[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 512;
  if (slots[dev] == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    slots[dev] = 2 * cus;
  }
  return slots[dev];
}

// The split of the last round for a launch over T tokens of K features (see TailSplit); parts == 1: no split pays.
static TailSplit tail_split(int64_t K, int64_t T) {
  constexpr int TN = 128;
  TailSplit ts{0, 0, 1, nullptr};
  if (K % TM != 0 || T % BT != 0) return ts;
  const int ntr = (int)(K / TM), ntc = (int)(K / TN), q = TM / TN;
  int64_t total = 0;
  for (int r = 0; r < ntr; ++r) total += (ntc - q * r > 0) ? (ntc - q * r) : 0;
  const int per_xcd = (int)((total + 7) / 8), slots_x = hessian_slots() / 8;
  if (slots_x <= 0 || per_xcd < 2 * slots_x) return ts;          // fewer than two full rounds: token shares serve better
  const int full_x = per_xcd / slots_x * slots_x, rem_x = per_xcd - full_x;
  if (rem_x == 0 || 2 * rem_x > slots_x) return ts;               // the last round is at least half full as it is
  int parts = slots_x / rem_x;
  if (parts > 8) parts = 8;
  if (T / BT < 4 * parts) return ts;                              // too few tokens to cut
  ts.full_x = full_x; ts.rem_x = rem_x; ts.parts = parts;
  return ts;
}

int64_t lcq_hessian_balanced_workspace_bytes(int64_t K, int64_t T) {
  if (K <= 0 || T <= 0 || K > (1 << 20)) return 0;
  const TailSplit ts = tail_split(K, T);
  return ts.parts > 1 ? (int64_t)8 * ts.rem_x * (ts.parts - 1) * TM * 128 * 4 : 0;
}

static int hessian_launch(float* H, int64_t K, const void* X, const void* XB, int dtype, int64_t T, int64_t ldx,
                          float alpha, float beta, int slices, int64_t slice_stride, TailSplit ts, void* stream);

int lcq_hessian_accum_balanced(float* H, int64_t K, const void* XA, const void* XB, int dtype, int64_t T, int64_t ldx, float alpha,
                               float beta, void* workspace, int64_t workspace_bytes, void* stream) {
  TailSplit ts = (K > 0 && T > 0 && K <= (1 << 20)) ? tail_split(K, T) : TailSplit{0, 0, 1, nullptr};
  if (ts.parts > 1) {
    if (!workspace || workspace_bytes < lcq_hessian_balanced_workspace_bytes(K, T)) return LCQ_EWORKSPACE;
    if (((uintptr_t)workspace % 16) != 0) return LCQ_EALIGN;
    ts.scratch = (float*)workspace;
  }
  return hessian_launch(H, K, XA, XB, dtype, T, ldx, alpha, beta, 1, 0, ts, stream);
}

int lcq_hessian_accum_sliced(float* H, int64_t K, const void* X, const void* XB, int dtype, int64_t T, int64_t ldx,
                             float alpha, float beta, int slices, int64_t slice_stride, void* stream) {
  return hessian_launch(H, K, X, XB, dtype, T, ldx, alpha, beta, slices, slice_stride, TailSplit{0, 0, 1, nullptr}, stream);
}

static int hessian_launch(float* H, int64_t K, const void* X, const void* XB, int dtype, int64_t T, int64_t ldx,
                          float alpha, float beta, int slices, int64_t slice_stride, TailSplit ts, void* stream) {
  if (!H || !X || !XB || K <= 0 || T < 0) return LCQ_EINVAL;
  if (K % 8 != 0 || K > (1 << 20) || T > 0x7fffffff || ldx < K || ldx % 8 != 0 || ldx > (1 << 21)) return LCQ_EINVAL;
  if (slices < 1 || slices > 64 || (slices > 1 && slice_stride < K * K)) return LCQ_EINVAL;
  if (slices > 1 && T > (1 << 30)) return LCQ_ESIZE;               // the kernel's slab arithmetic is 32-bit
  if (((uintptr_t)X % 16) != 0 || ((uintptr_t)XB % 16) != 0 || ((uintptr_t)H % 4) != 0) return LCQ_EALIGN;
  if (T == 0 && alpha == 1.0f) return LCQ_OK;                      // nothing to add and nothing to scale
  constexpr int TN = 128;
  const int ntr = (int)((K + TM - 1) / TM), ntc = (int)((K + TN - 1) / TN), q = TM / TN;
  int64_t total = 0;
  for (int r = 0; r < ntr; ++r) total += (ntc - q * r > 0) ? (ntc - q * r) : 0;
  total *= slices;
  if (total > 0x7ffffff0) return LCQ_ESIZE;
  int64_t grid = (total + 7) / 8 * 8;                             // 8 XCD queues of equal length
  hipStream_t st = (hipStream_t)stream;
  const bool edge = (K % TM != 0) || (T % BT != 0);
  if (ts.parts > 1 && (edge || slices != 1 || dtype == LCQ_F32)) ts.parts = 1;
  if (ts.parts > 1) grid = (int64_t)8 * (ts.full_x + ts.rem_x * ts.parts);
  #define LCQ_HESS(BF, E) hessian_kernel<BF, E, TN><<<dim3((unsigned)grid), dim3(HessCfg<TN>::NW * 64), 0, st>>>( \
      H, (int)K, (const uint16_t*)X, (const uint16_t*)XB, (int)ldx, (int)T, alpha, beta, ntr, ntc, (int)total, slices, \
      (long long)slice_stride, ts)
  if (dtype == LCQ_BF16) { if (edge) LCQ_HESS(true, true); else LCQ_HESS(true, false); }
  else if (dtype == LCQ_F16) { if (edge) LCQ_HESS(false, true); else LCQ_HESS(false, false); }
  else return LCQ_EDTYPE;
  #undef LCQ_HESS
  if (ts.parts > 1)
    tail_fold_kernel<TN><<<dim3((unsigned)(8 * ts.rem_x), 8), dim3(256), 0, st>>>(H, (int)K, ntr, ntc, (int)total, ts);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_hessian_gather_slices(float* H, int64_t K, int slices, int64_t slice_stride, void* stream) {
  if (!H || K <= 0 || K % 8 != 0 || slices < 1 || slices > 64 || (slices > 1 && slice_stride < K * K) || slice_stride % 4 != 0)
    return LCQ_EINVAL;
  if (((uintptr_t)H % 16) != 0) return LCQ_EALIGN;
  if (slices == 1) return LCQ_OK;
  const int64_t n4 = K * K / 4;
  int64_t grid = (n4 + 255) / 256;
  if (grid > 8192) grid = 8192;
  gather_slices_kernel<<<dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream>>>((f32x4*)H, n4, slices, slice_stride / 4);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_split_f32_bf16(const float* x, int64_t n, void* hi, void* lo, void* stream) {
  if (!x || !hi || !lo || n < 0 || n % 4 != 0) return LCQ_EINVAL;
  if ((((uintptr_t)x % 16) | ((uintptr_t)hi % 8) | ((uintptr_t)lo % 8)) != 0) return LCQ_EALIGN;
  if (n == 0) return LCQ_OK;
  int64_t grid = (n / 4 + 255) / 256;
  if (grid > 65536 * 4) grid = 65536 * 4;
  split_f32_kernel<<<dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream>>>((const f32x4*)x, n / 4, (u32x2*)hi, (u32x2*)lo);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_stage_copy(const void* src, void* dst, int64_t bytes, void* stream) {
  if (!src || !dst || bytes < 0 || bytes % 16 != 0) return LCQ_EINVAL;
  if ((((uintptr_t)src | (uintptr_t)dst) % 16) != 0) return LCQ_EALIGN;
  if (bytes == 0) return LCQ_OK;
  const int64_t n16 = bytes / 16;
  int64_t grid = (n16 + 1023) / 1024;
  if (grid > 2048) grid = 2048;
  stage_copy_kernel<<<dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream>>>((const u32x4*)src, (u32x4*)dst, n16);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_compare_bytes(const void* a, const void* b, int64_t bytes, int* flag, void* stream) {
  if (!a || !b || !flag || bytes < 0 || bytes % 16 != 0) return LCQ_EINVAL;
  if ((((uintptr_t)a | (uintptr_t)b) % 16) != 0 || ((uintptr_t)flag % 4) != 0) return LCQ_EALIGN;
  if (bytes == 0) return LCQ_OK;
  const int64_t n16 = bytes / 16;
  int64_t grid = (n16 + 1023) / 1024;
  if (grid > 2048) grid = 2048;
  compare_kernel<<<dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream>>>((const u32x4*)a, (const u32x4*)b, n16, flag);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

int lcq_symmetrize(float* H, int64_t K, void* stream) {
  if (!H || K <= 0 || K > (1 << 20)) return LCQ_EINVAL;
  const unsigned nb = (unsigned)((K + 31) / 32);
  symmetrize_kernel<<<dim3(nb, nb), dim3(256), 0, (hipStream_t)stream>>>(H, (int)K);
  LCQ_CHECK_LAUNCH();
  return LCQ_OK;
}

}  // extern "C"
