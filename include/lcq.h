/* lcq.h — C ABI of liblcq.so: gfx950 (MI355X) kernels for the layer-wise
 * quantization hot path of ModelTC/LightCompress (`llmc`).
 *
 * The reference has no FFI: its boundary for this path is a Python class API
 * (IntegerQuantizer / FloatQuantizer, GPTQ, Awq, *RealQuantLinear.pack).  The
 * Python layer in `lightcompress_amd/` keeps those classes and calls the
 * entry points below through ctypes.  Each entry point cites the reference
 * function it replaces as file:line under llmc/compression/quantization/.
 *
 * Conventions
 *  - every pointer is a DEVICE pointer owned by the caller (a torch tensor's
 *    data_ptr()); `stream` is a hipStream_t passed as void* (NULL = default
 *    stream); calls only enqueue work and return immediately;
 *  - no entry point allocates device memory: scratch memory is a
 *    caller-provided workspace whose size the matching *_workspace_bytes()
 *    call returns;
 *  - return value: 0 ok, <0 rejected before any launch (LCQ_E*);
 *  - matrices are dense row-major;
 *  - calls on one stream execute in order.  Entry points keep no state between
 *    calls, with these exceptions, all of them stated again where they apply:
 *      * lcq_set_gemm_split / lcq_set_chain_lookahead are process-wide
 *        switches (atomic words, read by every later call);
 *      * lcq_chol_inv_upper / lcq_chol_block_factor with K >= 8192 and the
 *        look-ahead switch on create, on first use for a (device, caller's
 *        stream) pair, one more HIP stream (default priority) and two events,
 *        and keep them until the process ends; at most 16 such pairs exist,
 *        later pairs run the chain on the caller's stream alone.  The pair's
 *        events order the two streams, so ONE host thread at a time may
 *        submit chains to a given stream (two threads on two streams are
 *        fine);
 *      * lcq_sq_err_mean_static uses one scratch array per GPU (below).
 */
#ifndef LCQ_H
#define LCQ_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types */
#define LCQ_F32 0
#define LCQ_BF16 1
#define LCQ_F16 2

/* storage of integer / float codes */
#define LCQ_CODE_NONE 0
#define LCQ_CODE_U8 1
#define LCQ_CODE_I8 2
#define LCQ_CODE_I32 3
#define LCQ_CODE_SAME 4      /* codes stored as floats of the input type (what .quant() returns) */
#define LCQ_CODE_F32 5       /* FloatQuantizer.quant(): fp32 values on the minifloat grid */
#define LCQ_CODE_FP8 6       /* float8_e4m3fn / float8_e5m2 bytes */
#define LCQ_CODE_CT4 7       /* lcq_quant_int: 4-bit codes packed like VllmRealQuantLinear.pack (module_utils.py:929-955):
                                nibble i of int32 word j of a tensor row = code[8j+i] + 8; needs -8 <= qmin, qmax <= 7
                                and cols % 8 == 0; `codes` is int32 [rows * cols / 8] */

/* flags */
#define LCQ_FLAG_SYM 1            /* symmetric: zero point is 0 */
#define LCQ_FLAG_NO_ROUND_ZP 2    /* round_zp=False, quant.py:556-557,702-706 */
#define LCQ_FLAG_STATIC 4         /* scales/zeros are INPUTS (…_static methods) */
#define LCQ_FLAG_SCALAR_QP 8      /* one (scale, zero) for the whole tensor (per_tensor) */
#define LCQ_FLAG_TIE_EVEN 16      /* minifloat rounding: ties to even instead of away from zero */
#define LCQ_FLAG_NO_SUBNORMALS 32 /* minifloat rounding: flush below the minimum normal */
#define LCQ_FLAG_DQ_F32 64        /* lcq_quant_fp: write dq as fp32 instead of the input type */
#define LCQ_FLAG_RANGE_BF16 128   /* lcq_qparams_int on fp32 I/O: (max-min) and the 1e-5 clamp act in bf16,
                                     the rest in fp32 — torch's promotion when 0-dim bf16 ranges meet the
                                     0-dim fp32 (qmax-qmin) of a per_tensor quantizer */
#define LCQ_FLAG_SCALE_F32 256    /* STATIC only: `scales` / `zeros` hold fp32 even for bf16 rows (a 0-dim fp32 qparam
                                     next to a bf16 tensor).  torch on a GPU converts a 0-dim tensor operand to the
                                     type of the result before every operation: the parameters are rounded to the row
                                     type where they meet the rows (x / s, + z, - z, * s), scales * output_scale_factor
                                     is formed in fp32 first; lcq_quant_fp multiplies its fp32 codes by the fp32 scale */

#define LCQ_FLAG_CLAMP_RANGE 1024  /* lcq_fp8_block_quant: s = clamp(max|x|, 1e-5) / 448 (the FloatQuantizer path) instead of max|x| / 448 */
#define LCQ_FLAG_TIE_AWAY 2048     /* lcq_fp8_block_quant: exact ties round away from zero instead of to even */
#define LCQ_FLAG_RANGE_F16 8192    /* LCQ_FLAG_RANGE_BF16 for ranges that were fp16 */
#define LCQ_FLAG_ROWS16 4096       /* lcq_gptq_block: 16 rows per workgroup whatever R is (the default takes 32 from 6144 rows on; same results bit for bit) */
#define LCQ_FLAG_ROW_QP 512       /* lcq_quant_fp_emu, STATIC only: `scales` holds one value per row */

/* errors */
#define LCQ_OK 0
#define LCQ_EINVAL (-1)
#define LCQ_EALIGN (-2)
#define LCQ_EDTYPE (-3)
#define LCQ_ELAUNCH (-4)
#define LCQ_EWORKSPACE (-5)
#define LCQ_ESIZE (-6)        /* input larger than an entry point's stated maximum */

/* ---- integer quantizer -------------------------------------------------- */

/* Fused get_tensor_qparams + quant (+ dequant) over `rows` rows of `cols`
 * elements (the reshaped tensor of quant.py:611-641).
 * Replaces quant.py:134-145 (min/max), :544-558 (get_qparams), :698-716
 * (quant / dequant / quant_dequant) and so the bodies of
 * fake_quant_{weight,act}_{dynamic,static} (:718-868) and
 * real_quant_weight_{dynamic,static} (:870-952).
 *  x       [rows, cols] of `dtype` (LCQ_F32 | LCQ_BF16 | LCQ_F16; fp16 rows run through the element-wise kernel,
 *          one wave per row: correct to the bit, not tuned; no LCQ_CODE_CT4 for them)
 *  dq      same shape/type or NULL        -> (q - z) * (s * out_scale_factor)
 *  codes   [rows, cols] of code_dtype or NULL
 *  scales  [rows] (or [1] with SCALAR_QP) of `dtype`: output, input if STATIC
 *  zeros   likewise; may be NULL (zero point 0; never written when SYM)
 * bf16 / fp16 rows round to their type after every arithmetic step like torch does. */
int lcq_quant_int(const void* x, int dtype, int64_t rows, int64_t cols, float qmin, float qmax, int flags,
                  float out_scale_factor, void* dq, void* codes, int code_dtype, void* scales, void* zeros,
                  void* stream);

/* get_minmax_range, quant.py:141-143: per-row amin / amax, outputs [rows] of `dtype`. */
int lcq_minmax_rows(const void* x, int dtype, int64_t rows, int64_t cols, void* min_out, void* max_out, void* stream);

/* get_minmax_range per_tensor, quant.py:135-137: outputs [1] of `dtype`. */
int64_t lcq_minmax_all_workspace_bytes(void);
int lcq_minmax_all(const void* x, int dtype, int64_t n, void* min_out, void* max_out, void* workspace, void* stream);

/* The torch.histc(tensor.float(), bins, min, max) of get_static_hist_range, quant.py:461-511 (calib_algo
 * 'static_hist'): hist[b] = number of elements with lo <= v <= hi and b = (int)((v - lo) * bins / (hi - lo)) in fp32
 * (b == bins counts into the last bin); lo == hi widens the range to [lo - 1, hi + 1] as torch does.
 *  x [n] of `dtype` (LCQ_F32 | LCQ_BF16 | LCQ_F16), counts: workspace of `bins` uint32, hist [bins] fp32; bins <= 8192. */
int lcq_histc(const void* x, int dtype, int64_t n, int bins, float lo, float hi, void* counts, float* hist, void* stream);

/* get_qparams, quant.py:544-558, on n explicit (min, max) pairs. */
int lcq_qparams_int(const void* min_in, const void* max_in, int dtype, int64_t n, float qmin, float qmax, int flags,
                    void* scales, void* zeros, void* stream);

/* get_mse_range, quant.py:147-205 (calib_algo 'mse'): per row the shrunken range p * (min, max), p = 1 - i / grid_n,
 * i < steps, with the smallest sum_j |quant_dequant(x_j) - x_j| ^ norm; a better step replaces the range the next
 * steps shrink (the reference's aliasing of best_min_val with min_val).  x [rows, cols] of `dtype`, arithmetic and
 * outputs [rows] in fp32 (the reference upcasts with tensor.float()). */
int lcq_mse_range(const void* x, int dtype, int64_t rows, int64_t cols, float qmin, float qmax, int flags, int steps,
                  int grid_n, float norm, float* min_out, float* max_out, void* stream);

/* One iteration of BaseQuantizer.optimize_weights_proximal (the HQQ zero-point solver), quant.py:587-609:
 *   W_q = clamp(round(x * inv_s + z), qmin, qmax), inv_s = 1/s;  W_r = (W_q - z) / inv_s
 *   W_e = sign(d) relu(|d| - inv_beta |d|^(lp_norm-1)), d = x - W_r   (lp_norm == 1: |d| - inv_beta; the
 *   reference's shrink_op reads self.beta, not the annealed beta it is handed, quant.py:94-103)
 *   zeros_out[r] = mean_c(W_q - (x - W_e) * inv_s);  abs_err_rowsum[r] = sum_c |x - W_r|
 *  x [rows, cols] fp32 (get_hqq_qparams casts to float first, quant.py:680); scales, zeros_in, zeros_out,
 *  abs_err_rowsum [rows] fp32; zeros_in NULL = 0 (symmetric start); zeros_out must not alias zeros_in;
 *  scales_roundtrip [rows] or NULL: 1/(1/s), what the reference returns as scales.
 *  The caller owns the loop: error = sum(abs_err_rowsum) / (rows*cols), stop at the first iteration that does
 *  not improve on the best error (the zeros of that iteration are the result). */
int lcq_hqq_step(const float* x, int64_t rows, int64_t cols, const float* scales, const float* zeros_in, float* zeros_out,
                 float* abs_err_rowsum, float* scales_roundtrip, float inv_beta, float lp_norm, float qmin, float qmax,
                 void* stream);


/* dequant, quant.py:709-711: out = (q - z) * (s * out_scale_factor). */
int lcq_dequant_int(const void* q, int dtype, int64_t rows, int64_t cols, const void* scales, const void* zeros,
                    int flags, float out_scale_factor, void* out, void* stream);

/* ---- minifloat quantizer (FloatQuantizer, use_qtorch=True) -------------- */

/* Fused get_tensor_qparams + quant (+ dequant), quant.py:1042-1080 and the
 * bodies of fake_quant_* (:1082-1158) and real_quant_weight_* (:1160-1220):
 *   s = clamp(absmax, 1e-5) / qmax;  t = x / s + 0;  q = float_quantize(float(t));
 *   dq = (q - 0) * s  (fp32), cast to the row type unless LCQ_FLAG_DQ_F32.
 *  codes: LCQ_CODE_F32 (what .quant() returns) or LCQ_CODE_FP8 (e4m3fn / e5m2 bytes)
 * float_quantize's tie rule / subnormal handling are third-party semantics
 * (QPyTorch) selectable with LCQ_FLAG_TIE_EVEN / LCQ_FLAG_NO_SUBNORMALS. */
int lcq_quant_fp(const void* x, int dtype, int64_t rows, int64_t cols, int e_bits, int m_bits, float qmax, int flags,
                 void* dq, void* codes, int code_dtype, void* scales, void* stream);

/* FloatQuantizer.dequant, quant.py:1073-1075, on fp32 codes: out = (q - 0) * s in fp32. */
int lcq_dequant_fp(const float* q, int64_t rows, int64_t cols, const void* scales, int scale_dtype, int flags,
                   float* out, void* stream);

/* FloatQuantizer with use_qtorch=False: get_float_qparams (quant.py:1004-1026) + quant / dequant
 * (:1058-1075) in one pass.  Dynamic (default): per-row ranges `min_in` / `max_in` [rows] give
 *   maxval = max(max, -min);  bias = 2^e - log2(maxval) + log2(2 - 2^-m) - 1  and per element
 *   xc = clamp(x, -maxval, maxval);  s = 2^(clamp(floor(log2|xc| + bias), 1) - m - bias);
 *   q = round(xc / s + 0);  dq = (q - 0) * s
 * LCQ_FLAG_STATIC: `scales_in` is given ([rows, cols], or [rows] with LCQ_FLAG_ROW_QP, or [1] with
 * LCQ_FLAG_SCALAR_QP) and xc = x.  Every output is optional and has the shape and type of x, except
 * q with LCQ_CODE_FP8 (float8 bytes, e4m3 / e5m2 only).  cols % (16 / element size) == 0. */
int lcq_quant_fp_emu(const void* x, int dtype, int64_t rows, int64_t cols, int e_bits, int m_bits, int flags,
                     const void* min_in, const void* max_in, const void* scales_in, void* xc, void* scales_out,
                     void* q, int code_dtype, void* dq, void* stream);

/* Block-wise float8 casts: weight_cast_to_fp8 / act_quant, kernel.py:7-85 (Triton) and their fallback through
 * FloatQuantizer(granularity='per_block'), quant.py:33-45:  per block  s = max|x| / 448 (fp32),
 * y = float8_e4m3fn(x / s) computed in fp32.  block_rows = 128: blocks of 128 x 128 of x [M, N], scales [ceil(M/128),
 * ceil(N/128)]; block_rows = 1: blocks of 1 x 128 (activations; N % 128 == 0), scales [M, N/128].
 * x of `dtype` (LCQ_F32 | LCQ_BF16), y float8 bytes [M, N]. */
int lcq_fp8_block_quant(const void* x, int dtype, int64_t M, int64_t N, int block_rows, int flags, void* y, float* scales,
                        void* stream);

/* weight_cast_to_bf16, kernel.py:88-138 / quant.py:20-31: out[i, j] = float(y[i, j]) * scales[i / 128, j / 128];
 * out of `out_dtype` (LCQ_BF16 | LCQ_F32). */
int lcq_fp8_block_dequant(const void* y, const float* scales, int64_t M, int64_t N, void* out, int out_dtype, void* stream);

/* ---- packing ------------------------------------------------------------ */

/* VllmRealQuantLinear.pack, module_utils.py:929-955 (compressed-tensors order).
 *  codes [R, K] of LCQ_CODE_I32 | LCQ_CODE_I8 | LCQ_CODE_U8 ; packed [R, ceil(K / (32/bits))] int32 */
int lcq_pack_ct(const void* codes, int code_dtype, int64_t R, int64_t K, int bits, int32_t* packed, void* stream);

/* AutoawqRealQuantLinear.gemm_pack, module_utils.py:1097-1158 (4-bit, order 0,2,4,6,1,3,5,7).
 *  w [R, K] of `dtype` (F32 | BF16 | F16); scales [R, K/g] of `dtype`; zeros [R, K/g] int32
 *  qweight [K, R/8] int32 ; scales_f16_out [K/g, R] fp16 ; qzeros [K/g, R/8] int32 ; R % 32 == 0 */
int lcq_pack_awq(const void* w, int dtype, const void* scales, const int32_t* zeros, int64_t R, int64_t K, int group_size,
                 int32_t* qweight, void* scales_f16_out, int32_t* qzeros, void* stream);

/* ---- GPTQ --------------------------------------------------------------- */

/* GPTQ.add_batch, gptq.py:253-295:  H <- alpha*H + beta * X^T X  with
 * alpha = n/(n+b), beta = 2/(n+b) (n = batches seen so far, b = batches in this call).
 *  H [K, K] fp32; X [T, K] tokens x in_features of LCQ_BF16 | LCQ_F16, 16-byte aligned; K % 8 == 0;
 *  ldx = elements between consecutive token rows (>= K, % 8 == 0).
 * Only the tiles that reach the upper triangle are updated: call lcq_symmetrize before reading
 * anything below the diagonal. alpha == 0 does not read H.  T == 0 leaves H <- alpha*H (no launch when alpha == 1). */
int lcq_hessian_accum(float* H, int64_t K, const void* X, int dtype, int64_t T, int64_t ldx, float alpha, float beta,
                      void* stream);

/* The same update with different matrices on the two sides:  H <- alpha*H + beta * XA^T XB  on the tiles that reach
 * the upper triangle (XA supplies the rows of H, XB the columns; both [T, K] with the same ldx and dtype).
 * add_batch on fp32 activations (gptq.py:289 `chunk.float()`) uses it with the two bf16 halves of
 * lcq_split_f32_bf16: X^T X = hi^T hi + hi^T lo + lo^T hi + lo^T lo. */
int lcq_hessian_accum_ab(float* H, int64_t K, const void* XA, const void* XB, int dtype, int64_t T, int64_t ldx, float alpha,
                         float beta, void* stream);

/* x [n] fp32 -> hi = bf16(x), lo = bf16(x - hi)  ([n] bf16 each; n % 4 == 0): x == hi + lo to 2^-17 relative. */
int lcq_split_f32_bf16(const float* x, int64_t n, void* hi, void* lo, void* stream);

/* The same update with the tokens cut into `slices` contiguous shares (whole 32-token slabs, dealt out evenly), share
 * s accumulating into its own matrix H + s * slice_stride (elements; >= K*K):
 *   H_s <- alpha*H_s + beta * XA_s^T XB_s   for every s < slices (a share without tokens only scales its matrix; T == 0 scales all of them),
 * so the sum over s of the H_s follows the recurrence of gptq.py:279-294 like a single H does.  For Linears whose
 * Hessian has too few tiles to fill the chip (272 at K = 4096 against 512 workgroup slots) three shares are ~17 %
 * faster than one.  slices in 1..64 (T <= 2^30 when > 1); slices == 1 is lcq_hessian_accum_ab.  Matrices start zeroed (or alpha == 0). */
int lcq_hessian_accum_sliced(float* H, int64_t K, const void* XA, const void* XB, int dtype, int64_t T, int64_t ldx,
                             float alpha, float beta, int slices, int64_t slice_stride, void* stream);

/* lcq_hessian_accum_ab with the last round of workgroups filled.  A launch has one workgroup per 256 x 128 tile that
 * reaches the upper triangle and the chip runs 2 x CUs of them at a time; when the tiles are several such rounds and a
 * small rest (K = 14336: 3192 tiles = 6 rounds of 512 and 120), the rest keeps a quarter of the chip busy for the time of a
 * whole tile.  Here every tile of the rest is cut into 2..8 token ranges that run side by side: the first updates H like
 * any tile, the others leave their beta * XA^T XB in the workspace, and a second small launch adds them to H in a fixed
 * order (results are reproducible; they differ from lcq_hessian_accum_ab's by the order of fp32 additions).
 * lcq_hessian_balanced_workspace_bytes(K, T) is the workspace this takes for a launch of T tokens, 0 where no split
 * pays (K not in whole 256-column tiles, T not in whole 32-token slabs, fewer than two rounds, or a rest that fills
 * half a round anyway): the call then is lcq_hessian_accum_ab and takes a NULL workspace.  Workspace 16-byte aligned. */
int64_t lcq_hessian_balanced_workspace_bytes(int64_t K, int64_t T);
int lcq_hessian_accum_balanced(float* H, int64_t K, const void* XA, const void* XB, int dtype, int64_t T, int64_t ldx, float alpha,
                               float beta, void* workspace, int64_t workspace_bytes, void* stream);

/* H_0 <- ((H_0 + H_1) + H_2) + ... and H_s <- 0 for s >= 1, over all K*K entries: the shares of
 * lcq_hessian_accum_sliced back into the one matrix that gptq.py keeps (layers_cache[name]['H']); accumulation may
 * go on afterwards.  H 16-byte aligned, slice_stride % 4 == 0. */
int lcq_hessian_gather_slices(float* H, int64_t K, int slices, int64_t slice_stride, void* stream);

/* *flag = 1 if a[0 .. bytes) and b[0 .. bytes) differ in any bit; *flag is left alone otherwise (the caller clears it
 * once and may let several calls report into it).  Both 16-byte aligned, bytes % 16 == 0.  No counterpart in the
 * reference: GPTQ.add_batch here lets Linears that are handed the same tensor (the hooks of q/k/v, gptq.py:246-251)
 * share one Hessian, and checks with this call that the tensor still holds what the first Linear saw. */
int lcq_compare_bytes(const void* a, const void* b, int64_t bytes, int* flag, void* stream);

/* The staging copy of GPTQ.add_batch (gptq.py:283-290 consumes `inp` at once; here the tokens of several calls are
 * kept until one folded Hessian launch): dst[0 .. bytes) = src[0 .. bytes), both 16-byte aligned, bytes % 16 == 0. */
int lcq_stage_copy(const void* src, void* dst, int64_t bytes, void* stream);

/* H[j][i] = H[i][j] for i < j. */
int lcq_symmetrize(float* H, int64_t K, void* stream);

/* The weight side of GPTQ.process_hessian_and_weights, gptq.py:133-141, 150-151, in one pass:
 *   W = weight.clone().float(); W[:, dead] = 0; W = W[:, perm]
 *  w [R,K] fp32 / bf16 / fp16; perm [K] int64 or NULL; dead [K] bytes (non-zero = dead column, indexed in the
 *  ORIGINAL column order) or NULL; out [R,K] fp32, must not alias w. */
int lcq_gptq_prepare_weights(const void* w, int dtype, int64_t R, int64_t K, const int64_t* perm, const uint8_t* dead,
                             float* out, void* stream);

/* How the large fp32 products of the Cholesky chain (torch.linalg.cholesky / cholesky_inverse, gptq.py:172-174) and of
 * the deferred loop update (gptq.py:244) are evaluated.  1 (default): launches of more than 256 output tiles run on
 * the bf16 matrix pipe with every fp32 operand split into three bf16 planes and six partial products per product
 * (accuracy of an fp32 multiply-add, 16/6 of the fp32 pipe's rate); 0: everything on the fp32 matrix pipe.
 * Process-wide (an atomic word that every later call reads); returns the previous setting. */
int lcq_set_gemm_split(int on);

/* Chains of K >= 8192: 1 (default) runs the deep trailing update behind a 512-column super-panel in two parts, the
 * columns of the next super-panel on the caller's stream and the rest on a stream the library creates once per
 * (device, caller's stream), beside the next super-panel's narrow launches; the two are ordered by events and joined
 * before the call's last launches, so the caller sees one stream-ordered call.  0: everything on the caller's stream.
 * The results agree to fp32 rounding (a part of an update may select the other GEMM kernel than the whole update
 * would) and are reproducible from run to run either way.  Process-wide (an atomic word that every later chain reads
 * once); returns the previous setting.  The side stream and its two events are created on the first such chain of a
 * (device, caller's stream) pair and kept until the process ends; 16 pairs at most, further pairs run on the caller's
 * stream alone; one host thread at a time per caller's stream. */
int lcq_set_chain_lookahead(int on);

/* Dead columns, act-order permutation, damping and the Cholesky chain of
 * GPTQ.process_hessian_and_weights, gptq.py:139-141, 150-153, 169-174:
 *   dead = diag(H)==0; H[dead,dead] = 1; W[:,dead] = 0; H = H[perm][:,perm];
 *   H += percdamp*mean(diag H)*I; U = chol(cholesky_inverse(chol(H)), upper)
 *  H [K,K] fp32, valid on and above the diagonal (its diagonal is rewritten for dead columns, and with a
 *  permutation its lower triangle is filled in from the upper one)
 *  perm [K] int64 or NULL (identity); W [R,K] fp32 in ORIGINAL column order or NULL
 *  U [K,K] fp32 out: upper triangular, zeros below the diagonal; U may alias H
 *  status [1] int32 device word or NULL: 1 if a non-positive pivot was met (H not positive definite) */
int64_t lcq_chol_inv_upper_workspace_bytes(int64_t K);
int lcq_chol_inv_upper(float* H, int64_t K, const int64_t* perm, float percdamp, float* W, int64_t R, float* U,
                       void* workspace, int64_t workspace_bytes, int* status, void* stream);

/* The same chain without the triangular inverse, for the column loop alone (K % 128 == 0, blocks of 128 columns).
 * With H_d = M M^T (M upper triangular) the reference's factor is U = M^-1; P [K,K] out is block upper triangular:
 *   P[b, b] = U[b, b] = (M[b, b])^-1        the 128 x 128 diagonal blocks of U, exactly what gptq.py:205 takes as Hinv1
 *   P[p, b] = M[p, b] U[b, b],  p < b        in place of U[p, b]
 * From E U = W0 - Q (E the loop's errors Err1, Q the quantized weights, W0 the weights before the loop) the weights
 * the loop finds at block b are  W0[:, b] + sum_{p<b} (W0 - Q)[:, p] P[p, b]:  lcq_gptq_block / lcq_gptq_trailing give
 * the reference's results on P when a block hands (Q - W0) to the deferred update (the W0 argument of
 * lcq_gptq_block).  Valid while every group of the quantizer lies inside one block (group_size divides 128, or
 * given parameters); saves the K^3/3 flop of the inverse.  Same workspace, arguments and status as above. */
int lcq_chol_block_factor(float* H, int64_t K, const int64_t* perm, float percdamp, float* W, int64_t R, float* P,
                          void* workspace, int64_t workspace_bytes, int* status, void* stream);

/* One lazy-batch block of GPTQ.weight_transform, gptq.py:203-243 (columns i1 .. i1+count, count <= 128):
 * per-group scale/zero refresh (search_column_qparams, :358-366), quantize-dequantize,
 * tmp[:, i] = w, Losses[:, i], in-block error feedback; Err [R,128] receives Err1.
 *  W, tmp, Losses [R,K] fp32; Err [R, ldErr] fp32 (column i of the block -> Err[:, i]);
 *  U [K,K] upper factor; scales / zeros [R,G] fp32
 *  dynamic groups (default): group_size > 0, G >= ceil(n_quant/group_size), qparams are written
 *  LCQ_FLAG_STATIC: qparams are inputs; group of column c is gidx[c] (or c/group_size, or 0 if group_size == 0)
 *  n_quant: the columns [0, n_quant) are quantized, a group's range ends there at the latest (gptq.py:218-221,
 *  `self.columns - self.n_out`); K without OWQ outlier columns
 *  W0: NULL, or the [R,K] weights as they were before the loop when U is the block factor P of
 *  lcq_chol_block_factor: Err then receives (quantized value - W0) instead of Err1, which is what the deferred
 *  update needs with P. */
int lcq_gptq_block(float* W, float* tmp, float* Losses, float* Err, int64_t ldErr, const float* U, const float* W0, int64_t R,
                   int64_t K, int64_t n_quant, int64_t i1, int count, int group_size, float qmin, float qmax, int flags,
                   float* scales, float* zeros, const int32_t* gidx, int64_t G, void* stream);

/* Deferred update of gptq.py:244, generalised to a column window (fp32 MFMA):
 *   W[:, j1:j2] -= Err[:, :k2-k1] @ U[k1:k2, j1:j2],   k2 <= j1.
 * The reference's call is (k1, k2, j1, j2) = (i1, i2, i2, K); splitting the column range lets the
 * caller apply far-away columns once per several blocks with a deeper contraction. */
int lcq_gptq_trailing(float* W, const float* Err, int64_t ldErr, const float* U, int64_t R, int64_t K, int64_t k1,
                      int64_t k2, int64_t j1, int64_t j2, void* stream);

/* ---- AWQ scale search ------------------------------------------------------- */

/* Awq.fake_quantize_weight, awq.py:147-164 with scaling_weight :39-46 fused in:
 *   out = fake_quant_weight_dynamic(W * s[None, :])   (W*s rounds to the tensor type first)
 *  W, out [R, K] of `dtype`; colscale [K] of `dtype`, 16-byte aligned; group_size 0 = per_channel.
 * W is not modified (the reference multiplies in place and restores the weights afterwards). */
int lcq_awq_scale_quant(const void* w, int dtype, int64_t R, int64_t K, const void* colscale, int group_size,
                        float qmin, float qmax, int flags, void* out, void* stream);

/* workspace of lcq_absmean_cols / lcq_awq_weight_scale / lcq_sq_err_mean for K columns */
int64_t lcq_awq_workspace_bytes(int64_t K);

/* Awq.get_act_scale, awq.py:74-85: out[k] = mean_t |x[t, k]| (fp32 accumulation, result in `dtype`).
 * The mean is torch's GPU mean: the fp32 sum times the fp32 factor float(K) / (T * K), cast to `dtype` (torch's CPU
 * kernel divides by T instead: the last place differs when T is no power of two). */
int lcq_absmean_cols(const void* x, int dtype, int64_t T, int64_t K, void* out, void* workspace, void* stream);

/* Awq.get_weight_scale (one layer), awq.py:58-66: out[k] = mean_r ( |W[r,k]| / max|W[r, group(k)]| ), the mean as in
 * lcq_absmean_cols. */
int lcq_awq_weight_scale(const void* w, int dtype, int64_t R, int64_t K, int group_size, void* out, void* workspace,
                         void* stream);

/* scaling_input, base_blockwise_quantization.py:899-912: out = x / s[None, :]. */
int lcq_div_cols(const void* x, int dtype, int64_t T, int64_t K, const void* s, void* out, void* stream);

/* Folding searched scales into neighbouring weights, base_blockwise_quantization.py:664-723, 772-801
 * (scale_fc_fc, scale_ln_fcs: `fc.weight.mul_(scales.view(1, -1))`, `fc1.weight.div_(scales.view(-1, 1))`,
 * `ln.weight.div_(scales)`):  out = x (* or /) s  with s a column vector [K] (mode 0 multiply, 1 divide) or a row
 * vector [T] (mode 2 multiply, 3 divide) of `dtype`; x, out [T, K] of `dtype` (LCQ_F32 | LCQ_BF16), out may be x.
 * One IEEE operation per element, rounded to `dtype`. */
int lcq_scale_matrix(const void* x, int dtype, int64_t T, int64_t K, const void* s, int mode, void* out, void* stream);

/* Awq.calculate_loss, awq.py:134-145: out[0] = mean( float((a - b) in `dtype`)^2 ), kept on the device. */
int lcq_sq_err_mean(const void* a, const void* b, int dtype, int64_t n, float* out, void* workspace, void* stream);

/* lcq_sq_err_mean for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc): same kernels, same result bit for bit, but the partial sums live in a 64 KiB array that is
 * part of the library's device image instead of a caller workspace.  No counterpart in the reference.
 * Calls no hipMalloc / hipFree or other allocating routine; the first call on a device looks the array's address up
 * (hipGetSymbolAddress, under a mutex), which is not a kernel launch: make one call on the device OUTSIDE any stream
 * capture first; every later call is two kernel launches and nothing else, and may be captured.
 *  n <= LCQ_SQ_ERR_STATIC_MAX_N, else LCQ_ESIZE.
 * Every call on one GPU uses that GPU's single array: calls that overlap on one GPU (different streams) race;
 * calls on one stream, or ordered by events, are safe.  Nothing needs clearing between calls. */
#define LCQ_SQ_ERR_STATIC_MAX_N (((int64_t)1) << 34)
int lcq_sq_err_mean_static(const void* a, const void* b, int dtype, int64_t n, float* out, void* stream);

/* AutoClipper.auto_clip_layer, auto_clip.py:83-191 (clip_version v1, weight-only, per_group with group_size 128):
 * for every (output row, group) the shrink step i in [0, n_steps) of the group range
 *   max_i = org_max * (1 - i / n_grid),  min_i = org_min * (1 - i / n_grid)   (min_i = -max_i if clip_sym)
 * that minimises  mean_t ( sum_j x[t, g, j] * (fq(clamp(w, min_i, max_i)) - w)[r, g, j] )^2 ; the first minimum wins.
 *  w [R, K] LCQ_BF16; x [T, K] LCQ_BF16 (the sampled tokens); K % 128 == 0; G = K / 128
 *  best_max, best_min [R, G] bf16 out;  errs [R, G, n_steps] fp32 out or NULL (the means, before their rounding to bf16)
 *  qmin / qmax / flags (LCQ_FLAG_SYM, LCQ_FLAG_NO_ROUND_ZP): the weight quantizer of fake_quant_weight_dynamic.
 * bf16 MFMA with fp32 accumulation: the reference's two bf16-rounded dot products are evaluated as one product with
 * the bf16-rounded weight difference. */
int lcq_awq_clip_search(const void* w, const void* x, int64_t R, int64_t K, int64_t T, int n_grid, int n_steps,
                        int clip_sym, float qmin, float qmax, int flags, void* best_max, void* best_min, float* errs,
                        void* stream);

/* The grouped products of AutoClipper.auto_clip_layer, auto_clip.py:141,160: `(x * w).sum(dim=-1)` with
 * x [1, T, G, gs] and w [R, 1, G, gs]:  out[r, g, t] = round(sum_j round(x[t, g*gs + j] * w[r, g*gs + j])) - every
 * product rounded to the tensors' type as the materialised product tensor is, fp32 accumulation, one final rounding
 * (the reference's [R, T, G] result, stored with the token index fastest).
 * With org != NULL (such sums for the original weights, same layout) nothing is stored in `out` (may be NULL) and
 *   err[r, g] = round(mean_t round(round(out - org)^2))        auto_clip.py:163, `(cur_out - org_out).pow(2).mean(dim=1)`
 *  x [T, K], w [R, K], out / org [R, K / group_size, T], err [R, K / group_size], all of `dtype` (LCQ_F32 | LCQ_BF16). */
int lcq_group_dots(const void* x, const void* w, int dtype, int64_t R, int64_t K, int64_t T, int group_size, void* out,
                   const void* org, void* err, void* stream);

/* AutoClipper.apply_clip v1, auto_clip.py:194-211: out[r, g*gs + j] = clamp(w[r, g*gs + j], lo[r, g], hi[r, g]);
 * w, out [R, K] of `dtype` (LCQ_F32 | LCQ_BF16), lo / hi [R, K / group_size] of `dtype`; out may alias w. */
int lcq_clamp_groups(const void* w, int dtype, int64_t R, int64_t K, int group_size, const void* lo, const void* hi,
                     void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LCQ_H */
