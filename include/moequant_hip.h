/* moequant_hip.h -- C ABI of libmoequant_hip.so (AMD gfx950 / MI355X).
 *
 * Conventions (all entry points):
 *   - every pointer is a DEVICE pointer owned by the caller, including workspaces; the library never
 *     allocates, frees or synchronises;
 *   - every kernel is launched on `stream` (a hipStream_t passed as void*; NULL = the default stream);
 *   - return value: 0 = launched, <0 = MQ_ERR_* (nothing launched, or launching stopped at the failing
 *     kernel); numerical trouble is reported through a device-side `info` word, LAPACK style;
 *   - matrices are row-major, `ld*` are leading dimensions in ELEMENTS;
 *   - no exceptions cross the boundary; calls are re-entrant per stream and may come from several host threads
 *     (one-time set-up inside the library is guarded).
 *
 * Citations name the MoE-Quant code each entry point replaces (paths relative to that repository).
 */
#ifndef MOEQUANT_HIP_H
#define MOEQUANT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MQ_OK 0
#define MQ_ERR_ARG (-1)
#define MQ_ERR_LAUNCH (-2)
#define MQ_ERR_WORKSPACE (-3)
#define MQ_ERR_TOO_LARGE (-4)

/* element types for `x_dtype` / `w_dtype` / `round_dtype` */
#define MQ_DT_F32 0 /* round_dtype: no rounding */
#define MQ_DT_BF16 1
#define MQ_DT_F16 2

/* ---- (1) Hessian accumulation -------------------------------------------------------------------
 * H <- beta*H + alpha * X^T X.   Replaces `self.H.addmm_(input.T, input, beta, alpha)` together with
 * the `input.float()` up-cast in GPTQ.update, src/gptq.py:97-103.
 *   H  : C x C fp32 (ldh).  Only the upper triangle of the old H is read.  The upper triangle is always
 *        written; with mirror != 0 the lower triangle is written too (symmetric copy).
 *   X  : n x C tokens (ldx) of type x_dtype, as the forward hook delivers them (quant.py:79-81 lets the model
 *        run in float16, bfloat16 or float32):
 *          MQ_DT_BF16 / MQ_DT_F16 : read as they are by the 16-bit matrix cores -- the products of two such values
 *                                   are exact in fp32, the same terms the reference sums after its up-cast;
 *                                   C and ldx even, X 4-byte aligned;
 *          MQ_DT_F32              : upper tiles of the fp32 GEMM core (fp32-accurate products), no workspace.
 *        n == 0 just scales H by beta.
 *   workspace: mq_hessian_syrk_workspace_bytes(n, C) bytes, 16-byte aligned: partial tiles of token ranges when the
 *        tile count alone does not fill the GPU, and, for wide Hessians with many 16-bit tokens (n >= 4096, C >= 4096),
 *        room for the tokens re-laid out for the matrix cores (see mq_pack_tokens below), which the call then does itself.
 * mq_hessian_syrk_bf16 is the same call with x_dtype = MQ_DT_BF16.
 */
size_t mq_hessian_syrk_workspace_bytes(int n, int C);
int mq_hessian_syrk(float* H, long ldh, const void* X, int x_dtype, long ldx, int n, int C, float beta, float alpha,
                    int mirror, void* workspace, size_t workspace_bytes, void* stream);
int mq_hessian_syrk_bf16(float* H, long ldh, const void* X, long ldx, int n, int C, float beta, float alpha,
                         int mirror, void* workspace, size_t workspace_bytes, void* stream);

/* The same accumulation for `groups` independent Hessians of one width C in one call (the experts of an MoE
 * block: the reference loops over forward hooks, one addmm_ per expert, src/gptq.py:97-103 via quant.py:258-277).
 * H, ldh, X, ldx, n, beta, alpha are HOST arrays with one entry per problem; the device pointers they hold follow
 * the rules above; all X share x_dtype.  When every problem has 16-bit tokens, n >= 256 of them and 16-byte aligned
 * rows, up to 16 problems share a launch (wide problems with many tokens are re-laid out into the workspace first, one
 * after another); otherwise each problem runs as a plain mq_hessian_syrk call with the given workspace
 * (mq_hessian_syrk_grouped_workspace_bytes = the larger of the largest single requirement and the sum of the re-laid
 * out copies).  mq_hessian_syrk_bf16_grouped is the same call with x_dtype = MQ_DT_BF16. */
size_t mq_hessian_syrk_grouped_workspace_bytes(int groups, const int* n, int C);
int mq_hessian_syrk_grouped(int groups, float* const* H, const long* ldh, const void* const* X, int x_dtype,
                            const long* ldx, const int* n, int C, const float* beta, const float* alpha, int mirror,
                            void* workspace, size_t workspace_bytes, void* stream);
int mq_hessian_syrk_bf16_grouped(int groups, float* const* H, const long* ldh, const void* const* X, const long* ldx,
                                 const int* n, int C, const float* beta, const float* alpha, int mirror, void* workspace,
                                 size_t workspace_bytes, void* stream);

/* The same accumulation on tokens that were copied anyway and therefore laid out for the matrix cores by the copy
 * (replaces the same src/gptq.py:97-103 product; the copies it rides on are the per-expert token gather of the block
 * forward, quant.py:280-281, and the output of the SiLU product that feeds down_proj, mq_swiglu_packed below):
 *   packed layout  Xp[o][c][j] = X[8 o + j][c]:  o = token octet, c = channel padded with zeros to a multiple of 256,
 *   j = 0..7; tokens padded with zeros to a multiple of 128; mq_packed_tokens_bytes(n, C) bytes, 16-byte aligned.
 *   mq_pack_tokens writes it from token-major 16-bit X (C and ldx multiples of 8, 16-byte aligned); rows != NULL
 *   (device array of n int64 row indices) gathers X[rows[t]] in the same pass; Xg != NULL also receives the gathered
 *   rows token-major (n x C, ldg), for the GEMMs of the model's own forward.
 *   mq_hessian_syrk_packed reads it: H as in mq_hessian_syrk, n >= 1 real tokens, workspace of
 *   mq_hessian_syrk_packed_workspace_bytes(n, C) bytes.  mq_hessian_syrk_packed_grouped: `groups` problems of one
 *   width in one call (host arrays as in mq_hessian_syrk_grouped; no workspace). */
size_t mq_packed_tokens_bytes(int n, int C);
int mq_pack_tokens(const void* X, int x_dtype, long ldx, const long* rows, int n, int C, void* Xp, void* Xg, long ldg,
                   void* stream);
size_t mq_hessian_syrk_packed_workspace_bytes(int n, int C);
int mq_hessian_syrk_packed(float* H, long ldh, const void* Xp, int x_dtype, int n, int C, float beta, float alpha,
                           int mirror, void* workspace, size_t workspace_bytes, void* stream);
int mq_hessian_syrk_packed_grouped(int groups, float* const* H, const long* ldh, const void* const* Xp, int x_dtype,
                                   const int* n, int C, const float* beta, const float* alpha, int mirror, void* stream);

/* lower triangle <- transpose of the upper triangle (what mirror != 0 does after the accumulation; exported so
 * that a caller accumulating many batches can mirror once at the end). */
int mq_symmetrize_upper(float* H, long ldh, int C, void* stream);

/* ---- (1b) Hessian hygiene before the factorisation ---------------------------------------------------
 * Device-side restatement of the Hessian part of GPTQ.quantization_pre_step, src/gptq.py:140-146:
 *   `if torch.isnan(self.H).any().item(): self.H = torch.eye(...)`, `pruned_ids = torch.diag(self.H) == 0`,
 *   `self.H[pruned_ids, pruned_ids] = 1`.  The reference reads the NaN verdict back to the host; here it
 *   stays in `flags`, so nothing synchronises.
 *   upper_only : 1 = H holds only its upper triangle (what mq_hessian_syrk_bf16 leaves with mirror == 0);
 *                the lower triangle is written here as its mirror image.  0 = H is full, only scanned.
 *   pruned : out, C bytes, 1 where diag(H) was 0 (the caller treats those weight columns as zero,
 *            `self.W[:, pruned_ids] = 0`, src/gptq.py:152).
 *   flags  : out, int32[4]: [0] != 0 when H held a NaN and was replaced by the identity, [1] = number of
 *            pruned channels; [2] is written by mq_hessian_damp; [3] unused.
 */
int mq_hessian_prestep(float* H, long ldh, int C, int upper_only, uint8_t* pruned, int* flags, void* stream);

/* Device-side restatement of the regularisation in GPTQ._get_hessian_inverse, src/gptq.py:221-234:
 *   `zero_cols = torch.nonzero(w.eq(0).all(dim=0))`, `H[zero_cols, :] = 0`, `H[:, zero_cols] = 0`,
 *   `H[zero_cols, zero_cols] = 1`, `damp = rel_damp * torch.diag(H).mean()`, `H[diag] += damp`.
 *   W      : R x C weights (ldw) of type w_dtype, read only; column c counts as zero when every entry is +-0
 *            or pruned[c] != 0 (pruned nullable).  Column indices of W address rows/columns of H as they are,
 *            as the reference does (also after an activation-order permutation of H).
 *   flags  : the array mq_hessian_prestep wrote; [2] receives the number of cleared channels.
 *   workspace : mq_hessian_damp_workspace_bytes(C) bytes.
 */
size_t mq_hessian_damp_workspace_bytes(int C);
int mq_hessian_damp(float* H, long ldh, int C, const void* W, int w_dtype, long ldw, int R, const uint8_t* pruned,
                    float rel_damp, int* flags, void* workspace, size_t workspace_bytes, void* stream);

/* Activation order: Hp[i, j] = H[perm[i], perm[j]].  Replaces `self.H = self.H[perm][:, perm]`, src/gptq.py:187
 * (perm = argsort(diag(H), descending), src/gptq.py:181), in one pass and without the intermediate the two chained
 * gathers build.  H (C x C, ldh) is read only, Hp (C x C, ldp) must not alias it; perm: C int32 on the device.
 * C <= 40960 (a source row passes through LDS), otherwise MQ_ERR_TOO_LARGE. */
int mq_permute_symmetric(const float* H, long ldh, const int* perm, float* Hp, long ldp, int C, void* stream);

/* mq_hessian_damp without a workspace argument and without any allocation.  It has no counterpart in MoE-Quant: it
 * exists for callers that cannot allocate or pass scratch memory -- code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  Same arguments, same kernels and bit-identical results; the scratch area
 * (per-strip masks, dead-channel mask, damping scalar) is a device array inside the library, one copy per GPU, held
 * until the process ends (17 * 32768 + 16 bytes, about 0.53 MiB).
 *   Limit  : C <= 32768, otherwise MQ_ERR_TOO_LARGE and nothing is launched.
 *   Sharing: every call on one GPU uses that GPU's one array: calls that overlap in time on one GPU (different
 *            streams or host threads) race and must be serialised by the caller.  Nothing in the array needs to be
 *            cleared between calls.
 *   The first call on each device looks the array's address up (hipGetSymbolAddress); make that call outside
 *   stream capture. */
int mq_hessian_damp_noalloc(float* H, long ldh, int C, const void* W, int w_dtype, long ldw, int R,
                            const uint8_t* pruned, float rel_damp, int* flags, void* stream);

/* ---- (2) damped Cholesky / Cholesky-inverse -------------------------------------------------------
 * In place: A (SPD, upper triangle read, C % 128 == 0) -> unit-diagonal upper-triangular
 * U = chol(A^-1, upper) / diag, strictly lower part zeroed.  Replaces
 * `linalg_utils.inv_sym` (src/linalg_utils.py:8-12) + `torch.linalg.cholesky(H, upper=True)` +
 * `H_inv_cho.div_(H_inv_cho.diag()[:, None])` in GPTQ._get_hessian_inverse, src/gptq.py:236-242.
 *   normalize : 1 = rows divided by the diagonal (what the GPTQ loop wants); 0 = plain R^-1 = chol(A^-1, upper),
 *          from which inv_sym assembles A^-1 = R^-T R^-1.
 *   info : one device int, must be 0 on entry; a non-positive/NaN pivot stores its 1-based index
 *          (the torch path raises LinAlgError there and the caller falls back to identity,
 *          src/gptq.py:239-240).  When info != 0 the output is the identity matrix: that fallback, taken on
 *          the device so that the caller need not read info back before queueing the loop.
 */
int mq_factor_upper_inverse(float* A, long ld, int C, int normalize, int* info, void* stream);
/* The same with the input left untouched, as the torch calls it replaces leave self.H (src/gptq.py:236-242 build
 * H_inv_cho in new tensors): H (upper triangle read, pitch ldh) -> U in A (pitch lda), A != H, A's contents on
 * entry irrelevant.  The first elimination step reads from H what later steps find in A, so no copy is made.
 */
int mq_factor_upper_inverse_from(const float* H, long ldh, float* A, long lda, int C, int normalize, int* info,
                                 void* stream);

/* `groups` matrices of one size C in one sequence of launches: the experts of an MoE block, which the reference
 * factors one after another inside its per-linear loop (quant.py:291-386 calling src/gptq.py:236-242).  One
 * factorisation is a chain of ~2 C/128 dependent launches with a one-workgroup step on its critical path and cannot
 * fill the GPU; here every launch carries that step's work for all matrices, so the chain is paid once per call.
 *   H, A, info : HOST arrays of `groups` device pointers (H[e] != A[e] for all e, or H[e] == A[e] for all e: in place);
 *   ldh, lda, C, normalize : shared.  Results are bit-identical to `groups` separate calls.
 *   Up to 16 matrices share a launch sequence; more run as consecutive batches. */
int mq_factor_upper_inverse_grouped(int groups, const float* const* H, long ldh, float* const* A, long lda, int C,
                                    int normalize, int* const* info, void* stream);

/* Cholesky-only factorisation for the loop in its inverse-free form (mq_gptq_loop_chol).  Replaces the same torch calls
 * as mq_factor_upper_inverse (src/linalg_utils.py:8-12, src/gptq.py:236-242) at half the flop: with H = R R^T, R upper,
 * the factor of the inverse is U = R^-1, and the loop's recurrence  x_k = w_k + sum_{j<k} e_j U[j,k]/U[j,j]  (e_j the
 * quantization error of column j, src/gptq_loop.py:141-148) is the same as
 *     x_k = w_k - (1/R_kk) sum_{j<k} z_j R[j,k],    z_j = dequantized minus ORIGINAL weight of column j,
 * so R^-1 is never needed.  Output: F[j,k] = -R[j,k] / R[k,k] for k > j; the diagonal and the lower triangle of F hold
 * no defined values (the loop reads k > j only).  info and the identity fallback (F = 0 above the diagonal) as above.
 *   H, F, info, workspace : as in mq_factor_upper_inverse_from; workspace = mq_factor_chol_workspace_bytes(C) bytes per
 *   matrix (the 128x128 diagonal blocks of R), 16-byte aligned.  _grouped: HOST arrays of `groups` device pointers,
 *   one launch sequence for up to 16 matrices at a time, results bit-identical to separate calls. */
size_t mq_factor_chol_workspace_bytes(int C);
int mq_factor_chol(const float* H, long ldh, float* F, long ldf, int C, int* info, void* workspace, size_t workspace_bytes,
                   void* stream);
int mq_factor_chol_grouped(int groups, const float* const* H, long ldh, float* const* F, long ldf, int C, int* const* info,
                           void* const* workspace, size_t workspace_bytes, void* stream);

/* ---- (3) quantization grid and column loop ---------------------------------------------------------
 * Symmetric per-group scales.  Replaces find_quantization_meta (symmetric branch) as called from
 * get_quantization_grid, src/quant_utils.py:75-96,213-220:
 *   scale = round_to(round_dtype)((2/maxq) * max|w| + 1e-12) over each group of `group_size` columns.
 *   W : R x C (w_dtype, ldw); dead_cols (nullable, C bytes): columns treated as zero (src/gptq.py:152).
 *   scale_rg : R x G fp32 out;  scale_gr (nullable): the same values transposed, G x R.
 */
int mq_quant_grid_sym(const void* W, int w_dtype, long ldw, int R, int C, int group_size, int bits,
                      const uint8_t* dead_cols, int round_dtype, float* scale_rg, float* scale_gr, void* stream);

/* Scale search on top of the scales above.  Replaces mse_scale / mse_scale_triton_kernel, src/quant_utils.py:104-192,
 * as called from get_quantization_grid, :221-232 (QuantizationScale.MSE):
 *   for every (row, group): candidates s_i = round_to(round_dtype)(scale * p[i]), i < P <= 256;
 *   loss_i = sum over the group of |dq_i(q_i(w)) - w|^norm with q = clamp(floor(w/s_i + qzero + 0.5), 0, maxq),
 *   dq = round_to(round_dtype)((q - qzero) * s_i);  scale <- s_best, best = the LAST index of minimal loss
 *   (tl.argmin(..., tie_break_left=False)).
 *   p : P fp32 shrink factors on the device (the reference builds them with torch.linspace(1, 0.2, 100)).
 *   scale_rg : R x G fp32, in (from mq_quant_grid_sym) and out;  scale_gr (nullable): transposed copy, G x R.
 */
int mq_mse_scale_sym(const void* W, int w_dtype, long ldw, int R, int C, int group_size, const uint8_t* dead_cols,
                     const float* p, int P, float qzero, float maxq, float norm, int round_dtype, float* scale_rg,
                     float* scale_gr, void* stream);

/* Wt[j, r] = fp32(W[r, perm[j]]), 0 for dead columns.  Replaces `self.W.clone().float()`,
 * `self.W[:, pruned_ids] = 0` (src/gptq.py:149-152) and `self.W.transpose(-2, -1)[perm]` (src/gptq.py:192).
 * perm nullable = identity. */
int mq_prepare_wt(const void* W, int w_dtype, long ldw, int R, int C, const int* perm, const uint8_t* dead_cols,
                  float* Wt, long ldwt, void* stream);

/* mq_prepare_wt writing the same values twice (Wt2 nullable): the inverse-free loop updates one copy in place and
 * reads the original weights from the other. */
int mq_prepare_wt_pair(const void* W, int w_dtype, long ldw, int R, int C, const int* perm, const uint8_t* dead_cols,
                       float* Wt, float* Wt2, long ldwt, void* stream);

/* The blocked GPTQ loop.  Replaces gptq_loop / gptq_loop_graph with both Triton kernels and the per-block
 * addmm_, src/gptq_loop.py:12-40,68-88,141-148.
 *   Wt    : C x R fp32 (ldw), in/out: original (permuted) weights in, dequantized weights out.
 *   U     : C x C fp32 (ldu), unit-diagonal upper factor from mq_factor_upper_inverse (only k > j read).
 *   scale : scale of (column j, row r) is scale[srow*ld_scale + r] with srow = scale_row ? scale_row[j] : j,
 *           so both the replicated C x R array of the reference and a compact G x R array work.
 *   qzero : nullable, same indexing; NULL means the constant qzero_const.
 *   round_dtype : rounding of the dequantized value ((q - z) * s), the `dtype` of tl_dequantize.
 *   block : columns per lazy-batch block; values <= 0 or > 128 use 128 (only reassociates fp32 sums).
 *   Qt    : C x R u8 out, integer codes.   E : mq_gptq_loop_scratch_bytes(R) bytes of scratch (a ring of sixteen
 *           128 x R fp32 error blocks: a block's sequential walk overlaps the trailing update of a batch of up to
 *           eight blocks before it).
 */
size_t mq_gptq_loop_scratch_bytes(int R);
int mq_gptq_loop(float* Wt, long ldw, int C, int R, const float* U, long ldu, const float* scale, long ld_scale,
                 const int* scale_row, const float* qzero, float qzero_const, float maxq, int round_dtype, int block,
                 uint8_t* Qt, float* E, void* stream);

/* The loop for `groups` linears of one shape (C, R, pitches, block, rounding and qzero_const shared) in one sequence
 * of launches: every launch carries one block's column walk and trailing tiles for all of them (the reference runs
 * its experts one after another, quant.py:291-386).  Wt, U, scale, scale_row, qzero, Qt, E: HOST arrays of `groups`
 * device pointers, each as in mq_gptq_loop; scale_row / qzero may be NULL, otherwise their entries are all NULL or
 * all set.  Every linear needs its own E ring.  Results are bit-identical to `groups` separate calls.
 * Up to 16 linears share a launch sequence; more run as consecutive batches. */
int mq_gptq_loop_grouped(int groups, float* const* Wt, long ldw, int C, int R, const float* const* U, long ldu,
                         const float* const* scale, long ld_scale, const int* const* scale_row,
                         const float* const* qzero, float qzero_const, float maxq, int round_dtype, int block,
                         uint8_t* const* Qt, float* const* E, void* stream);

/* The same loop (src/gptq_loop.py:12-40,68-88,141-148) in its inverse-free form: F from mq_factor_chol in U's place,
 * and W0t, a read-only copy of the original Wt (mq_prepare_wt_pair), from which every column computes its total change
 * z = y - w_original, the quantity handed on to later columns in place of the quantization error.  Same outputs as
 * mq_gptq_loop on the corresponding U up to fp32 rounding; E holds z blocks.  _grouped as mq_gptq_loop_grouped. */
int mq_gptq_loop_chol(float* Wt, const float* W0t, long ldw, int C, int R, const float* F, long ldf, const float* scale,
                      long ld_scale, const int* scale_row, const float* qzero, float qzero_const, float maxq,
                      int round_dtype, int block, uint8_t* Qt, float* E, void* stream);
int mq_gptq_loop_chol_grouped(int groups, float* const* Wt, const float* const* W0t, long ldw, int C, int R,
                              const float* const* F, long ldf, const float* const* scale, long ld_scale,
                              const int* const* scale_row, const float* const* qzero, float qzero_const, float maxq,
                              int round_dtype, int block, uint8_t* const* Qt, float* const* E, void* stream);

/* codes[r, c] = Qt[perm_inv[c], r].  Replaces `[perm_inv].transpose(-2, -1).contiguous().to(torch.uint8)`,
 * src/gptq.py:199.  perm_inv nullable = identity. */
int mq_untranspose_codes(const uint8_t* Qt, int R, int C, const int* perm_inv, uint8_t* codes, long ldc,
                         void* stream);

/* ---- (4) int4 -> int32 packing (compressed_tensors "pack-quantized" layout) -------------------------
 * word[r, k] = sum_{i<8} ((codes[r, 8k+i] - zero[r, (8k+i)/g] + 8) & 15) << 4i, columns past C pack as 0.
 * Replaces pack_weight's `qweight.to(int8) - zero...` + compressed_tensors.pack_to_int32(., 4),
 * pack_quantized_model.py:66-67.   zero (R x G fp32) nullable = 8 everywhere (symmetric).
 * out : R x ceil(C/8) int32 (ldo).
 */
int mq_pack_int4(const uint8_t* codes, long ldc, int R, int C, const float* zero, int group_size, int32_t* out,
                 long ldo, void* stream);

/* Same words, straight from the loop's transposed codes (symmetric, zero = 8): fuses mq_untranspose_codes
 * and mq_pack_int4 so the codes are read once. */
int mq_pack_from_qt(const uint8_t* Qt, int R, int C, const int* perm_inv, int32_t* out, long ldo, void* stream);

/* ---- building block, exported for tests -----------------------------------------------------------
 * C[m,n] = beta*C[m,n] + alpha * sum_k A(m,k) B(k,n) on the fp32 matrix cores; A(m,k) = A[m*sam + k*sak]
 * (one of sam/sak must be 1), B(k,n) = B[k*sbk + n*sbn] likewise.  tri != 0: only 128x128 tiles on or above
 * the block diagonal.  ktrim: 0 full K, 1 K < end of the row tile, 2 K >= start of the row tile. */
int mq_gemm_f32(const float* A, long sam, long sak, const float* B, long sbk, long sbn, float* C, long ldc, int M,
                int N, int K, float alpha, float beta, int tri, int ktrim, void* stream);

/* ---- checkpoint ingest: FP8 weights with per-128x128-block inverse scales -> bf16 / fp16 -------------------
 * Replaces `W.to(dtype)`, `s.to(dtype)` and dequantize_weight_from_fp8, src/quant_utils.py:267-296, in one pass:
 *   out[r, c] = round_to(out_dtype)( e4m3fn(W[r, c]) * round_to(out_dtype)(scale_inv[r/128, c/128]) ).
 *   W : R x C bytes (ldw), OCP e4m3fn (torch.float8_e4m3fn); scale_inv : ceil(R/128) x ceil(C/128) fp32 (ld_scale);
 *   out : R x C 16-bit floats (ldo), out_dtype = MQ_DT_BF16 or MQ_DT_F16.  No padding is needed for ragged edges.
 */
int mq_dequant_fp8_block(const uint8_t* W, long ldw, int R, int C, const float* scale_inv, long ld_scale, int out_dtype,
                         void* out, long ldo, void* stream);

/* ---- the step before GPTQ.update of a down projection: the expert's SwiGLU product ------------------------------
 * Replaces the elementwise part of the expert forward that feeds the down projection's hook (quant.py:280-281 runs the
 * block; an expert computes act_fn(gate_proj(x)) * up_proj(x)): out[r, j] = round(round(silu(GU[r, j])) * GU[r, I + j])
 * for GU (n x 2I, ldg) holding the gate projection's outputs followed by the up projection's (one GEMM against the
 * stacked weights), both roundings to `dtype` (MQ_DT_BF16 / MQ_DT_F16) as the chained torch ops round.
 *   I % 8 == 0, 16-byte aligned rows; out : n x I (ldo). */
int mq_swiglu(const void* GU, long ldg, int n, int I, int dtype, void* out, long ldo, void* stream);
/* The same product (same roundings) written straight into the packed-token layout mq_hessian_syrk_packed reads
 * (mq_packed_tokens_bytes(n, I) bytes): its only reader is the down projection's Hessian.  G, U: the gate and the up
 * projection's outputs, n x I each (ldg, ldu) -- two matrices or the two halves of one stacked GEMM output. */
int mq_swiglu_packed(const void* G, long ldg, const void* U, long ldu, int n, int I, int dtype, void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOEQUANT_HIP_H */
