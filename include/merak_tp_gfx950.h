/*
 * merak_tp_gfx950 — C ABI of the gfx950 (MI355X) kernels behind Merak's
 * Megatron-style tensor-parallel layers.
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream
 * (hipStream_t passed as void*; NULL = the null stream).  Nothing here
 * allocates, frees or synchronises: the caller owns every buffer, and
 * the kernels are enqueued on `stream` and return immediately.
 *
 * Return value: 0 on success, a negative MTP_E* code otherwise.  After a
 * failure mtp_last_error() returns a thread-local, human readable reason.
 * The library is re-entrant (backward passes call it from PyTorch's autograd
 * worker thread while forward runs on the main thread).  What it keeps
 * between calls, all of it guarded:
 *   - the thread-local error string;
 *   - the values of the MTP_* tuning variables, read from the environment at
 *     first use and again on mtp_reload_tuning() (one list, behind a mutex;
 *     the values are atomics);
 *   - for mtp_gemv_argmax_noalloc only: a 4 MiB file-scope device array per
 *     GPU and the table of its per-device addresses (filled once per device
 *     under a mutex).  Calls of that entry point that overlap on one GPU
 *     share the array and race; no other entry point touches it.
 *
 * File:line citations name the interface in the reference tree
 * (HPDL-Group/Merak) that each entry point stands in for.
 */
#ifndef MERAK_TP_GFX950_H
#define MERAK_TP_GFX950_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MTP_ABI_VERSION 12

/* element types.  MTP_F16 is IEEE half, what the reference's --fp16 sets as
 * params_dtype (Merak/merak_args/args.py:584-585). */
#define MTP_F32  0
#define MTP_BF16 1
#define MTP_F16  2

/* error codes */
#define MTP_OK            0
#define MTP_EINVAL       -1   /* bad argument (null pointer, negative size, unknown enum) */
#define MTP_EUNSUPPORTED -2   /* shape/alignment the kernels do not cover */
#define MTP_EDEVICE      -3   /* current device is not gfx950, or a HIP call failed */
#define MTP_EWORKSPACE   -4   /* workspace too small */

/* epilogues of mtp_linear_fwd / mtp_gemv */
#define MTP_EPI_NONE      0   /* Y = X W^T                                   */
#define MTP_EPI_BIAS      1   /* Y = X W^T + b                               */
#define MTP_EPI_BIAS_GELU 2   /* Y = X W^T + b ; ACT = gelu_new(Y)           */
#define MTP_EPI_SWIGLU    3   /* Y = X W^T (+ b); ACT = silu(Y[:, :N/2]) * Y[:, N/2:] */
#define MTP_EPI_GELU      4   /* Y = X W^T ; ACT = gelu_new(Y)               */

int         mtp_abi_version(void);
const char* mtp_last_error(void);

/* Name of the gfx architecture of the current HIP device ("gfx950"), written
 * into buf (NUL terminated, truncated to len).  MTP_EDEVICE if no device. */
int mtp_device_arch(char* buf, int len);

/* ------------------------------------------------------------------------
 * Linear layers.  All matrices are row-major and dense (leading dimension
 * = number of columns).  dtype (f32, bf16 or f16) is the element type of X,
 * W, Y, dY, dX and bias; accumulation is always fp32.
 * ------------------------------------------------------------------------ */

/* Y[M,N] = X[M,K] W[N,K]^T (+ bias[N]) with an optional fused activation.
 * Replaces F.linear in ColumnParallelLinear.forward
 * (Merak/core/mpu/layers.py:251-252) and RowParallelLinear.forward
 * (layers.py:354 and the "+ bias" of :357-358, which at tensor-parallel
 * world size 1 follows an identity reduce), plus the elementwise activation
 * HF applies between the two (gelu_new for GPT-2, silu(gate)*up for Llama).
 *
 *  y   : [M,N] pre-activation output; may be NULL when an activation
 *        epilogue is selected and the caller does not need it.
 *  act : activation output, required for *_GELU ([M,N]) and SWIGLU
 *        ([M,N/2]); must be NULL otherwise.
 *  bias: [N] or NULL (required for MTP_EPI_BIAS, MTP_EPI_BIAS_GELU). */
int mtp_linear_fwd(const void* x, const void* w, const void* bias,
                   void* y, void* act,
                   int64_t M, int64_t N, int64_t K,
                   int dtype, int epilogue, void* stream);

/* dX[M,K] = dY[M,N] W[N,K]  — the input gradient autograd derives for
 * F.linear (entered from loss.backward(), Merak/core/merak_engine.py:926;
 * at world size 1 the all-reduce of _CopyToModelParallelRegion.backward,
 * Merak/core/mpu/mappings.py:320, is the identity). */
int mtp_linear_dgrad(const void* dy, const void* w, void* dx,
                     int64_t M, int64_t N, int64_t K,
                     int dtype, void* stream);

/* dW[N,K] (+)= dY[M,N]^T X[M,K]; db[N] (+)= sum_m dY[m,:]  — the weight and
 * bias gradients of F.linear.  dw_dtype selects the element type of dW and
 * db: dtype itself, or MTP_F32 (an fp32 main gradient); accumulate != 0
 * adds into the existing contents instead of overwriting.  db may be NULL. */
int mtp_linear_wgrad(const void* dy, const void* x, void* dw, void* db,
                     int64_t M, int64_t N, int64_t K,
                     int dtype, int dw_dtype, int accumulate, void* stream);

/* db[N] (+)= sum_m dY[m,:] alone: the bias gradient of F.linear for a layer
 * whose weight takes no gradient (otherwise mtp_linear_wgrad delivers it with
 * dW in one launch).  db_dtype: dtype or MTP_F32.  M == 0 writes zeros. */
int mtp_linear_bias_grad(const void* dy, void* db, int64_t M, int64_t N,
                         int dtype, int db_dtype, int accumulate, void* stream);

/* The three products above with device scratch.  On the 16-bit path a product
 * whose 256x256 tiling would leave much of the last round of workgroups idle
 * (few tiles with a long reduction: one rank's narrow shard of a wide layer)
 * is cut "stream-K" fashion: the k range of the tiles of that round is dealt
 * evenly to all compute units, the parts of a tile shared by several workgroups
 * meet in the scratch and a second small kernel adds them up in k order and
 * writes the tile, so results are reproducible bit for bit from run to run
 * (they may differ in the last bit from the call without scratch, which sums
 * each tile in one piece).  On the fp32 path a product with fewer 128x128
 * output tiles than compute units and a long reduction (a weight gradient) is
 * cut into up to 8 slices along k, one workgroup per tile and slice; the
 * slices meet in the scratch and a second kernel adds them in slice order
 * (reproducible bit for bit as well); it takes a scratch of any size and cuts
 * only when the slices fit.
 * workspace: 16-byte aligned, mtp_linear_workspace_bytes() bytes (about 138 MB,
 * shape independent); its contents on entry do not matter.  Launches that
 * share a workspace must not overlap (one workspace per stream).  NULL or too small:
 * exactly the call without scratch.  The reference has no counterpart (its
 * F.linear at layers.py:252,354 leaves such choices to the BLAS library). */
int64_t mtp_linear_workspace_bytes(void);
/* Bytes of scratch a product of a layer with these sizes (M tokens, N output
 * features, K input features) can make use of — kind 0 forward, 1 input
 * gradient, 2 weight gradient, 3 both gradients — or 0 if it never touches
 * the scratch (most shapes): lets a caller allocate only when it pays.  Never
 * more than mtp_linear_workspace_bytes() on the 16-bit path. */
int64_t mtp_linear_workspace_need(int kind, int64_t M, int64_t N, int64_t K, int dtype);
int mtp_linear_fwd_ws(const void* x, const void* w, const void* bias,
                      void* y, void* act, void* workspace, int64_t workspace_bytes,
                      int64_t M, int64_t N, int64_t K,
                      int dtype, int epilogue, void* stream);
int mtp_linear_dgrad_ws(const void* dy, const void* w, void* dx,
                        void* workspace, int64_t workspace_bytes,
                        int64_t M, int64_t N, int64_t K, int dtype, void* stream);
int mtp_linear_wgrad_ws(const void* dy, const void* x, void* dw, void* db,
                        void* workspace, int64_t workspace_bytes,
                        int64_t M, int64_t N, int64_t K,
                        int dtype, int dw_dtype, int accumulate, void* stream);

/* Input gradient and weight gradient of one layer, dX = dY W and dW (+)= dY^T X
 * (db likewise, may be NULL), what autograd derives for F.linear at
 * layers.py:252,354 — the two calls above as one.  Where both products run on
 * the 64-deep bf16 / fp16 loop and their 256x256 tiles together fill fewer
 * rounds of 256 workgroups than apart (896 + 896 tiles: 7 rounds instead of
 * 4 + 4), they go out as ONE launch; the results are those of mtp_linear_dgrad
 * + mtp_linear_wgrad to the rounding order of the sums (another tile
 * configuration may serve a product there), and the same bits on every run.
 * In every other case it is those two calls, one after the other.  Same
 * workspace rules. */
int mtp_linear_bwd_ws(const void* dy, const void* x, const void* w,
                      void* dx, void* dw, void* db,
                      void* workspace, int64_t workspace_bytes,
                      int64_t M, int64_t N, int64_t K,
                      int dtype, int dw_dtype, int accumulate, void* stream);

/* Backward of the fused activations: given dACT and the saved
 * pre-activation Y, writes dY.
 *   MTP_EPI_BIAS_GELU / MTP_EPI_GELU: dY[M,N]   = dACT[M,N] * gelu_new'(Y)
 *   MTP_EPI_SWIGLU:                   dY[M,N]   from dACT[M,N/2], Y=[gate|up]
 * dy may alias dact only for the GELU forms. */
int mtp_activation_bwd(const void* dact, const void* y, void* dy,
                       int64_t M, int64_t N, int dtype, int epilogue,
                       void* stream);

/* ------------------------------------------------------------------------
 * Vocab-parallel embedding (Merak/core/mpu/layers.py:145-165).
 * out[i,:] = table[ids[i]-vocab_start,:] if vocab_start <= ids[i] < vocab_end
 *            else 0                         (layers.py:148-152,162)
 * row_bytes = embedding_dim * element size; any value >= 1 is accepted
 * (wider vector copies are used when table, out and row_bytes are 16/8/4
 * byte aligned).  oob_count (device int32, may be NULL) is incremented once
 * per id outside [vocab_start, vocab_end).
 * ------------------------------------------------------------------------ */
int mtp_embedding_gather(const int64_t* ids, const void* table, void* out,
                         int64_t n_ids, int64_t row_bytes,
                         int64_t vocab_start, int64_t vocab_end,
                         int32_t* oob_count, void* stream);

/* Dense gradient of the lookup: dtable[ids[i]-vocab_start,:] += dout[i,:]
 * for in-range ids; dtable is [rows,dim] of dtable_dtype (fp32, or the
 * 16-bit dtype of dout).  This is the embedding_dense_backward ATen runs behind
 * F.embedding (layers.py:156).  Tokens that share an id are summed in fp32 in
 * an order fixed by the ids alone (ascending token order; an id carried by
 * more than 32 tokens: ascending inside blocks of 32 of its tokens, the block
 * sums ascending inside blocks of 32 blocks, then those in ascending order)
 * and added to the table row once, so the result is reproducible bit for
 * bit, and the longest dependent chain is 64 + count/1024 steps however many
 * tokens share an id (a padded batch).  The
 * caller zeroes dtable first unless it wants accumulation, e.g. onto the
 * LM-head weight gradient when the two are tied
 * (Merak/core/pipeline/module.py:646-662).  workspace: device scratch of
 * mtp_embedding_bwd_workspace_bytes(n_ids, dim) bytes, 16-byte aligned. */
int64_t mtp_embedding_bwd_workspace_bytes(int64_t n_ids, int64_t dim);
int mtp_embedding_bwd(const int64_t* ids, const void* dout, void* dtable,
                      void* workspace, int64_t workspace_bytes,
                      int64_t n_ids, int64_t dim, int dtype, int dtable_dtype,
                      int64_t vocab_start, int64_t vocab_end, void* stream);

/* ------------------------------------------------------------------------
 * Vocab-parallel cross entropy (Merak/core/mpu/cross_entropy.py:29-106).
 * logits: [n_rows, vocab] contiguous, this rank's vocab slice
 * [vocab_start, vocab_start+vocab).  One pass, fp32 arithmetic.
 *
 *   row_max[i]    = max_j logits[i,j]                       (:32)
 *   row_sumexp[i] = sum_j exp(logits[i,j] - row_max[i])     (:70-71)
 *   pred[i]       = logits[i, t_i - vocab_start] if t_i in range else 0
 *                   (raw logit, not max-subtracted)          (:48-62)
 *   loss[i]       = log(row_sumexp[i]) - (pred[i]-row_max[i]) in range,
 *                   log(row_sumexp[i]) otherwise             (:77)
 * loss is the single-rank result; the three partials are what ranks would
 * exchange (MAX, SUM, SUM; :33,64,72).  Targets outside the range — -100
 * included — get no one-hot term, exactly as the reference's mask does.
 * The logits are NOT modified by the forward.
 * ------------------------------------------------------------------------ */
int mtp_vocab_ce_fwd(const void* logits, const int64_t* target,
                     float* loss, float* row_max, float* row_sumexp,
                     float* pred,
                     int64_t n_rows, int64_t vocab, int64_t vocab_start,
                     int dtype, void* stream);

/* In place: logits[i,j] <- (exp(logits[i,j]-row_max[i]) / row_sumexp[i]
 *                           - [j == t_i - vocab_start]) * grad_out[i]
 * (cross_entropy.py:86-106).  row_max / row_sumexp are the (globally
 * combined) values from the forward.  grad_out may be NULL (= 1 for every
 * row), which together with out-of-range targets yields the softmax the
 * reference leaves in the caller's logits after forward (:80).
 * row_max == row_sumexp == NULL means the buffer already holds that softmax
 * (the reference's backward, :92-104): logits[i,j] <- (logits[i,j] - onehot) * grad_out[i]. */
int mtp_vocab_ce_bwd(void* logits, const int64_t* target,
                     const float* row_max, const float* row_sumexp,
                     const float* grad_out,
                     int64_t n_rows, int64_t vocab, int64_t vocab_start,
                     int dtype, void* stream);

/* Forward and backward in one launch, for callers that know the upstream
 * gradient of the per-row losses before the forward runs (the trainer's
 * loss = mean(losses), Merak/merak_trainer.py:313-326, makes it 1/n_rows
 * times the loss scale).  Outputs as mtp_vocab_ce_fwd (cross_entropy.py:29-84),
 * and logits[i,j] <- (softmax[i,j] - onehot) * g_i as mtp_vocab_ce_bwd
 * (:92-104), with g_i = (grad_rows ? grad_rows[i] : 1) * grad_scale.  Each row
 * stays in registers between the two, so memory sees one read and one write
 * of the logits.  Rows longer than mtp_vocab_ce_fwd_bwd_max_vocab(dtype)
 * return MTP_EUNSUPPORTED (use the two calls above). */
int mtp_vocab_ce_fwd_bwd(void* logits, const int64_t* target,
                         const float* grad_rows, float grad_scale,
                         float* loss, float* row_max, float* row_sumexp, float* pred,
                         int64_t n_rows, int64_t vocab, int64_t vocab_start,
                         int dtype, void* stream);
int64_t mtp_vocab_ce_fwd_bwd_max_vocab(int dtype);

/* grad[i,:] *= grad_rows[i] / assumed for the rows where grad_rows[i] !=
 * assumed; rows where they are equal are not touched (no memory traffic).
 * Turns the gradient mtp_vocab_ce_fwd_bwd wrote for an assumed upstream
 * gradient into the one for the upstream gradient autograd delivers
 * (cross_entropy.py:103, grad_input.mul_(grad_output.unsqueeze(-1))). */
int mtp_vocab_ce_rescale(void* grad, const float* grad_rows, float assumed,
                         int64_t n_rows, int64_t vocab, int dtype, void* stream);

/* ------------------------------------------------------------------------
 * Decode step (Merak/inference/text_generation_inference.py:223,226-227):
 * a handful of single-token activation rows through a linear layer, and the
 * greedy pick over the LM-head row.  dtype bf16 or f16, B <= 32, K % 8 == 0.
 * ------------------------------------------------------------------------ */

/* Y[B,N] = X[B,K] W[N,K]^T (+bias) ; epilogue NONE, BIAS or SWIGLU
 * (SWIGLU: y is [B,N/2] = silu(gate)*up with W = [gate rows | up rows]).
 * y must not be x (every workgroup reads all of X). */
int mtp_gemv(const void* x, const void* w, const void* bias, void* y,
             int64_t B, int64_t N, int64_t K, int epilogue, int dtype, void* stream);

/* mtp_gemv with device scratch.  Matrices with few rows at B > 16 are cut
 * along k into slices that run as separate workgroups (each reads only its
 * part of X); the slices' partial sums meet in the workspace and are added
 * in slice order, so the result is reproducible.  workspace: 16-byte
 * aligned, mtp_gemv_workspace_bytes(B, N, K, epilogue) bytes (0 = this shape
 * is not cut; then workspace may be NULL).  ITS FIRST 8192 BYTES MUST BE
 * ZERO before the first launch that uses it; every launch leaves them zero,
 * whatever its shape, so one workspace (of the largest size any of them
 * asks for) serves launches of different shapes in turn.  Launches that
 * share a workspace must not overlap.  A NULL or too small workspace gives
 * mtp_gemv's uncut behaviour. */
int64_t mtp_gemv_workspace_bytes(int64_t B, int64_t N, int64_t K, int epilogue);
int mtp_gemv_ws(const void* x, const void* w, const void* bias, void* y,
                void* workspace, int64_t workspace_bytes,
                int64_t B, int64_t N, int64_t K, int epilogue, int dtype, void* stream);

/* Two products over the same activations in one call:
 *   y1   [B, N1]   = x W1^T (+ bias1)
 *   act2 [B, N2/2] = silu(G) * U, (G | U) = x W2^T (+ bias2), W2 = [gate rows | up rows]
 * — what a block whose QKV and gate/up projections read the same rows computes
 * (the decode step of Merak/inference/text_generation_inference.py:199-203 on
 * the linears of one block).  Where the second product fills the chip with one
 * workgroup per compute unit, both go out as one grid: the rows of the first
 * product ride as one or two more row groups in the loop of the second's
 * workgroups (or, above 16 batch rows, as a block in front of it), so that the
 * smaller product neither starts nor drains the chip on its own.  For other
 * shapes the call is the two launches of mtp_gemv_ws, with the same workspace
 * rules.  Results equal those of the separate calls to rounding (other orders
 * of the sums along k); above 16 batch rows act2 has the separate call's bits. */
int mtp_gemv_pair(const void* x, const void* w1, const void* bias1, void* y1, int64_t N1,
                  const void* w2, const void* bias2, void* act2, int64_t N2,
                  void* workspace, int64_t workspace_bytes,
                  int64_t B, int64_t K, int dtype, void* stream);

/* mtp_gemv_ws with what a decoder block puts around its linears (HF
 * LlamaDecoderLayer.forward: `residual + hidden_states`, LlamaRMSNorm in
 * front of the QKV and the gate/up projections), so that a block is five
 * launches and the normalised row is never stored:
 *   norm_weight != NULL: X is the residual stream and the product is taken
 *     with RMSNorm(X) = norm_weight * dtype(x * rsqrt(mean_k x^2 + eps));
 *     sumsq_in [B, K/16] fp32 holds the sums of squares of X per 16 elements
 *     (what sumsq_out of the producing call wrote).  Every workgroup keeps
 *     RMSNorm(X) in its LDS: K % 512 == 0, K <= 8192, B K <= 8 x 4096 elements
 *     (mtp_gemv_norm_fits(B, K) == 1); both pointers 16-byte aligned; the
 *     product is not cut along k.
 *   residual != NULL ([B,N], epilogue NONE or BIAS):
 *     y = dtype(dtype(W x + bias) + residual); y may be residual itself.
 *   sumsq_out != NULL ([B, ceil(N/16)] fp32, epilogue NONE or BIAS): sum of
 *     the squares of the stored y per batch row and 16 output rows.
 * All three NULL: exactly mtp_gemv_ws. */
int mtp_gemv_norm_fits(int64_t B, int64_t K);
int mtp_gemv_fused(const void* x, const void* w, const void* bias, void* y,
                   const void* norm_weight, const float* sumsq_in, float eps,
                   const void* residual, float* sumsq_out,
                   void* workspace, int64_t workspace_bytes,
                   int64_t B, int64_t N, int64_t K, int epilogue, int dtype, void* stream);

/* Bytes of device scratch mtp_gemv_argmax needs for this shape. */
int64_t mtp_gemv_argmax_workspace_bytes(int64_t B, int64_t N, int64_t K);

/* idx[b] = argmax_n (X[b,:] . W[n,:]) — first index among equal maxima, NaN
 * counts as the maximum (torch.argmax semantics, :227); maxval[b] (may be
 * NULL) receives the winning fp32 logit.  The [B,N] logits are never
 * written to memory.  "Equal" means equal as computed: rows handled by
 * different workgroups are summed along k in a different (fixed) order, so
 * two identical weight rows far apart may differ in the last bit. */
int mtp_gemv_argmax(const void* x, const void* w,
                    int64_t* idx, float* maxval,
                    void* workspace, int64_t workspace_bytes,
                    int64_t B, int64_t N, int64_t K, int dtype, void* stream);

/* mtp_gemv_argmax for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid it): the
 * scratch is an array inside the library, mtp_gemv_argmax_noalloc_max_bytes()
 * = 4 MiB per GPU, held until the process ends; a shape whose
 * mtp_gemv_argmax_workspace_bytes exceeds that returns MTP_EWORKSPACE.  No
 * call allocates or frees.  All calls on one GPU share that GPU's array:
 * calls that overlap on one GPU (different streams) race.  Nothing in the
 * array needs clearing between calls.  It has no counterpart in the
 * reference. */
int64_t mtp_gemv_argmax_noalloc_max_bytes(void);
int mtp_gemv_argmax_noalloc(const void* x, const void* w,
                            int64_t* idx, float* maxval,
                            int64_t B, int64_t N, int64_t K, int dtype, void* stream);

/* Row-wise argmax of materialised logits [B,V] (dtype f32, bf16 or f16): the
 * literal torch.argmax(logits, dim=-1) of :227. */
int mtp_argmax_rows(const void* logits, int64_t* idx,
                    int64_t B, int64_t V, int dtype, void* stream);

/* Sampling tail of the generation loop
 * (Merak/inference/text_generation_inference.py:229-235 with top_k_logits,
 * :35-69): z = float(logits)/temperature; top_k > 0 drops z below the k-th
 * largest; top_p > 0 drops, in descending order, every token whose
 * predecessors already hold more than top_p of the remaining softmax mass
 * (the first token always stays); then one token per row is drawn with
 * probability softmax(z kept).  The draw replaces torch.multinomial's private
 * random stream by the caller's uniforms[b] in [0,1): token = first index
 * whose cumulative kept probability, in index order, exceeds uniforms[b].
 * logits: [B,V] f32, bf16 or f16, untouched.  tokens (int64 [B]) and filtered
 * (f32 [B,V]: z where kept, -inf where dropped, what top_k_logits returns) may
 * each be NULL.  workspace: device scratch of mtp_sample_workspace_bytes(B)
 * bytes, 8-byte aligned (the rows are spread over many workgroups and the
 * passes of the selection are separate launches; their state lives there).
 * Same inputs give the same outputs bit for bit. */
int64_t mtp_sample_workspace_bytes(int64_t B);
int mtp_sample_top_k_top_p(const void* logits, int dtype, int64_t B, int64_t V,
                           float temperature, int top_k, float top_p,
                           const float* uniforms, int64_t* tokens, float* filtered,
                           void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * Single-position step with a key/value cache.  The reference's generation
 * loop re-runs the whole sequence for every new token and keeps one row of
 * the output (Merak/inference/text_generation_inference.py:199-203, row
 * picked at :223); for a causal model the same row comes from running only
 * the new position against cached keys and values.  These are the pieces
 * of the HF Llama block between the tensor-parallel linears; head_dim is
 * 128, dtype is bf16 or f16 (f32 too where stated).
 * ------------------------------------------------------------------------ */
/* h = x (+ residual, may be NULL), rounded to the tensor dtype;
 * residual_out (may be NULL) = h; y = weight * dtype(h * rsqrt(mean(h^2) +
 * eps)) with the mean and the scaling in fp32 (HF LlamaRMSNorm.forward in
 * front of which the block's `residual + hidden_states` has been folded).
 * x, residual, y, residual_out: [rows, dim]; weight: [dim]; dtype f32,
 * bf16 or f16.  y may alias x; residual_out may alias residual. */
int mtp_rmsnorm(const void* x, const void* residual, const void* weight,
                void* y, void* residual_out,
                int64_t rows, int64_t dim, float eps, int dtype, void* stream);

/* qkv: [B, (n_q_heads + 2 n_kv_heads) * 128], q heads first, then k, then v
 * (the fused QKV linear's output).  positions: int64 [B], position of the
 * new token of each row.  Rotary embedding x*cos + rotate_half(x)*sin (HF
 * apply_rotary_pos_emb) with cos/sin tables [max_positions, 128] of the
 * tensor dtype; rotated q -> q_out [B, n_q_heads, 128]; rotated k and plain
 * v -> row positions[b] of k_cache / v_cache [B, n_kv_heads, max_len, 128].
 * A row whose position lies outside the tables or the cache is left
 * unwritten (no fault). */
int mtp_rope_kv_append(const void* qkv, const void* cos_table, const void* sin_table,
                       const int64_t* positions, void* q_out, void* k_cache, void* v_cache,
                       int64_t B, int n_q_heads, int n_kv_heads, int head_dim,
                       int64_t max_len, int64_t max_positions, int dtype, void* stream);

/* out[b,h,:] = softmax_t(scale * q[b,h,:] . K[b,h/g,t,:]) V[b,h/g,t,:] over
 * t < lens[b] (int64 [B] on the device, clamped to [0, max_len]; a row with
 * no tokens gives zeros), g = n_q_heads / n_kv_heads <= 16: grouped-query
 * attention of one new position (HF eager attention: fp32 softmax,
 * probabilities rounded to the tensor dtype for the product with V).  len_bound: an
 * upper bound of lens known on the host (<= max_len); it only decides over
 * how many workgroups a sequence is split.  workspace: device scratch of
 * mtp_attn_decode_workspace_bytes(B, n_q_heads, n_kv_heads, len_bound)
 * bytes, 16-byte aligned (may be NULL when that is 0).  ITS FIRST
 * 4 * B * n_kv_heads BYTES MUST BE ZERO before the first launch that uses
 * it; every launch leaves them zero again (they count the splits of a
 * sequence that have delivered, the last one merges).  Launches that share a
 * workspace must not overlap. */
int64_t mtp_attn_decode_workspace_bytes(int64_t B, int n_q_heads, int n_kv_heads, int64_t len_bound);
int mtp_attn_decode(const void* q, const void* k_cache, const void* v_cache,
                    const int64_t* lens, void* out,
                    void* workspace, int64_t workspace_bytes,
                    int64_t B, int n_q_heads, int n_kv_heads, int head_dim,
                    int64_t max_len, int64_t len_bound, float scale, int dtype, void* stream);

/* mtp_rope_kv_append followed by mtp_attn_decode with lens = positions + 1,
 * as one launch: the new query and key are rotated in registers, the new
 * key and value are appended to the caches and enter the softmax straight
 * from the QKV projection's output; the cached rows below positions[b] are
 * read as in mtp_attn_decode.  A row whose position lies outside the cache
 * or the tables appends nothing and gives zeros.  len_bound bounds
 * positions + 1.  Same workspace rules. */
int mtp_attn_decode_append(const void* qkv, const void* cos_table, const void* sin_table,
                           const int64_t* positions, void* k_cache, void* v_cache, void* out,
                           void* workspace, int64_t workspace_bytes,
                           int64_t B, int n_q_heads, int n_kv_heads, int head_dim,
                           int64_t max_len, int64_t max_positions, int64_t len_bound,
                           float scale, int dtype, void* stream);

/* ------------------------------------------------------------------------
 * Measurement helpers (used by bench.py to state what this GPU can do).
 * ------------------------------------------------------------------------ */
/* The library reads its MTP_* tuning variables (tile and slice choices that
 * select among kernels computing the same result) from the environment once,
 * at their first use; no launch calls getenv.  This re-reads all of them, for
 * a process that changes its environment between measurements or tests.  Must
 * not run concurrently with launches.  No counterpart in the reference. */
void mtp_reload_tuning(void);
/* dst[0:bytes] = src[0:bytes] with 16-byte accesses; bytes % 16 == 0. */
int mtp_stream_copy(const void* src, void* dst, int64_t bytes, void* stream);
/* Register-resident bf16 MFMA loop: iters x 32x32x16 MFMAs per wave on
 * n_waves waves (iters a multiple of 16); writes one float per lane to sink
 * (>= 64*n_waves floats).  random_data != 0 feeds operands with random
 * signs and mantissas, 0 feeds smooth small values: the sustained rate differs
 * because the chip runs against its power limit.  Reports nothing itself:
 * time it with events. */
int mtp_mfma_peak(float* sink, int64_t n_waves, int64_t iters, int random_data, void* stream);

/* The same for the instruction stream of the 64-deep GEMM loop: iters x
 * v_mfma_f32_16x16x32_bf16 per wave (iters a multiple of 128) on 64
 * accumulator quads with 32 register-resident operand fragments walked in
 * the GEMM's quadrant order; no LDS reads, no memory traffic.  Launch it on
 * 1024 waves (one per SIMD, as the GEMM runs) for the ceiling of that loop on
 * this board.  No counterpart in the reference: a measurement aid. */
int mtp_mfma_peak_gemm_loop(float* sink, int64_t n_waves, int64_t iters, int random_data, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MERAK_TP_GFX950_H */
