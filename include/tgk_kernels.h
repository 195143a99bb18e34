/*
 * tgk_* : the kernel-level C ABI of the MI355X (gfx950) training-step hot path.
 *
 * The reference (lostmsu/TurboGPT) inlines these operators into one persistent CUDA kernel and
 * has no ABI between its engine and its device code; each entry below names the device function
 * it stands in for.  All pointers are DEVICE pointers, bf16 tensors are raw 16-bit patterns
 * (uint16_t), leading dimensions are in elements, `stream` is a hipStream_t (NULL = the null
 * stream).  Entry points launch asynchronously on `stream`, never allocate and never
 * synchronise.  Return value: 0 = launched, -1 = rejected; tgk_error() then holds the reason
 * (thread local, valid until the next failing call on the same thread).
 */
#ifndef TGK_KERNELS_H
#define TGK_KERNELS_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef __HIP_PLATFORM_AMD__
typedef struct ihipStream_t *hipStream_t;
#endif
#define TGK_API __attribute__((visibility("default")))

TGK_API const char *tgk_error(void);

/* ---- GEMM family.  W is [N][K] row major ("[Out][In]", model.h:12-37), fp32 accumulate. ---- */

/* Forward projection, replaces project<In,Out> (cuda/mma.cuh:77-108).
 *   Y[M][N] = RN_bf16( X[M][K] . W[N][K]^T )
 *   residual != NULL : Y = RN_bf16( RN_bf16(acc) + residual )      (bf16 add, cuda/mma.cuh:95-97)
 *   gelu_out != NULL : additionally gelu_out = RN_bf16( gelu(Y) )  (Y keeps the pre-activation;
 *                      stands in for swiglu_activation, cuda/ops.cuh:120-128)
 * M multiple of 128, N multiple of 128 or 192, K multiple of 32; pointers 16-byte aligned; ld*
 * multiples of 8. */
TGK_API int tgk_gemm_fwd(hipStream_t stream, int M, int N, int K, const uint16_t *X, int ldx,
                 const uint16_t *W, int ldw, uint16_t *Y, int ldy, const uint16_t *residual, int ldr,
                 uint16_t *gelu_out, int ldg);

/* The same forward projection with the weight given transposed, Wt[K][N] (leading dimension ldwt):
 * whole rows of Wt are copied instead of 64-byte pieces of W, which is faster where tgk_gemm_fwd cannot
 * use its 64-k stages (K not a multiple of 64, or N not a multiple of 192).  Same epilogues and shape
 * rules as tgk_gemm_fwd. */
TGK_API int tgk_gemm_fwd_t(hipStream_t stream, int M, int N, int K, const uint16_t *X, int ldx,
                           const uint16_t *Wt, int ldwt, uint16_t *Y, int ldy, const uint16_t *residual,
                           int ldr, uint16_t *gelu_out, int ldg);

/* Input gradient, replaces matmul + cast_result as used by linear_backward
 * (cuda/ops.cuh:30-55, :115).
 *   dX[M][K] = RN_bf16( dY[M][N] . W[N][K] )
 *   gelu_pre != NULL : dX = RN_bf16( RN_bf16(acc) * gelu'(gelu_pre) )   (fused activation
 *                      backward, stands in for swiglu_backward, cuda/ops.cuh:133-144)
 * M multiple of 128, K multiple of 128 or 192, N multiple of 32. */
TGK_API int tgk_gemm_dgrad(hipStream_t stream, int M, int N, int K, const uint16_t *dY, int lddy,
                   const uint16_t *W, int ldw, uint16_t *dX, int lddx, const uint16_t *gelu_pre,
                   int ldu);

/* The same input gradient with the weight given transposed, Wt[K][N] (leading dimension ldwt): both
 * operands are then contiguous along the reduced dimension and the product runs on the forward
 * kernel (64-k stages when N is a multiple of 64 and K of 192).  Same epilogue and shape rules as
 * tgk_gemm_dgrad. */
TGK_API int tgk_gemm_dgrad_t(hipStream_t stream, int M, int N, int K, const uint16_t *dY, int lddy,
                             const uint16_t *Wt, int ldwt, uint16_t *dX, int lddx,
                             const uint16_t *gelu_pre, int ldu);

/* Weight gradient, replaces weight_gradient (cuda/ops.cuh:83-109) and, through its fixed-order
 * split-K reduction, reduce_gradients (cuda/trainer.cuh:9-47).
 *   dW[N][K] (= | +=) dY[M][N]^T . X[M][K]      fp32, deterministic
 * N multiple of 128, K multiple of 128 or 192, M multiple of 32.  `workspace` must hold
 * tgk_gemm_wgrad_workspace(M,N,K) bytes (may be NULL when that is 0). */
TGK_API int tgk_gemm_wgrad(hipStream_t stream, int M, int N, int K, const uint16_t *dY, int lddy,
                   const uint16_t *X, int ldx, float *dW, int lddw, int accumulate, void *workspace,
                   size_t workspace_bytes);
TGK_API size_t tgk_gemm_wgrad_workspace(int M, int N, int K);

/* Up to four weight gradients that share the reduced dimension M (the tokens) in one launch, e.g. the four of
 * a transformer block: dW_j[N_j][K_j] (= | +=) dY_j[M][N_j]^T . X_j[M][K_j], fp32, deterministic.  The output
 * tiles of all jobs are cut into equal runs of work over the resident blocks, so the matrices need not fill the
 * GPU one by one and far fewer partial sums are written than by one tgk_gemm_wgrad per matrix.  Every N_j a
 * multiple of 128, every K_j of 192, M of 64.  `workspace` holds tgk_gemm_wgrad_batch_workspace(M, count, jobs)
 * bytes.  No counterpart in the reference, which computes one weight_gradient at a time (cuda/ops.cuh:83-109). */
typedef struct TgkWgradJob {
    int N, K;
    const uint16_t *dY;
    int lddy;
    const uint16_t *X;
    int ldx;
    float *dW;
    int lddw;
} TgkWgradJob;
TGK_API int tgk_gemm_wgrad_batch(hipStream_t stream, int M, int count, const TgkWgradJob *jobs, int accumulate,
                                 void *workspace, size_t workspace_bytes);
TGK_API size_t tgk_gemm_wgrad_batch_workspace(int M, int count, const TgkWgradJob *jobs);

/* Every weight gradient of a training step in one launch: any number of jobs (1..4096) that share the reduced
 * dimension M, dW_j[N_j][K_j] = dY_j[M][N_j]^T . X_j[M][K_j], fp32, deterministic.  Takes the slot of all the
 * weight_gradient calls of a backward pass (cuda/ops.cuh:83-109, called per matrix from cuda/model.cuh:61-99) and of
 * reduce_gradients (cuda/trainer.cuh:9-47).  With several 256 x 256 output tiles per compute unit, all but the last
 * (tiles mod compute units) tiles are reduced over all M rows by one block, in row order, and written once; the
 * last ones are cut into row ranges whose partial sums a second launch adds in row order.  The caller keeps all
 * operands alive until this call (the output gradients of every layer).  Every N_j and K_j a multiple of 256, M of
 * 128, accumulate = 0.  The job and tile tables live in device memory: tgk_gemm_wgrad_list_prepare writes them into
 * `table` (tgk_gemm_wgrad_list_table_bytes bytes, 16-byte aligned) with a synchronous copy, once per job list;
 * tgk_gemm_wgrad_list is then called with the same M, jobs and table.  `workspace` holds
 * tgk_gemm_wgrad_list_workspace bytes (may be NULL when that is 0). */
TGK_API size_t tgk_gemm_wgrad_list_table_bytes(int M, int count, const TgkWgradJob *jobs);
TGK_API size_t tgk_gemm_wgrad_list_workspace(int M, int count, const TgkWgradJob *jobs);
TGK_API int tgk_gemm_wgrad_list_prepare(int M, int count, const TgkWgradJob *jobs, void *table, size_t table_bytes);
TGK_API int tgk_gemm_wgrad_list(hipStream_t stream, int M, int count, const TgkWgradJob *jobs, const void *table,
                                int accumulate, void *workspace, size_t workspace_bytes, float *sumsq);
/* `sumsq` (may be NULL) receives tgk_gemm_wgrad_list_sumsq_count floats whose sum is the sum of squares of every
 * gradient element the call writes: the kernels that write a gradient square it on the way, in a fixed order, so that
 * the clip norm (cuda/trainer.cuh:35-46, cuda/optim.cuh:67-80) needs no second pass over these matrices. */
TGK_API int tgk_gemm_wgrad_list_sumsq_count(int M, int count, const TgkWgradJob *jobs);


/* ---- Causal softmax attention, head_dim 64.  Takes the slot of attention_forward /
 * attention_backward (cuda/attention.cuh:48-106); the reference's arg-max attention is replaced
 * by softmax(Q K^T * scale + causal mask) V as the target specifies.  Layout is the reference's
 * (cuda/attention.cuh:38-39,68): Q, K, V are [B*T][ld] views with head h at columns h*64..h*64+63
 * (normally three column slices of the packed qkv buffer, ld = 3*d), O is [B*T][ldo].
 * lse is [B][H][T] fp32 = natural log of the row sums of exp(scaled scores).
 * T multiple of 128; pointers 16-byte aligned; leading dimensions multiples of 8. ---- */
TGK_API int tgk_attn_fwd(hipStream_t stream, int B, int H, int T, int hd, const uint16_t *Q,
                         const uint16_t *K, const uint16_t *V, int ld, uint16_t *O, int ldo, float *lse,
                         float scale);
/* Recompute backward from Q, K, V, O, lse: dQ, dK, dV ([B*T][lddq] views, same head layout).
 * Deterministic (no atomics).  workspace: tgk_attn_bwd_workspace(B,H,T) bytes. */
TGK_API int tgk_attn_bwd(hipStream_t stream, int B, int H, int T, int hd, const uint16_t *Q,
                         const uint16_t *K, const uint16_t *V, int ld, const uint16_t *O, int ldo,
                         const float *lse, const uint16_t *dO, int lddo, uint16_t *dQ, uint16_t *dK,
                         uint16_t *dV, int lddq, float scale, void *workspace, size_t workspace_bytes);
TGK_API size_t tgk_attn_bwd_workspace(int B, int H, int T);
/* tgk_attn_bwd without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * two row vectors the backward kernels exchange (2 * B*H*T floats) live in a device array inside the library:
 * 8 MiB per GPU the library runs on, held until the process ends.  B*H*T <= tgk_attn_bwd_static_max_rows()
 * (1048576); larger shapes are rejected and need tgk_attn_bwd.  The call allocates and frees nothing.  All
 * calls on one GPU share the array: calls that overlap on one GPU (different streams or threads) race.
 * Same kernels and results, bit for bit, as tgk_attn_bwd.  The array's address is looked up once per device, on the
 * first tgk_attn_bwd_static or tgk_attn_bwd_static_max_rows call made with that device current: make one of them
 * outside any stream capture on every device that will run it (a lookup inside a capture may be refused), and call
 * with the stream's device current - the array used is the current device's. */
TGK_API int tgk_attn_bwd_static(hipStream_t stream, int B, int H, int T, int hd, const uint16_t *Q,
                                const uint16_t *K, const uint16_t *V, int ld, const uint16_t *O, int ldo,
                                const float *lse, const uint16_t *dO, int lddo, uint16_t *dQ, uint16_t *dK,
                                uint16_t *dV, int lddq, float scale);
TGK_API size_t tgk_attn_bwd_static_max_rows(void);

/* ---- HBM-bound operators.  Parameters are held as two 16-bit halves of their fp32 master:
 * `hi` (the bf16 compute weight, truncated) and `lo` (cuda/ops.cuh:6-14); operators that need
 * full fp32 parameters (norm scales) take both halves, as precise_weight does. ---- */

/* out[t] = RN_bf16(table[x[t]] + positions[t % T]); replaces the gather of load_tile
 * (cuda/dataset.cuh:31-32) and adds the learned positions the target model uses. */
TGK_API int tgk_embed_fwd(hipStream_t stream, int rows, int T, int D, const uint8_t *x,
                          const uint16_t *table, const uint16_t *positions, uint16_t *out);
/* dtable[v] (=|+=) sum_{t: x[t]=v} dh[t]; dpositions[p] (=|+=) sum_b dh[b*T+p]; fp32.  Replaces
 * the atomicAdd scatter of cuda/model.cuh:96-97 with a fixed-order sum. D multiple of 64, vocab
 * 256.  workspace: tgk_embed_bwd_workspace(B*T, D) bytes. */
TGK_API int tgk_embed_bwd(hipStream_t stream, int B, int T, int D, int vocab, const uint8_t *x,
                          const uint16_t *dh, float *dtable, float *dpositions, int accumulate,
                          void *workspace, size_t workspace_bytes);
TGK_API size_t tgk_embed_bwd_workspace(int rows, int D);
/* The same in two parts, for a caller that multiplies weight gradients as one list (tgk_gemm_wgrad_list): writes the
 * exact one-hot matrix of the tokens, onehot[B*T][256] (bf16, 16-byte aligned), whose product onehot^T . dh IS dtable -
 * one more job {N = 256, K = D, dY = onehot, X = dh} of that list - and computes dpositions as above. */
TGK_API int tgk_embed_bwd_onehot(hipStream_t stream, int B, int T, int D, const uint8_t *x, const uint16_t *dh,
                                 uint16_t *onehot, float *dpositions, int accumulate);

/* y = RN_bf16((x - mean) * rsqrt(var + eps) * gamma + beta) per row; takes the slot of normalize
 * (cuda/ops.cuh:57-66; RMSNorm there, LayerNorm in the target model). D multiple of 8, <= 2048. */
TGK_API int tgk_layernorm_fwd(hipStream_t stream, int rows, int D, const uint16_t *x,
                              const uint16_t *gamma_hi, const uint16_t *gamma_lo,
                              const uint16_t *beta_hi, const uint16_t *beta_lo, uint16_t *y, float eps);
/* dx = RN_bf16(LN'(x) dy), or with residual != 0: dx = RN_bf16(dx + RN_bf16(LN'(x) dy)) (residual
 * gradients stay in bf16, cuda/ops.cuh:74-76); dgamma/dbeta (=|+=) fixed-order column sums in
 * fp32 (replaces the atomicAdd of cuda/ops.cuh:77); D multiple of 64.  Takes the slot of norm_backward
 * (cuda/ops.cuh:67-80).  workspace: tgk_layernorm_bwd_workspace(rows, D) bytes. */
TGK_API int tgk_layernorm_bwd(hipStream_t stream, int rows, int D, const uint16_t *x, const uint16_t *dy,
                              const uint16_t *gamma_hi, const uint16_t *gamma_lo, uint16_t *dx,
                              float *dgamma, float *dbeta, float eps, int residual, int accumulate,
                              void *workspace, size_t workspace_bytes);
/* The same with the residual gradient taken from a buffer of its own: dx = RN_bf16(residual + RN_bf16(LN'(x) dy));
 * residual may be NULL (no addition) or dx itself.  Lets a caller keep the incoming gradient for later use. */
TGK_API int tgk_layernorm_bwd_add(hipStream_t stream, int rows, int D, const uint16_t *x, const uint16_t *dy,
                                  const uint16_t *gamma_hi, const uint16_t *gamma_lo, const uint16_t *residual,
                                  uint16_t *dx, float *dgamma, float *dbeta, float eps, int accumulate,
                                  void *workspace, size_t workspace_bytes);
TGK_API size_t tgk_layernorm_bwd_workspace(int rows, int D);
/* The two halves of tgk_layernorm_bwd_add, for a caller that runs many LayerNorm backwards before it needs
 * their parameter gradients (a training step has 2 * depth + 1): _rows writes dx and this LayerNorm's partial
 * sums (tgk_layernorm_bwd_workspace(rows, D) bytes at `partials`, which must stay untouched until the fold);
 * _fold sums `count` such partial blocks, job j at partials + j * job_stride_bytes, into the dgamma / dbeta
 * pointer pairs of a DEVICE array `targets` ({float *dgamma, *dbeta} per job) in one launch.  Same sums in the
 * same order as tgk_layernorm_bwd_add: the gradients are bit-identical. */
TGK_API int tgk_layernorm_bwd_rows(hipStream_t stream, int rows, int D, const uint16_t *x, const uint16_t *dy,
                                   const uint16_t *gamma_hi, const uint16_t *gamma_lo, const uint16_t *residual,
                                   uint16_t *dx, float eps, void *partials, size_t partials_bytes);
TGK_API int tgk_layernorm_bwd_fold(hipStream_t stream, int rows, int D, int count, const void *partials,
                                   size_t job_stride_bytes, const void *targets, int accumulate);

/* Softmax cross-entropy over 256 byte classes on bf16 logits [rows][256] (cuda/model.cuh:33-58):
 * loss[t] = logsumexp - logit[y[t]]; logits_f32 (optional) receives the logits as fp32;
 * write_grad != 0 overwrites the logits with RN_bf16((softmax - onehot) * inv_count). */
TGK_API int tgk_cross_entropy(hipStream_t stream, int rows, int vocab, uint16_t *logits, const uint8_t *y,
                              float *loss, float *logits_f32, float inv_count, int write_grad);

/* out[c][r] = in[r][c] for `count` row-major bf16 matrices that sit at the same element offset in
 * `in` and `out` (the engine's transposed copy of the compute weights).  jobs: device array of
 * {int64 offset; int32 rows, cols, first_tile, pad} with rows, cols multiples of 64 and
 * first_tile the running count of 64x64 tiles; total_tiles = their sum. */
TGK_API int tgk_transpose_batch(hipStream_t stream, const uint16_t *in, uint16_t *out, const void *jobs,
                                int count, int total_tiles);

/* partials[i] = sum of squares of block i's share of g (cuda/trainer.cuh:35-46); count <= 4096. */
TGK_API int tgk_sumsq_partials(hipStream_t stream, const float *g, size_t n, float *partials, int count);
/* partials[i] = sum of squares of g[start_i .. start_i + length_i): the same for a list of ranges, one block each
 * (the tensors whose gradients tgk_gemm_wgrad_list does not write, cut into ranges of a few thousand elements).
 * segments: device array of {int64 start, length}, both multiples of 4; count <= 4096. */
TGK_API int tgk_sumsq_segments(hipStream_t stream, const float *g, const void *segments, int count, float *partials);
/* AdamW on the hi/lo weight halves (cuda/optim.cuh:67-106): clip scale min(1, clip/(||g||+1e-6))
 * from the folded partials when clip > 0, m += (1-b1)(g-m), v = b2 v + (1-b2) g^2,
 * w = w (1 - lr*wd) - (lr/bc1) m / (sqrt(v)/sqrt(bc2) + eps), bias corrections from `step`
 * (0-based) with the current beta1.  segment_starts (device, sorted, first = 0) and
 * segment_flags (device, bit 0 = apply weight decay, bit 1 = leave the segment untouched: it belongs
 * to another optimizer) describe the parameter groups (cuda/optim.cuh:5-15).  n and all segment starts multiples of 4. */
TGK_API int tgk_adamw(hipStream_t stream, size_t n, uint16_t *weight_hi, uint16_t *weight_lo, float *m,
                      float *v, const float *g, const float *norm_partials, int norm_count,
                      const int64_t *segment_starts, const uint8_t *segment_flags, int segments, float lr,
                      float beta1, float beta2, float eps, float weight_decay, float clip, uint64_t step);

/* Hash-sampled batch (cuda/dataset.cuh:13-27): endpoint e = low + hash_u64(seed + step*batch + b)
 * mod (size - low), low = max(8, context); x = data[e-context : e], y = data[e-context+1 : e+1]. */
TGK_API int tgk_sample_batch(hipStream_t stream, const uint8_t *data, int64_t size, uint64_t seed,
                             uint64_t step, int batch, int context, uint8_t *x, uint8_t *y);
/* out[p] = mean over the batch of token_loss[b*context + p], in double (cuda/trainer.cuh:79-100). */
TGK_API int tgk_position_means(hipStream_t stream, const float *token_loss, int batch, int context,
                               float *out);

/* ---- The reference's own width-16 network (config.h:4, model.h:12-37): RMSNorm, partial RoPE, causal
 * arg-max attention with a GELU gate, SwiGLU(48), 4 heads of 4, vocabulary 256.  These four calls stand in
 * for forward / backward / optimize of the persistent kernel (cuda/model.cuh:8-99, cuda/optim.cuh:17-119)
 * when an engine is created from the plain Config.  depth 1..8, context 1..8 (the RoPE table of
 * cuda/attention.cuh:7-14 has eight entries); weights in the flat order of model.h:12-37. ---- */
TGK_API int tgk_w16_parameter_count(int depth);
/* bytes of device workspace (256-byte aligned) that forward fills and backward consumes */
TGK_API size_t tgk_w16_workspace(int depth, int batch, int context);
/* x, y: [batch*context] tokens and targets.  token_losses[batch*context]; logits (may be NULL) receives
 * [batch*context][256] floats; with_gradient != 0 also leaves RN_bf16((softmax - onehot) / tokens) in the
 * workspace for tgk_w16_backward (cuda/model.cuh:54-55). */
TGK_API int tgk_w16_forward(hipStream_t stream, int depth, int batch, int context, const uint16_t *weight_hi,
                            const uint16_t *weight_lo, const uint8_t *x, const uint8_t *y, void *workspace,
                            float *token_losses, float *logits, int with_gradient);
/* after tgk_w16_forward(with_gradient) on the same workspace: every element of gradient[parameter_count]
 * is overwritten; weight gradients are folded in a fixed order (no atomics). */
TGK_API int tgk_w16_backward(hipStream_t stream, int depth, int batch, int context, const uint16_t *weight_hi,
                             const uint16_t *weight_lo, const uint8_t *x, void *workspace, float *gradient);
/* Muon update of the 5*depth hidden matrices (cuda/optim.cuh:17-62, :107-118): Nesterov momentum, bf16
 * Newton-Schulz with the 3.4445 / -4.775 / 2.0315 quintic, decoupled decay, lr * sqrt(max(1, rows/cols)).
 * The clip scale is folded from the same norm partials tgk_adamw uses; the other parameters are
 * tgk_adamw's, whose segment flag bit 1 makes it leave the hidden matrices alone. */
TGK_API int tgk_w16_muon(hipStream_t stream, int depth, uint16_t *weight_hi, uint16_t *weight_lo, float *momentum,
                         const float *gradient, const float *norm_partials, int norm_count, float clip, float lr,
                         float momentum_rate, float weight_decay, int ns_steps);

#ifdef __cplusplus
}
#endif
#endif
