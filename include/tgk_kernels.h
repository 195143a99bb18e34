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
 * M, N multiples of 128, K multiple of 64; pointers 16-byte aligned; ld* multiples of 8. */
TGK_API int tgk_gemm_fwd(hipStream_t stream, int M, int N, int K, const uint16_t *X, int ldx,
                 const uint16_t *W, int ldw, uint16_t *Y, int ldy, const uint16_t *residual, int ldr,
                 uint16_t *gelu_out, int ldg);

/* Input gradient, replaces matmul + cast_result as used by linear_backward
 * (cuda/ops.cuh:30-55, :115).
 *   dX[M][K] = RN_bf16( dY[M][N] . W[N][K] )
 *   gelu_pre != NULL : dX = RN_bf16( RN_bf16(acc) * gelu'(gelu_pre) )   (fused activation
 *                      backward, stands in for swiglu_backward, cuda/ops.cuh:133-144)
 * M, K multiples of 128, N multiple of 64. */
TGK_API int tgk_gemm_dgrad(hipStream_t stream, int M, int N, int K, const uint16_t *dY, int lddy,
                   const uint16_t *W, int ldw, uint16_t *dX, int lddx, const uint16_t *gelu_pre,
                   int ldu);

/* Weight gradient, replaces weight_gradient (cuda/ops.cuh:83-109) and, through its fixed-order
 * split-K reduction, reduce_gradients (cuda/trainer.cuh:9-47).
 *   dW[N][K] (= | +=) dY[M][N]^T . X[M][K]      fp32, deterministic
 * N, K multiples of 128, M multiple of 64.  `workspace` must hold
 * tgk_gemm_wgrad_workspace(M,N,K) bytes (may be NULL when that is 0). */
TGK_API int tgk_gemm_wgrad(hipStream_t stream, int M, int N, int K, const uint16_t *dY, int lddy,
                   const uint16_t *X, int ldx, float *dW, int lddw, int accumulate, void *workspace,
                   size_t workspace_bytes);
TGK_API size_t tgk_gemm_wgrad_workspace(int M, int N, int K);

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

#ifdef __cplusplus
}
#endif
#endif
