/*
 * C ABI of libelf_stage.so: the MI355X (gfx950) execution path of one ELF pipeline stage.
 *
 * The reference (topal-team/elf) is pure Python on PyTorch and has no FFI; its plug points on
 * this path are Python objects.  Every entry point below cites the reference code whose work it
 * takes over.  Conventions:
 *   - plain pointers and sizes only; device pointers are HIP device memory owned by the caller
 *     unless stated otherwise; bf16 tensors are row-major with the stated leading dimension;
 *   - every call returns 0 on success, <0 on failure; elf_last_error() returns the message for
 *     the calling host thread;
 *   - all device work is enqueued asynchronously on the hipStream_t passed in (`stream`, given as
 *     void* so that the header needs no HIP include); one host thread drives one stage.
 */
#ifndef ELF_STAGE_H
#define ELF_STAGE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Message of the last failed call on this host thread ("" if none). */
const char* elf_last_error(void);
/* Library ABI version (bumped when a signature changes). */
int elf_abi_version(void);

/* ---------------------------------------------------------------------------------------------
 * Dense contraction used by every linear layer of the stage.
 *   C[M,N] (+)= sum_k A(m,k) * B(n,k), bf16 inputs, fp32 accumulation on MFMA.
 *   a_t = 0: A is [M,K] (k contiguous, leading dim lda); a_t = 1: A is [K,M] (m contiguous).
 *   b_t = 0: B is [N,K] (k contiguous, leading dim ldb); b_t = 1: B is [K,N] (n contiguous).
 *   epilogue: 0 C(bf16) = acc; 1 C(bf16) = acc + R(bf16, leading dim ldr);
 *             2 C(fp32) += acc; 3 C(fp32) = acc.
 *   tile_cfg = 0 picks a tile shape from M,N; k_splits = 0 picks a K split (epilogue 2 only).
 * Replaces: F.linear in LinearDX.forward (elf/zb_utils.py:20)            -> a_t=0,b_t=0
 *           torch.mm(grad_output, weight) in LinearDX.backward (:34-37)  -> a_t=0,b_t=1
 *           torch.mm(go.t(), inp) + weight.grad.add_ in LinearDW.backward (:238-244) -> a_t=1,b_t=1, epilogue 2
 * M, N multiples of 64, K a multiple of 64, pointers 16-byte aligned. */
int elf_gemm_bf16(int a_t, int b_t, int M, int N, int K, const void* A, int64_t lda, const void* B,
                  int64_t ldb, void* C, int64_t ldc, int epilogue, const void* R, int64_t ldr,
                  int tile_cfg, int k_splits, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Bandwidth-bound stage ops.  bf16 row-major tensors, fp32 math, one rounding on store.
 * kind: 0 = RMSNorm (y = x * rsqrt(mean(x^2)+eps) * gamma; no reference module, textbook form),
 *       1 = LayerNorm (nn.LayerNorm, benchmarks/models/simple.py:444-445).
 * stats: fp32 [T,2] = {mean, rstd} per row, written by the forward and read by the backward.
 * elf_norm_bwd: dx = norm_backward(dy) (+ dres if non-null: the residual gradient that bypasses
 * the norm); dgamma / dbeta are fp32 accumulators updated with +=; workspace holds
 * elf_norm_bwd_workspace_floats(T, d) floats.  Replaces the autograd backward of the norm module
 * that runs inside PipelineBlock.backward_inputs (elf/execution/block.py:281-306). */
int elf_norm_fwd(int kind, const void* x, const void* gamma, const void* beta, void* y, void* stats,
                 int T, int d, float eps, void* stream);
int64_t elf_norm_bwd_workspace_floats(int T, int d);
int elf_norm_bwd(int kind, const void* dy, const void* x, const void* gamma, const void* stats,
                 const void* dres, void* dx, float* dgamma, float* dbeta, float* workspace, int T,
                 int d, void* stream);

/* Exact (erf) GELU of nn.GELU() (benchmarks/models/simple.py:44-52) over n elements. */
int elf_gelu_fwd(const void* x, void* y, int64_t n, void* stream);
int elf_gelu_bwd(const void* dy, const void* x, void* dx, int64_t n, void* stream);
/* SwiGLU: h[T,F] = silu(gu[:, :F]) * gu[:, F:], gu is [T,2F] (no reference module). */
int elf_swiglu_fwd(const void* gu, void* h, int64_t T, int F, void* stream);
int elf_swiglu_bwd(const void* dh, const void* gu, void* dgu, int64_t T, int F, void* stream);

/* Rotary embedding, half-split convention, in place on the first n_heads heads (width D) of a
 * packed [T, ld] buffer; position = token index mod S.  cs = fp32 [S, D/2, 2] (cos, sin) table
 * filled by elf_rope_table (angles evaluated in fp64).  backward != 0 applies the inverse
 * rotation (the gradient of the forward).  No reference module; textbook form. */
int elf_rope_table(void* cs, int S, int D, double theta, void* stream);
int elf_rope_apply(void* buf, const void* cs, int64_t T, int S, int ld, int n_heads, int D,
                   int backward, void* stream);

/* acc_f32[i] *= scale; out_bf16[i] = bf16(acc_f32[i]) if out_bf16 != NULL.
 * Replaces PipelineBlock.scale_grads (elf/execution/block.py:518-527). */
int elf_scale_grads(void* acc_f32, void* out_bf16, int64_t n, float scale, void* stream);
/* out = a + b over n bf16 elements: gradient fan-in of an output with several targets
 * (elf/execution/block.py:651-655) and residual adds (simple.py:460,466). */
int elf_add_bf16(const void* a, const void* b, void* out, int64_t n, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Attention on the packed projection layout: q/k/v/o are column slices of [T, ld*] bf16 buffers,
 * T = B*S tokens, head h at columns [h*D, (h+1)*D).  Hq % Hkv == 0 (grouped-query attention),
 * D in {64, 128}, S % 128 == 0.  lse: fp32 [B, Hq, S] (natural log of the softmax denominator).
 * Replaces SDPA / softmax(QK^T*scale)V forward and its autograd backward
 * (benchmarks/models/simple.py:362-367, 379-386).  The backward needs
 * elf_attn_bwd_workspace_bytes() of 16-byte aligned scratch. */
int elf_attn_fwd(const void* q, const void* k, const void* v, void* o, void* lse, int64_t ldq,
                 int64_t ldk, int64_t ldv, int64_t ldo, int B, int S, int Hq, int Hkv, int D,
                 int causal, float scale, void* stream);
int64_t elf_attn_bwd_workspace_bytes(int B, int S, int Hq, int D);
int elf_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dO,
                 const void* lse, void* dq, void* dk, void* dv, void* workspace, int64_t ldq,
                 int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo, int64_t lddq, int64_t lddk,
                 int64_t lddv, int B, int S, int Hq, int Hkv, int D, int causal, float scale,
                 void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ELF_STAGE_H */
