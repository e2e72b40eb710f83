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

#ifdef __cplusplus
}
#endif
#endif /* ELF_STAGE_H */
