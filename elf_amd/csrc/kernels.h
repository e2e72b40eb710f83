// Internal launcher prototypes shared by the C-ABI layer and the stage executor.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace elf {

enum GemmEpilogue {
	EPI_BF16 = 0,        // C(bf16) = acc
	EPI_BF16_RESID = 1,  // C(bf16) = acc + R(bf16)
	EPI_F32_ACC = 2,     // C(fp32) += acc
	EPI_F32_STORE = 3,   // C(fp32) = acc
};

int gemm_bf16(int a_t, int b_t, int M, int N, int K, const void* A, int64_t lda, const void* B, int64_t ldb,
              void* C, int64_t ldc, int epi, const void* R, int64_t ldr, int tile_cfg, int k_splits,
              hipStream_t stream);

}  // namespace elf
