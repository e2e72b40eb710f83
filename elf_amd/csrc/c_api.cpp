// extern "C" surface of libelf_stage.so (declared in include/elf_stage.h).
#include "common.h"
#include "kernels.h"
#include "../../include/elf_stage.h"

extern "C" {

const char* elf_last_error(void) { return elf::get_error(); }
int elf_abi_version(void) { return 1; }

int elf_gemm_bf16(int a_t, int b_t, int M, int N, int K, const void* A, int64_t lda, const void* B,
                  int64_t ldb, void* C, int64_t ldc, int epilogue, const void* R, int64_t ldr,
                  int tile_cfg, int k_splits, void* stream) {
	return elf::gemm_bf16(a_t, b_t, M, N, K, A, lda, B, ldb, C, ldc, epilogue, R, ldr, tile_cfg, k_splits,
	                      (hipStream_t)stream);
}

}  // extern "C"
