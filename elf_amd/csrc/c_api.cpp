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

int elf_gemm_dw_group(int n, const elf_dw_problem* problems, int K, float scale, void* stream) {
	// the header's plain-C problem record and the launcher's are the same eight fields in the same order
	static_assert(sizeof(elf_dw_problem) == sizeof(elf::DwProblem) && offsetof(elf_dw_problem, acc) == offsetof(elf::DwProblem, acc) &&
	                  offsetof(elf_dw_problem, N) == offsetof(elf::DwProblem, N),
	              "elf_dw_problem and elf::DwProblem differ");
	return elf::gemm_dw_group(n, reinterpret_cast<const elf::DwProblem*>(problems), K, scale, (hipStream_t)stream);
}

int elf_gemm_act_bf16(int act, int M, int F, int K, const void* A, int64_t lda, const void* W, int64_t ldw,
                      void* pre, int64_t ldpre, void* out, int64_t ldout, void* stream) {
	return elf::gemm_act_bf16(act, M, F, K, A, lda, W, ldw, pre, ldpre, out, ldout, (hipStream_t)stream);
}

int elf_gemm_swiglu_bwd_bf16(int M, int F, int K, const void* dY, int64_t lddy, const void* W, int64_t ldw,
                             const void* gu, int64_t ldgu, void* dgu, int64_t lddgu, void* scratch, void* stream) {
	return elf::gemm_swiglu_bwd_bf16(M, F, K, dY, lddy, W, ldw, gu, ldgu, dgu, lddgu, scratch, (hipStream_t)stream);
}

#define S_(x) ((hipStream_t)(x))
int elf_gemm_rope_bf16(int M, int N, int K, const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, const void* cs, int S,
                       int n_rot_heads, int D, void* stream) {
	return elf::gemm_rope_bf16(M, N, K, A, lda, W, ldw, C, ldc, cs, S, n_rot_heads, D, S_(stream));
}
int elf_norm_fwd(int kind, const void* x, const void* gamma, const void* beta, void* y, void* stats, int T, int d,
                 float eps, void* stream) {
	return elf::norm_fwd(kind, x, gamma, beta, y, stats, T, d, eps, S_(stream));
}
int64_t elf_norm_bwd_workspace_floats(int T, int d) { return elf::norm_bwd_workspace_floats(T, d); }
int elf_norm_bwd(int kind, const void* dy, const void* x, const void* gamma, const void* stats, const void* dres,
                 void* dx, float* dgamma, float* dbeta, float* workspace, int T, int d, void* stream) {
	return elf::norm_bwd(kind, dy, x, gamma, stats, dres, dx, dgamma, dbeta, workspace, T, d, S_(stream));
}
int elf_norm_bwd_noalloc(int kind, const void* dy, const void* x, const void* gamma, const void* stats, const void* dres,
                         void* dx, float* dgamma, float* dbeta, int T, int d, void* stream) {
	return elf::norm_bwd_noalloc(kind, dy, x, gamma, stats, dres, dx, dgamma, dbeta, T, d, S_(stream));
}
int elf_gelu_fwd(const void* x, void* y, int64_t n, void* stream) { return elf::gelu_fwd(x, y, n, S_(stream)); }
int elf_gelu_bwd(const void* dy, const void* x, void* dx, int64_t n, void* stream) {
	return elf::gelu_bwd(dy, x, dx, n, S_(stream));
}
int elf_swiglu_fwd(const void* gu, void* h, int64_t T, int F, void* stream) {
	return elf::swiglu_fwd(gu, h, T, F, S_(stream));
}
int elf_swiglu_bwd(const void* dh, const void* gu, void* dgu, int64_t T, int F, void* stream) {
	return elf::swiglu_bwd(dh, gu, dgu, T, F, S_(stream));
}
int elf_rope_table(void* cs, int S, int D, double theta, void* stream) {
	return elf::rope_table(cs, S, D, theta, S_(stream));
}
int elf_rope_apply(void* buf, const void* cs, int64_t T, int S, int ld, int n_heads, int D, int backward, void* stream) {
	return elf::rope_apply(buf, cs, T, S, ld, n_heads, D, backward, S_(stream));
}
int elf_scale_grads(void* acc_f32, void* out_bf16, int64_t n, float scale, void* stream) {
	return elf::scale_grads(acc_f32, out_bf16, n, scale, S_(stream));
}
int elf_add_bf16(const void* a, const void* b, void* out, int64_t n, void* stream) {
	return elf::add_bf16(a, b, out, n, S_(stream));
}
int64_t elf_colsum_workspace_floats(int64_t T, int N) { return elf::colsum_workspace_floats(T, N); }
int elf_colsum_bf16(const void* x, int64_t ld, void* out_f32, int64_t T, int N, float* workspace, void* stream) {
	return elf::colsum_bf16(x, ld, out_f32, T, N, workspace, S_(stream));
}
int elf_embedding_fwd(const void* ids, const void* table, void* out, int64_t T, int d, int V, void* stream) {
	return elf::embedding_fwd(ids, table, out, T, d, V, S_(stream));
}
int elf_embedding_bwd(const void* ids, const void* dx, void* dtable_f32, int64_t T, int d, int V, void* stream) {
	return elf::embedding_bwd(ids, dx, dtable_f32, T, d, V, S_(stream));
}
int elf_cross_entropy(const void* logits, int64_t ld, const void* target, int64_t rows, int64_t V, int64_t ignore_index, float scale,
                      const void* dev_div, void* row_loss, void* dlogits, int64_t ld_out, void* stream) {
	return elf::cross_entropy(logits, ld, target, rows, V, ignore_index, scale, dev_div, row_loss, dlogits, ld_out, S_(stream));
}
int elf_cross_entropy_reduce(const void* row_loss, const void* target, int64_t rows, int64_t ignore_index, void* out2, void* stream) {
	return elf::cross_entropy_reduce(row_loss, target, rows, ignore_index, out2, S_(stream));
}
int elf_attn_fwd(const void* q, const void* k, const void* v, void* o, void* lse, int64_t ldq, int64_t ldk, int64_t ldv,
                 int64_t ldo, int B, int S, int Hq, int Hkv, int D, int causal, float scale, void* stream) {
	return elf::attn_fwd(q, k, v, o, lse, ldq, ldk, ldv, ldo, B, S, Hq, Hkv, D, causal, scale, S_(stream));
}
int64_t elf_attn_bwd_workspace_bytes(int B, int S, int Hq, int D, int causal) { return elf::attn_bwd_workspace_bytes(B, S, Hq, D, causal); }
int elf_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dO, const void* lse, void* dq,
                 void* dk, void* dv, void* workspace, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo,
                 int64_t lddq, int64_t lddk, int64_t lddv, int B, int S, int Hq, int Hkv, int D, int causal, float scale,
                 void* stream) {
	return elf::attn_bwd(q, k, v, o, dO, lse, dq, dk, dv, workspace, ldq, ldk, ldv, ldo, lddo, lddq, lddk, lddv, B, S, Hq,
	                     Hkv, D, causal, scale, S_(stream));
}

int elf_attn_bwd_rope(const void* q, const void* k, const void* v, const void* o, const void* dO, const void* lse, void* dq,
                      void* dk, void* dv, void* workspace, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo,
                      int64_t lddq, int64_t lddk, int64_t lddv, int B, int S, int Hq, int Hkv, int D, int causal, float scale,
                      const void* cs, void* stream) {
	return elf::attn_bwd(q, k, v, o, dO, lse, dq, dk, dv, workspace, ldq, ldk, ldv, ldo, lddo, lddq, lddk, lddv, B, S, Hq,
	                     Hkv, D, causal, scale, S_(stream), cs);
}

int elf_hbm_probe(int mode, const void* src, void* dst, int64_t bytes, void* stream) { return elf::hbm_probe(mode, src, dst, bytes, S_(stream)); }

int elf_gemm_turn_giveups(uint64_t* out) {
	if (!out) return -1;
	return elf::gemm_turn_giveups(out);
}

void elf_prof_enable(int on) { elf::prof_enable(on); }
int64_t elf_prof_launches(int kind, double* total_work) { return elf::prof_launches(kind, total_work); }
int elf_prof_collect(int kind, double* total_ms, double* total_work) {
	if (kind < 0 || kind >= elf::PROF_COUNT) return -1;
	return elf::prof_collect(kind, total_ms, total_work);
}

}  // extern "C"
