// Internal launcher prototypes shared by the C-ABI layer and the stage executor.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <tuple>
#include <utility>

namespace elf {

enum GemmEpilogue {
	EPI_BF16 = 0,        // C(bf16) = acc
	EPI_BF16_RESID = 1,  // C(bf16) = acc + R(bf16)
	EPI_F32_ACC = 2,     // C(fp32) += acc
	EPI_F32_STORE = 3,   // C(fp32) = acc
	// direct-to-LDS tiles with k-contiguous operands only (see gemm_act_bf16):
	EPI_BF16_SWIGLU = 4,  // B = [gate rows; up rows]: C(bf16) = acc = [g | u], C2(bf16) = silu(g) * u
	// k-contiguous A only (see gemm_swiglu_bwd_bf16): R = [g | u] (bf16, N columns each), acc rounded to bf16 = d:
	EPI_BF16_SWIGLU_BWD = 5,  // C(bf16) = [d silu'(g) u | d silu(g)]
	// k-contiguous operands (see gemm_rope_bf16): C(bf16) = acc rounded to bf16, then the half-split rotary rotation of
	// the heads (width rope_D) that lie in the first rope_cols columns, position = row mod rope_S
	EPI_BF16_ROPE = 6,
	// both operands reduction-major, 256x256 direct-to-LDS tiles without a K split (see gemm_dw_final):
	EPI_F32_ACC_SCALE = 7,  // C(fp32) = (C + acc) * scale, C2(bf16) = bf16 of that
};

int gemm_bf16(int a_t, int b_t, int M, int N, int K, const void* A, int64_t lda, const void* B, int64_t ldb,
              void* C, int64_t ldc, int epi, const void* R, int64_t ldr, int tile_cfg, int k_splits,
              hipStream_t stream);

// 256x256 tile (bm = 256; 8 waves) or 128x256 tile (bm = 128; 4 waves, A k-contiguous) with direct global->LDS
// loads (gemm_dma.hip); called by gemm_bf16 for tile_cfg 7 and 8.
// EPI_F32_ACC only: the last tail_tiles tiles (all of them when tail_tiles < 0) are split k_splits ways along K.
int gemm_bf16_dma(int a_t, int b_t, int M, int N, int K, const void* A, int64_t lda, const void* B, int64_t ldb, void* C,
                  int64_t ldc, int epi, const void* R, int64_t ldr, int k_splits, int tail_tiles, int bm, hipStream_t stream,
                  void* C2 = nullptr, int64_t ldc2 = 0, const void* rope_cs = nullptr, int rope_S = 0, int rope_cols = 0, int rope_D = 0,
                  float scale = 1.f);

// The weight gradient of the step's last micro-batch with the step's gradient scale folded in: acc [M, N] (fp32, dense)
// = (acc + dY^T X) * scale and grad_bf16 [M, N] = bf16(acc), with dY [K, M] and X [K, N] (both reduction-major).  One
// kernel when the shape fills the chip with whole 256x256 tiles (the scale and the bf16 copy leave from the epilogue
// that holds the fp32 tile anyway); otherwise gemm_bf16 (epilogue 2) followed by scale_grads.  Same bits either way:
// one fp32 add, one fp32 multiply, one rounding to bf16 per element.
int gemm_dw_final(int M, int N, int K, const void* dY, int64_t lddy, const void* X, int64_t ldx, float* acc, void* grad_bf16, float scale,
                  hipStream_t stream);

// The W pass of a stage in one launch: for each of n (at most 16) problems acc [M, N] (fp32, dense) += dY^T X with
// dY [K, M] and X [K, N] over the same K tokens, on 256x256 tiles whose workgroups fill the chip together (one partly
// filled round per launch instead of one per layer; when that round would leave half of the chip idle its tiles are
// split along K and add in a fixed order).  scale != 0: every accumulator leaves multiplied by it, with its bf16 copy in
// grad_bf16 (from the epilogue for whole tiles, by a small kernel behind the launch for split ones: same bits).  gemm_dw_groupable: a problem's
// shape and operands fit (M, N multiples of 256, K of 64, 16-byte aligned, dense enough).
struct DwProblem {
	const void* dY;
	int64_t lddy;
	const void* X;
	int64_t ldx;
	float* acc;
	void* grad_bf16;  // may be null when scale == 0
	int M, N;
};
bool gemm_dw_groupable(int M, int N, int K, const void* dY, int64_t lddy, const void* X, int64_t ldx, const void* acc);
int gemm_dw_group(int n, const DwProblem* problems, int K, float scale, hipStream_t stream);

// The attention block's packed q | k | v projection with the rotary embedding of the q and k heads: C [M, N] =
// A W^T rounded to bf16, then rope_apply's rotation on the first n_rot_heads heads of width D (cs: the table of
// rope_table for sequence length S; row r is at position r mod S).  One kernel (rotation in the GEMM epilogue, the
// projection is not read back) when the shape fits the direct-to-LDS tiles; otherwise the GEMM is followed by the
// RoPE kernel.  Both ways give the same bits.
bool gemm_rope_fused(int M, int N, int K, int D);
int gemm_rope_bf16(int M, int N, int K, const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, const void* cs,
                   int S, int n_rot_heads, int D, hipStream_t stream);

// Tag of one GEMM launch whose tiles are split along K (24 bits, never 0, different from launch to launch); see the
// turn counters in gemm_dma.hip and gemm_bf16.hip.
uint32_t next_turn_tag();
// Waves / workgroups of split-K launches on the current device that used up their bounded wait for their turn and added
// out of turn (right sums, rounding order not fixed) since the library was loaded.  Synchronous (one 4-byte copy each
// from two device counters).
int gemm_turn_giveups(uint64_t* out);

enum Activation { ACT_GELU = 0, ACT_SWIGLU = 1 };
// Up-projection of the MLP with its activation: pre = A W^T (A [M, K], W [N, K], N = F for GELU and 2F =
// [gate rows; up rows] for SwiGLU), out [M, F] = gelu(pre) or silu(pre[:, :F]) * pre[:, F:].  SwiGLU runs
// as one kernel (activation in the GEMM epilogue) when the shape fits the direct-to-LDS tiles; otherwise,
// and for GELU (whose erf costs as much in the epilogue as in a kernel of its own), the GEMM is followed
// by the activation kernel.  Both ways give the same bits.
int gemm_act_bf16(int act, int M, int F, int K, const void* A, int64_t lda, const void* W, int64_t ldw, void* pre,
                  int64_t ldpre, void* out, int64_t ldout, hipStream_t stream);

// Backward of the MLP's down projection into its SwiGLU: dgu [M, 2F] = the gradient of [g | u] for
// d = dY W (dY [M, K], W [K, F] = the down projection's weight as it lies in memory), with gu [M, 2F] the saved
// gate/up product.  One kernel (activation backward in the GEMM epilogue, d never reaches memory) when the shape
// fits the direct-to-LDS tiles; otherwise the GEMM writes d into `scratch` [M, F] and the activation backward
// kernel follows.  Both ways give the same bits.  `scratch` may be null when gemm_swiglu_bwd_fused(M, F, K).
// act non-null: the activation silu(g) * u [M, F] (leading dim ldact) is written as well, with the bits of swiglu_fwd
// (a stash that dropped it after the forward gets it back from the g and u the epilogue reads anyway).
bool gemm_swiglu_bwd_fused(int M, int F, int K);
int gemm_swiglu_bwd_bf16(int M, int F, int K, const void* dY, int64_t lddy, const void* W, int64_t ldw, const void* gu,
                         int64_t ldgu, void* dgu, int64_t lddgu, void* scratch, hipStream_t stream, void* act = nullptr, int64_t ldact = 0);

enum NormKind { NORM_RMS = 0, NORM_LAYER = 1 };

// stats: float2 per row {mean, rstd}. workspace: norm_bwd_workspace_floats(T, d) floats.
int norm_fwd(int kind, const void* x, const void* gamma, const void* beta, void* y, void* stats, int T, int d,
             float eps, hipStream_t s);
int64_t norm_bwd_workspace_floats(int T, int d);
// y_out non-null (norm_bwd_forms_output(d) only: rows wider than 768): the norm's output is written again as well, with
// the forward's bits (a stash that dropped it gets it back from the row this pass reads anyway); LayerNorm then needs beta.
bool norm_bwd_forms_output(int d);
int norm_bwd(int kind, const void* dy, const void* x, const void* gamma, const void* stats, const void* dres,
             void* dx, float* dgamma, float* dbeta, float* workspace, int T, int d, hipStream_t s, const void* beta = nullptr,
             void* y_out = nullptr);
// The same with the partial sums in an array of the library's device image instead of a workspace argument
// (no allocation anywhere on the path); norm_bwd_scratch_prepare looks the array's address up for the
// current device (done by the first call on a device otherwise).
int norm_bwd_scratch_prepare();
int norm_bwd_noalloc(int kind, const void* dy, const void* x, const void* gamma, const void* stats, const void* dres,
                     void* dx, float* dgamma, float* dbeta, int T, int d, hipStream_t s);
int gelu_fwd(const void* x, void* y, int64_t n, hipStream_t s);
int gelu_bwd(const void* dy, const void* x, void* dx, int64_t n, hipStream_t s);
int swiglu_fwd(const void* gu, void* h, int64_t T, int F, hipStream_t s);
// act non-null: silu(g) * u [T, F] is written as well (the bits of swiglu_fwd)
int swiglu_bwd(const void* dh, const void* gu, void* dgu, int64_t T, int F, hipStream_t s, void* act = nullptr);
int rope_table(void* cs, int S, int D, double theta, hipStream_t s);
int rope_apply(void* buf, const void* cs, int64_t T, int S, int ld, int n_heads, int D, int backward, hipStream_t s);
int scale_grads(void* acc_f32, void* out_bf16, int64_t n, float scale, hipStream_t s);
int add_bf16(const void* a, const void* b, void* out, int64_t n, hipStream_t s);
// out[c] (fp32) += sum over the T rows of x[t, c] (bf16 [T, N], row stride ld)
int64_t colsum_workspace_floats(int64_t T, int N);
int colsum_bf16(const void* x, int64_t ld, void* out_f32, int64_t T, int N, float* workspace, hipStream_t s);
// ids: int64 [T]; table bf16 [V, d]; dtable fp32 [V, d] (+=)
int embedding_fwd(const void* ids, const void* table, void* out, int64_t T, int d, int V, hipStream_t s);
int embedding_bwd(const void* ids, const void* dx, void* dtable_f32, int64_t T, int d, int V, hipStream_t s);
// Cross-entropy over bf16 logits [rows, V] (row stride ld), loss and gradient in one pass; target int64 [rows].
int cross_entropy(const void* logits, int64_t ld, const void* target, int64_t rows, int64_t V, int64_t ignore_index, float scale,
                  const void* dev_div, void* row_loss, void* dlogits, int64_t ld_out, hipStream_t s);
int cross_entropy_reduce(const void* row_loss, const void* target, int64_t rows, int64_t ignore_index, void* out2, hipStream_t s);

// Attention over the packed projection layout; lse is [B, Hq, S] fp32 (natural log).
int attn_fwd(const void* q, const void* k, const void* v, void* o, void* lse, int64_t ldq, int64_t ldk, int64_t ldv,
             int64_t ldo, int B, int S, int Hq, int Hkv, int D, int causal, float scale, hipStream_t stream);
int64_t attn_bwd_workspace_bytes(int B, int S, int Hq, int D, int causal);
int attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dO, const void* lse, void* dq,
             void* dk, void* dv, void* workspace, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo,
             int64_t lddq, int64_t lddk, int64_t lddv, int B, int S, int Hq, int Hkv, int D, int causal, float scale,
             hipStream_t stream, const void* rope_cs = nullptr);
// rope_cs non-null: q and k are the rotated heads (rope_apply with this table); dq and dk come out as the gradients
// of the heads before the rotation (rope_apply's backward applied to them), bit-identical to the separate pass.

// Memory-system yardstick: read (mode 0; dst receives up to 8192 * 256 * 16 bytes of sums), copy (1) or write (2) `bytes`
// bytes with the simplest possible kernel.
int hbm_probe(int mode, const void* src, void* dst, int64_t bytes, hipStream_t s);

// Optional live timing of kernel launches: when enabled, every launcher brackets its launches
// with an event pair on the launch stream and books the algorithmic work of the call.
enum ProfKind {
	PROF_GEMM = 0, PROF_ATTN_FWD, PROF_ATTN_BWD, PROF_NORM_FWD, PROF_NORM_BWD, PROF_ACT_FWD, PROF_ACT_BWD, PROF_ROPE,
	PROF_SCALE, PROF_ADD, PROF_EMBED, PROF_LOSS, PROF_COUNT
};
void prof_enable(int on);  // 0 off, 1 every launch carries events, n > 1 one launch in n (pseudo-random, the same picks every run)
bool prof_on();
struct ProfScope {
	// record = false: an inert scope (launches inside it are not timed)
	ProfScope(int kind, double work, hipStream_t stream, bool record = true);
	~ProfScope();
	int slot;
	hipStream_t stream;
	ProfScope* outer;
};
// The timing events of the innermost open scope of this thread, to be attached to the next kernel launch: the start
// event for the scope's first launch only, the stop event for every launch (the last one keeps it).  False when
// nothing is being timed.
bool prof_launch_events(hipEvent_t* start, hipEvent_t* stop);

// A launch that carries its scope's timing events in the dispatch itself (hipExtLaunchKernel): the kernel's own start
// and end timestamps, with no barrier packets between the launches of a stream (an event recorded before and after
// each launch costs two of them, about 3 us per launch).
template <class... P, size_t... I, class... A>
inline void launch_timed(void (*kern)(P...), dim3 grid, dim3 block, unsigned smem, hipStream_t s, hipEvent_t e0, hipEvent_t e1,
                         std::index_sequence<I...>, A&&... a) {
	static_assert(sizeof...(P) == sizeof...(A), "kernel argument count");
	std::tuple<P...> formal{static_cast<P>(a)...};
	void* ptrs[] = {(void*)&std::get<I>(formal)...};
	(void)hipExtLaunchKernel(reinterpret_cast<const void*>(kern), grid, block, ptrs, smem, s, e0, e1, 0);
}
template <class... P, class... A>
inline void launch_kernel(void (*kern)(P...), dim3 grid, dim3 block, unsigned smem, hipStream_t s, A&&... a) {
	hipEvent_t e0 = nullptr, e1 = nullptr;
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	// a stream under graph capture takes plain launches only
	if (prof_launch_events(&e0, &e1) && hipStreamIsCapturing(s, &capture) == hipSuccess && capture == hipStreamCaptureStatusNone)
		launch_timed(kern, grid, block, smem, s, e0, e1, std::index_sequence_for<P...>{}, a...);
	else hipLaunchKernelGGL(kern, grid, block, smem, s, static_cast<P>(a)...);
}
#define ELF_LAUNCH(kern, grid, block, smem, stream, ...) elf::launch_kernel(kern, grid, block, smem, stream, __VA_ARGS__)
// Waits for the recorded events; totals over the timed launches since the last prof_enable. Returns their count.
int prof_collect(int kind, double* total_ms, double* total_work);
// All launches of the kind since prof_enable, timed or not, and their summed work.
int64_t prof_launches(int kind, double* total_work);

}  // namespace elf
