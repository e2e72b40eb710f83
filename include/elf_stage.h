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
 *   epilogue: 0 C(bf16) = acc; 1 C(bf16) = acc + R(bf16, leading dim ldr; ldr = 0: R is one row of N values
 *             added to every row of C, the bias of nn.Linear);
 *             2 C(fp32) += acc; 3 C(fp32) = acc.
 *   tile_cfg = 0 picks a tile shape from M,N (1: 256x256, 2: 128x128, 3: 64x64, 5: 256x128 register-staged;
 *   7: 256x256 with direct-to-LDS loads; 8: 128x256 with direct-to-LDS loads: a_t = 1 is accepted only together with
 *   b_t = 1, and k_splits is honoured for epilogue 2);
 *   k_splits = 0 picks a K split (epilogue 2 only; at most 255).
 * Replaces: F.linear in LinearDX.forward (elf/zb_utils.py:20)            -> a_t=0,b_t=0
 *           torch.mm(grad_output, weight) in LinearDX.backward (:34-37)  -> a_t=0,b_t=1
 *           torch.mm(go.t(), inp) + weight.grad.add_ in LinearDW.backward (:238-244) -> a_t=1,b_t=1, epilogue 2
 * M, N multiples of 64, K a multiple of 64, pointers 16-byte aligned. */
int elf_gemm_bf16(int a_t, int b_t, int M, int N, int K, const void* A, int64_t lda, const void* B,
                  int64_t ldb, void* C, int64_t ldc, int epilogue, const void* R, int64_t ldr,
                  int tile_cfg, int k_splits, void* stream);
/* Epilogue 2 with a split K: the workgroups that share a tile add their parts in the order of their K ranges (turn
 * counters in device memory, tagged per launch), so the fp32 sums are bit-identical from run to run.  The counters are
 * shared by every stream of the process: split-K launches that overlap in time on two streams can make a wave wait for a
 * turn that is not its launch's; the wait is bounded (about a millisecond), after which the wave adds out of turn - still
 * the right sum, but its rounding order is no longer fixed.  *out receives how many waves did so on the current device
 * since the library was loaded (0 as long as split-K launches do not overlap).  Synchronous.  No counterpart in the
 * reference (torch.mm's split-K is not reproducible either way). */
int elf_gemm_turn_giveups(uint64_t* out);

/* The weight gradients of several linear layers over the same K tokens in one launch: for problem i,
 * acc[M, N] (fp32, dense) += dY^T X with dY [K, M] (leading dim lddy) and X [K, N] (leading dim ldx), i.e. what n calls of
 * elf_gemm_bf16(1, 1, ..., epilogue 2) compute.  The workgroups of all problems fill the chip together: only the
 * launch's last round of 256 tiles is partly filled, and when it would be at most half full its tiles (the last ones of
 * the last problems) are split along K, up to 8 ways with at least 16 slices of 64 each; split tiles add in the order of
 * their K ranges (see elf_gemm_turn_giveups), so the sums are bit-identical from run to run.  A tile's sum is rounded
 * once per K range: the bits equal elf_gemm_bf16's when that call splits the tile the same way.
 * scale != 0: every acc leaves multiplied by scale and grad_bf16[M, N] receives its bf16 rounding (the step's last W
 * pass with PipelineBlock.scale_grads folded in, elf/execution/block.py:518-527); grad_bf16 may be NULL otherwise.
 * n <= 16; M, N multiples of 256, K of 64; pointers 16-byte aligned.
 * Replaces: the loop over LayerDW modules of PipelineBlock.backward_params (elf/execution/block.py:384-389), each
 *           iteration torch.mm(go.t(), inp) + weight.grad.add_ of LinearDW.backward (elf/zb_utils.py:238-244). */
typedef struct elf_dw_problem {
	const void* dY;
	int64_t lddy;
	const void* X;
	int64_t ldx;
	float* acc;
	void* grad_bf16;
	int M, N;
} elf_dw_problem;
int elf_gemm_dw_group(int n, const elf_dw_problem* problems, int K, float scale, void* stream);

/* The MLP's up-projection with its activation: pre = A W^T with A [M, K] and W [N, K], both k contiguous;
 * act 0 (GELU): N = F, out[M, F] = gelu(pre); act 1 (SwiGLU): N = 2F, W = [gate rows; up rows],
 * pre[M, 2F] = [g | u], out[M, F] = silu(g) * u.  pre is kept because the backward needs it.  SwiGLU is
 * computed in the GEMM epilogue (one kernel, the pre-activation never re-read); GELU, and shapes the
 * fused tiles do not cover (M not a multiple of 128, N not of 256, or too few tiles to fill the chip),
 * run elf_gemm_bf16 (epilogue 0) followed by elf_gelu_fwd / elf_swiglu_fwd.  Same bits either way.
 * Replaces: fc1 + nn.GELU() of the GPT block's MLP (benchmarks/models/simple.py:44-52) run through
 *           LinearDX.forward (elf/zb_utils.py:20); no reference module for SwiGLU. */
int elf_gemm_act_bf16(int act, int M, int F, int K, const void* A, int64_t lda, const void* W, int64_t ldw,
                      void* pre, int64_t ldpre, void* out, int64_t ldout, void* stream);
/* Backward of the down-projection into the SwiGLU: d = dY W with dY [M, K] and W [K, F] (the down
 * projection's weight [d_model, F] as it lies in memory), then dgu[M, 2F] = [d silu'(g) u | d silu(g)]
 * from the saved gu[M, 2F] = [g | u].  One kernel (activation backward in the GEMM epilogue, d never
 * reaches memory) when M and F are multiples of 256, K of 64 and the tiles fill the chip; otherwise
 * elf_gemm_bf16(0, 1, ...) into scratch [M, F] followed by elf_swiglu_bwd (scratch may be null only for
 * the fused shapes).  Same bits either way.
 * Replaces: LinearDX.backward of fc2 (elf/zb_utils.py:29-41) followed by autograd's backward of
 *           silu(gate) * up; no reference module for SwiGLU. */
int elf_gemm_swiglu_bwd_bf16(int M, int F, int K, const void* dY, int64_t lddy, const void* W, int64_t ldw,
                             const void* gu, int64_t ldgu, void* dgu, int64_t lddgu, void* scratch, void* stream);

/* The attention block's packed q | k | v projection with the rotary embedding of its q and k heads:
 * C[M, N] = A W^T (A [M, K], W [N, K], both k contiguous) rounded to bf16, then the rotation of elf_rope_apply
 * on the first n_rot_heads heads of width D (64 or 128); cs is the table of elf_rope_table for sequence length
 * S, row r of A is the token at position r mod S.  One kernel (rotation in the GEMM epilogue, the projection
 * is never read back) when M is a multiple of 128, N of 256, K of 64 and the tiles fill the chip; otherwise
 * elf_gemm_bf16 followed by elf_rope_apply.  Same bits either way.
 * Replaces: the q / k / v projections of the attention block run through LinearDX.forward
 *           (elf/zb_utils.py:20); no reference module for the rotary embedding. */
int elf_gemm_rope_bf16(int M, int N, int K, const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                       const void* cs, int S, int n_rot_heads, int D, void* stream);

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

/* elf_norm_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results
 * as elf_norm_bwd without the workspace: the per-workgroup partial sums of dgamma / dbeta go to a 64 MiB
 * array that is part of the library's device image (1024 partial rows of 2 x 8192 floats: enough for every
 * T and every d <= 8192 that elf_norm_bwd accepts; a shape that needs more is refused with an error), held
 * by every GPU the library runs on until the process ends.  The call allocates nothing on the host or the
 * device (kernel timing through elf_prof_enable does not cover it).  All calls on one GPU share the array:
 * calls that overlap in time on one GPU (different streams or host threads) race and must be serialised by
 * the caller.  Nothing in the array has to be cleared between calls (every partial row is written in full
 * before it is read). */
int elf_norm_bwd_noalloc(int kind, const void* dy, const void* x, const void* gamma, const void* stats,
                         const void* dres, void* dx, float* dgamma, float* dbeta, int T, int d, void* stream);

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

/* out_f32[c] += sum over the T rows of x[t, c] (x: bf16 [T, N], row stride ld; N and ld multiples of 8).
 * workspace: elf_colsum_workspace_floats(T, N) floats of partial sums, added by one writer per column in a fixed
 * order (equal bits from run to run).
 * Replaces the bias gradient of LinearDW.backward, go.sum(0) added to bias.grad (elf/zb_utils.py:247-252),
 * with fp32 accumulation. */
int64_t elf_colsum_workspace_floats(int64_t T, int N);
int elf_colsum_bf16(const void* x, int64_t ld, void* out_f32, int64_t T, int N, float* workspace, void* stream);

/* Token embedding of a first pipeline stage: out[t, :] = table[ids[t], :] (ids: int64 [T], table: bf16
 * [V, d], d % 8 == 0; an id outside [0, V) gives a zero row) and its weight gradient dtable[ids[t], :] +=
 * dx[t, :] in fp32.  Replaces nn.Embedding forward / backward (benchmarks/models/simple.py:496, 502). */
int elf_embedding_fwd(const void* ids, const void* table, void* out, int64_t T, int d, int V, void* stream);
int elf_embedding_bwd(const void* ids, const void* dx, void* dtable_f32, int64_t T, int d, int V, void* stream);

/* Cross-entropy of a last pipeline stage, loss and gradient in one pass over the logits.  Replaces the
 * reference's loss function (benchmarks/models/simple.py:520-524: upcast to fp32, flatten,
 * torch.nn.functional.cross_entropy) and its backward as Engine.compute_loss runs them
 * (elf/execution/engine.py:374-410).
 *   logits   bf16 [rows, V], row stride ld elements (ld % 8 == 0, base 16-byte aligned)
 *   target   int64 [rows]; rows with target == ignore_index contribute no loss and a zero gradient;
 *            any other target outside [0, V) makes that row's loss NaN
 *   row_loss fp32 [rows] or NULL:  logsumexp(logits[r, :]) - logits[r, target[r]], arithmetic in fp32
 *   dlogits  bf16 [rows, ld_out] or NULL (ld_out % 8 == 0, >= V; must not overlap logits):
 *            (softmax(logits[r, :]) - onehot(target[r])) * scale / (dev_div ? *dev_div : 1), columns
 *            V .. ld_out-1 are written as zeros
 *   dev_div  optional device fp32 scalar (e.g. the count of non-ignored rows for reduction="mean")
 * elf_cross_entropy_reduce: out2[0] = sum of row_loss (untouched when row_loss is NULL), out2[1] =
 * number of rows whose target is not ignore_index; fixed summation order (bit-reproducible). */
int elf_cross_entropy(const void* logits, int64_t ld, const void* target, int64_t rows, int64_t V, int64_t ignore_index, float scale,
                      const void* dev_div, void* row_loss, void* dlogits, int64_t ld_out, void* stream);
int elf_cross_entropy_reduce(const void* row_loss, const void* target, int64_t rows, int64_t ignore_index, void* out2, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Attention on the packed projection layout: q/k/v/o are column slices of [T, ld*] bf16 buffers,
 * T = B*S tokens, head h at columns [h*D, (h+1)*D).  Hq % Hkv == 0 (grouped-query attention),
 * D in {64, 128}, S % 128 == 0.  lse: fp32 [B, Hq, S] (natural log of the softmax denominator).
 * Replaces SDPA / softmax(QK^T*scale)V forward and its autograd backward
 * (benchmarks/models/simple.py:362-367, 379-386).  The backward needs
 * elf_attn_bwd_workspace_bytes() of 16-byte aligned scratch (the bf16 partial dQ of every 128-key tile,
 * which a second kernel sums in fp32 in a fixed order — no atomics, run-to-run identical gradients —
 * plus two fp32 values per query and head): B * S * (S/128 + 1) / 2 * Hq * D * 2 bytes with a causal
 * mask, B * S * (S/128) * Hq * D * 2 without, + 8 * B * S * Hq. */
int elf_attn_fwd(const void* q, const void* k, const void* v, void* o, void* lse, int64_t ldq,
                 int64_t ldk, int64_t ldv, int64_t ldo, int B, int S, int Hq, int Hkv, int D,
                 int causal, float scale, void* stream);
int64_t elf_attn_bwd_workspace_bytes(int B, int S, int Hq, int D, int causal);
int elf_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dO,
                 const void* lse, void* dq, void* dk, void* dv, void* workspace, int64_t ldq,
                 int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo, int64_t lddq, int64_t lddk,
                 int64_t lddv, int B, int S, int Hq, int Hkv, int D, int causal, float scale,
                 void* stream);

/* elf_attn_bwd for q and k heads that carry a rotary embedding (q, k are the rotated heads as elf_rope_apply /
 * elf_gemm_rope_bf16 left them; cs is that table): dq and dk come out as the gradients of the heads BEFORE the
 * rotation, i.e. with elf_rope_apply(..., backward = 1) already applied where they are stored (the dQ reduction and
 * the dK epilogue), bit-identical to elf_attn_bwd followed by that call.  cs = NULL is elf_attn_bwd.
 * No reference module for the rotary embedding; replaces the autograd backward of the rotation. */
int elf_attn_bwd_rope(const void* q, const void* k, const void* v, const void* o, const void* dO,
                      const void* lse, void* dq, void* dk, void* dv, void* workspace, int64_t ldq,
                      int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo, int64_t lddq, int64_t lddk,
                      int64_t lddv, int B, int S, int Hq, int Hkv, int D, int causal, float scale,
                      const void* cs, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Stage executor: one pipeline stage = n_blocks transformer blocks on T = mb * seq tokens.
 * It is what PipelineBlock (elf/execution/block.py:134-694) does through nn.Module.__call__ and
 * autograd, with the LinearDX / LinearDW split backward (elf/zb_utils.py:9-256) made explicit.
 * The caller (torch) owns the boundary tensors X, Y, dY, dX, the weights and the fp32 gradient
 * accumulators; the library owns the per-micro-batch activation stash, the W stash (input X and
 * output gradient dY of every linear layer), temporaries, the pinned-host arena and the two side
 * streams of activation offload.  All calls for one stage come from one host thread and use ONE
 * stream for the stage's whole life (the offload copies, the release of pinned blocks and the reuse of
 * pooled device blocks are ordered against that stream only; a caller that must change streams
 * synchronises the device first).  The fp32 gradient accumulators, too, are updated by plain
 * read-modify-writes with one writer per element: two streams must not accumulate into the same
 * gradient buffer at the same time.  The external X of a micro-batch must stay valid until its B (and until its recompute
 * ops), the external dY until its W. */
typedef struct elf_stage elf_stage_t;

enum { ELF_ARCH_GPT = 0, ELF_ARCH_LLAMA = 1 };
/*  GPT block   (benchmarks/models/simple.py:437-468, dropout off): LayerNorm, bias-free q/k/v/o
 *              projections, multi-head attention, GELU FFN, two residual adds.
 *  Llama block (no reference module): RMSNorm, RoPE (half-split), grouped-query attention,
 *              SwiGLU FFN. */
typedef struct elf_stage_cfg {
	int arch;        /* ELF_ARCH_* */
	int n_blocks;
	int d_model;
	int n_heads;     /* query heads */
	int n_kv_heads;  /* == n_heads for ELF_ARCH_GPT */
	int head_dim;    /* 64 or 128; the attention width n_heads*head_dim may differ from d_model */
	int ffn;         /* FFN hidden size F */
	int seq;         /* tokens per sequence, multiple of 128 */
	int mb;          /* sequences per micro-batch */
	int causal;
	float eps;
	double rope_theta;
} elf_stage_cfg;

/* Parameter ids for elf_stage_bind_param (weights bf16 row-major [out, in], as nn.Linear):
 *  0 norm1 gamma [d]   1 norm1 beta [d] (GPT only)   2 Wqkv [(Hq+2Hkv)*D, d] (q rows, k rows, v rows)
 *  3 Wo [d, Hq*D]      4 norm2 gamma    5 norm2 beta (GPT only)
 *  6 W1 [F, d] (GPT fc1)  or  [2F, d] (Llama: gate rows then up rows)     7 W2 [d, F] */
enum { ELF_P_NORM1_G = 0, ELF_P_NORM1_B, ELF_P_WQKV, ELF_P_WO, ELF_P_NORM2_G, ELF_P_NORM2_B, ELF_P_W1, ELF_P_W2, ELF_P_COUNT };
/* Stage-level parameters of a first / last pipeline stage, bound with block = -1:
 *  8 token embedding [vocab_in, d]   9 final norm gamma [d]   10 final norm beta [d] (GPT only)
 *  11 output head [vocab_out_ld, d] (rows >= vocab_out are padding and must be zero) */
enum { ELF_P_EMBED = 8, ELF_P_FNORM_G, ELF_P_FNORM_B, ELF_P_HEAD };

/* Forward flags (FORWARD options, elf/scheduling/scheduling.py:58-86).  remat_strategy selects modules
 * whose forward runs under checkpoint(): what they keep for the backward is not kept, and the backward
 * runs them again (elf/execution/remat.py:26-74).  The strategies the benchmarks build
 * (benchmarks/benchmark_utils.py:295-335) map onto:
 *  REMAT_ROOT: the whole stage (name == "", "full"): only the stage input is kept and B re-runs the
 *              forward;
 *  REMAT_ATTN: the attention cores ("selective"): the attention output and log-sum-exp of every block
 *              are dropped after F and B runs the attention forward again from the kept q, k, v (same
 *              kernel on the same inputs: bit-identical);
 *  REMAT_NORM: the norm modules ("simple": LayerNorm; a GELU module keeps nothing but its own input, which
 *              the FFN pre-activation stash holds either way): the per-row statistics of every norm are
 *              dropped after F and B runs the norm forward again;
 *  OFFLOAD:    activation_offload: the stash goes to pinned host memory on a side stream
 *              (elf/execution/offload.py:228-268, 330-352).
 * REMAT_ROOT overrides the other two. */
enum { ELF_FWD_REMAT_ROOT = 1u, ELF_FWD_REMAT_ATTN = 2u, ELF_FWD_OFFLOAD = 4u, ELF_FWD_REMAT_NORM = 8u };
/* BACKWARD_INPUTS flags: recompute_activations drops the W-stash inputs after B,
 * recompute_gradients drops the W-stash output gradients (elf/execution/block.py:659-694). */
enum { ELF_BWD_RECOMPUTE_ACTIVATIONS = 1u, ELF_BWD_RECOMPUTE_GRADIENTS = 2u };

typedef struct elf_mem_stats {
	int64_t live_bytes;      /* device bytes held by stashes and temporaries now */
	int64_t peak_bytes;      /* high-water mark of live_bytes since create / reset_peak */
	int64_t reserved_bytes;  /* device bytes obtained from the driver (live + cached) */
	int64_t pinned_bytes;    /* size of the pinned-host arena */
	int64_t d2h_bytes;       /* total bytes offloaded */
	int64_t h2d_bytes;       /* total bytes brought back */
	int64_t workspace_bytes; /* fixed device scratch allocated at create (attention / norm backward, rope table) */
} elf_mem_stats;

int elf_stage_create(const elf_stage_cfg* cfg, elf_stage_t** out);
void elf_stage_destroy(elf_stage_t* s);
/* torch keeps ownership; grad_f32 is the fp32 accumulator of the same shape as the weight. */
int elf_stage_bind_param(elf_stage_t* s, int block, int which, void* weight_bf16, void* grad_f32);
/* First / last stage of a pipeline (FullTransformer.embed / .head, benchmarks/models/simple.py:496-509);
 * call once after elf_stage_create.  vocab_in > 0: the stage input x of F / B / RF is int64 token ids [T]
 * instead of activations, B adds the embedding gradient to its fp32 accumulator and writes no dx (dx may be
 * NULL).  vocab_out > 0: the stage output y is bf16 logits [T, vocab_out_ld] (vocab_out_ld a multiple of
 * 64, columns >= vocab_out are zero) and dy is their gradient in the same layout; final_norm != 0 puts a
 * norm of the architecture's kind in front of the head. */
int elf_stage_set_ends(elf_stage_t* s, int vocab_in, int vocab_out, int vocab_out_ld, int final_norm);
/* Number of sequences in micro-batch mb when it is smaller than cfg.mb: the last micro-batch of a
 * batch that the split size does not divide, or an explicit list of sizes (Pipeline._get_mb_sizes,
 * elf/pipeline.py:477-504; Engine.train_step splits the batch by those sizes, engine.py:123-160).
 * Every buffer of that micro-batch then has T = samples * seq rows.  Call before the micro-batch's F;
 * the value holds until it is set again or elf_stage_clear; unset micro-batches have cfg.mb. */
int elf_stage_set_mb_samples(elf_stage_t* s, int mb, int samples);
/* Lean stash (no counterpart in the reference, where autograd decides what a forward keeps).  Level 1: a
 * forward that keeps its activations drops the two norm outputs and the FFN activation of every block
 * (a third of the stash at the Llama shapes) and backward_inputs writes them again where W needs them, from
 * passes that read their inputs anyway (the norms' backward kernels, the SwiGLU backward's epilogue) and with
 * the forward's arithmetic: same results bit for bit, under 1 % of a block's B time.  Level 2 also drops the
 * QKV projection's output and the attention residual (a quarter of what level 1 keeps); backward_inputs forms
 * them again with the forward's own two GEMM calls (bit for bit; about 5 % of a block's F + B + W time): worth it
 * where the memory it frees saves whole recomputed forwards.  Level 0 keeps everything.  For stages that run under
 * a memory budget; applies to forwards issued after the call. */
int elf_stage_set_lean_stash(elf_stage_t* s, int level);
/* F: PipelineBlock.forward (block.py:210-279). x, y: bf16 [T, d_model]. */
int elf_stage_forward(elf_stage_t* s, int mb, const void* x, void* y, uint32_t flags, void* stream);
/* B: PipelineBlock.backward_inputs (block.py:624-694, 281-306). dy, dx: bf16 [T, d_model]; x is the
 * stage input again (needed when the forward was checkpointed; may be NULL otherwise). */
int elf_stage_backward_inputs(elf_stage_t* s, int mb, const void* x, const void* dy, void* dx, uint32_t flags, void* stream);
/* W: PipelineBlock.backward_params + LinearDW.backward (block.py:376-391, zb_utils.py:215-256):
 * grad_f32 += dY^T X for every linear layer, then the W stash of the micro-batch is dropped. */
int elf_stage_backward_params(elf_stage_t* s, int mb, void* stream);
/* W of the step's LAST micro-batch with the step's gradient scale folded in: every linear layer's accumulator leaves
 * the pass as (grad_f32 + dY^T X) * scale, and bf16(grad_f32) is written to the buffer bound with
 * elf_stage_bind_grad_bf16 (same shape as the weight).  Replaces that W followed by PipelineBlock.scale_grads
 * (block.py:518-527: grad /= batch size at ALL_REDUCE_PARAM_GRADS) for the linear layers, bit for bit, without the
 * extra pass over every gradient; the norm gains / biases and the token embedding, whose gradients accumulate in B, are
 * still scaled by elf_scale_grads.  The caller decides which W is the last one (the schedule is static). */
int elf_stage_bind_grad_bf16(elf_stage_t* s, int block, int which, void* grad_bf16);
int elf_stage_backward_params_scaled(elf_stage_t* s, int mb, float scale, void* stream);
/* RF: PipelineBlock.recompute_forward (block.py:308-338). save = 0 refills only the W-stash inputs,
 * save != 0 rebuilds the whole activation stash. */
int elf_stage_recompute_forward(elf_stage_t* s, int mb, const void* x, int save, void* stream);
/* RB*: PipelineBlock.recompute_backward_inputs + partial_dx_recomputation (block.py:340-374,
 * zb_utils.py:584-604): refills the W-stash output gradients; no norm gradients, no stage dX. */
int elf_stage_recompute_backward_inputs(elf_stage_t* s, int mb, const void* dy, void* stream);
/* Offload life cycle (OffloadToCPU, offload.py:166-411): offload is also implied by
 * ELF_FWD_OFFLOAD; prefetch = PREFETCH_ACTIVATIONS; release returns the pinned blocks.  Of the
 * stash, the two norm outputs, the FFN activation, the QKV projection's output and the attention
 * residual (x + o Wo^T) are not copied: backward_inputs forms them again from the restored buffers
 * with the forward's own kernel calls (bit-identical).  A prefetch brings the FFN pre-activation
 * back in row chunks and backward_inputs works through it chunk by chunk as they arrive. */
int elf_stage_offload(elf_stage_t* s, int mb, void* stream);
int elf_stage_prefetch(elf_stage_t* s, int mb, void* stream);
int elf_stage_release(elf_stage_t* s, int mb);
/* Grow the stage's pinned-host arena by one chunk of `bytes` now, so that the first offloaded micro-batches
 * do not pay for hipHostMalloc inside the step: what ELF_PREALLOCATE_POOL asks of the reference's pool
 * (preallocate_pool, elf/execution/engine.py:71-93; PinnedHostTensorPool.reserve, offload.py:45-70: the
 * chunk has exactly the requested size, not the next power of two). */
int elf_stage_reserve_pinned(elf_stage_t* s, int64_t bytes);
/* Drop every micro-batch state (Pipeline.step clears all slots after a step, pipeline.py:265-275). */
int elf_stage_clear(elf_stage_t* s);
int elf_stage_mem_stats(elf_stage_t* s, elf_mem_stats* out);
int elf_stage_reset_peak(elf_stage_t* s);

/* Pinned-host arena with the placement rules of PinnedHostTensorPool (offload.py:14-158).
 * host_backing != 0 backs it with malloc so the rules can be exercised without a GPU.
 * elf_pinned_pool_free returns 1 (and does nothing) for a pointer that is not a live block. */
typedef struct elf_pinned_pool elf_pinned_pool_t;
int elf_pinned_pool_create(int host_backing, elf_pinned_pool_t** out);
void elf_pinned_pool_destroy(elf_pinned_pool_t* p);
int elf_pinned_pool_allocate(elf_pinned_pool_t* p, int64_t elems, int elem_size, int dtype_key, void** ptr, int* parent, int64_t* offset);
int elf_pinned_pool_free(elf_pinned_pool_t* p, void* ptr);
int elf_pinned_pool_reserve(elf_pinned_pool_t* p, int64_t bytes, int elem_size, int dtype_key);
int64_t elf_pinned_pool_size(elf_pinned_pool_t* p);
int elf_pinned_pool_n_parents(elf_pinned_pool_t* p);
int elf_pinned_pool_n_free(elf_pinned_pool_t* p, int parent);
int elf_pinned_pool_free_segment(elf_pinned_pool_t* p, int parent, int i, int64_t* offset, int64_t* length);

/* ---------------------------------------------------------------------------------------------
 * Live kernel timing for measurements (no counterpart in the reference, whose per-op Timer wraps
 * whole F/B/W passes, elf/utils.py:249-324).  While enabled, every kernel launcher brackets its
 * launch with a HIP event pair on the launch stream.  kind: 0 GEMM (work = 2MNK flops),
 * 1 attention fwd, 2 attention bwd (algorithmic flops), 3 norm fwd, 4 norm bwd, 5 activation fwd,
 * 6 activation bwd, 7 RoPE, 8 grad scale, 9 add (work = algorithmic bytes).
 * elf_prof_enable(0) switches the timing off, (1) on for every launch, (n > 1) on for one launch in n, picked
 * pseudo-randomly (the same picks every run): an event pair carried in a dispatch costs the stream about 2 us.
 * elf_prof_collect waits for the events and returns the number of TIMED launches of that kind since
 * elf_prof_enable, with their summed duration (ms) and summed work; elf_prof_launches returns the number of
 * ALL launches of the kind since then and their summed work. */
/* Memory-system yardstick for the bandwidth-bound kernels (no counterpart in the reference): mode 0 reads `bytes`
 * bytes from src (dst receives at most 8192 * 256 * 16 bytes of per-lane sums), mode 1 copies them to dst, mode 2 writes
 * `bytes` bytes to dst, mode 3 reads three streams of `bytes` bytes each (src, src + bytes, src + 2 bytes: src holds
 * 3 * bytes) and writes their XOR to dst (the traffic pattern of a normalisation backward with a residual gradient);
 * 16-byte accesses, each workgroup on contiguous chunks of 16 or 32 KiB.  bench.py --hbm-ceiling times it. */
int elf_hbm_probe(int mode, const void* src, void* dst, int64_t bytes, void* stream);
void elf_prof_enable(int on);
int elf_prof_collect(int kind, double* total_ms, double* total_work);
int64_t elf_prof_launches(int kind, double* total_work);

#ifdef __cplusplus
}
#endif
#endif /* ELF_STAGE_H */
