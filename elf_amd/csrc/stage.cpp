// Stage executor: the per-micro-batch F / B / W / recompute / offload operations of one pipeline
// stage made of transformer blocks, as a sequence of HIP kernel launches on one stream.
//
// What the reference does with nn.Module.__call__ + autograd inside PipelineBlock
// (elf/execution/block.py:210-391, 624-694) and LinearDX/LinearDW (elf/zb_utils.py:9-256) is done
// here explicitly:
//   F  keeps, per block, what B needs (the "activation stash");
//   B  computes the input gradient and leaves, per linear layer, its input X and its output
//      gradient dY (the "W stash", the reference's LayerDW.ctx["input"] / ctx["grad_output"]);
//      norm weight gradients are accumulated here, as autograd does in the reference;
//   W  accumulates dW += dY^T X in fp32 for the four linear layers of every block and drops the
//      W stash.
// Remat and offload variants follow the options of elf/scheduling/scheduling.py:58-86.
#include <map>
#include <memory>
#include <vector>

#include "../../include/elf_stage.h"
#include "common.h"
#include "kernels.h"
#include "pools.h"

namespace elf {

enum BufId {
	B_X = 0,    // block input (owned by the stage for blocks > 0)
	B_ST1,      // norm1 statistics
	B_H1,       // norm1 output = input of the QKV projection
	B_QKV,      // packed projections (after RoPE for the llama block)
	B_O,        // attention output = input of the output projection
	B_LSE,      // attention log-sum-exp
	B_X2,       // x + attention branch
	B_ST2,      // norm2 statistics
	B_H2,       // norm2 output = input of the FFN up projection
	B_GU,       // FFN pre-activation ([T,2F] gate|up for SwiGLU, [T,F] for GELU)
	B_A,        // FFN activation = input of the down projection
	B_DY,       // gradient of the block output = dY of the down projection
	B_DGU,      // dY of the up projection
	B_DX2,      // dY of the output projection
	B_DQKV,     // dY of the QKV projection
	B_COUNT
};
static const unsigned ACT_MASK = (1u << B_X) | (1u << B_ST1) | (1u << B_H1) | (1u << B_QKV) | (1u << B_O) | (1u << B_LSE) |
                                 (1u << B_X2) | (1u << B_ST2) | (1u << B_H2) | (1u << B_GU) | (1u << B_A);
static const unsigned WIN_MASK = (1u << B_H1) | (1u << B_O) | (1u << B_H2) | (1u << B_A);
// Outputs of one bandwidth-bound kernel over a buffer that is kept anyway (norm of the block input, norm of
// the attention residual, activation of the gate/up product) and read by W only: an offloaded micro-batch
// drops them after F and B forms them again from the restored inputs instead of moving them over the host
// link twice (a third of the stash bytes; the same kernels on the same inputs: bit-identical).  A stage with a
// lean stash (elf_stage_set_lean_stash) does the same for every micro-batch, to hold less between F and B.
static const unsigned REFORM_MASK = (1u << B_H1) | (1u << B_H2) | (1u << B_A);
// An offloaded micro-batch (and every micro-batch of a stage at lean level 2) also leaves out the outputs of the two
// projections that a GEMM over buffers it holds anyway
// gives back for a third of their link time: the QKV projection's output (one GEMM over the re-formed norm output, plus
// RoPE: 1.0 ms against 2 x 3.4 ms of link time for its 168 MB at the 70B shape) and the attention residual x2 = x + o Wo^T
// (0.8 ms against 2 x 2.7 ms for 134 MB; the forward's own GEMM call with its residual epilogue: bit-identical).
static const unsigned OFFLOAD_REFORM_MASK = REFORM_MASK | (1u << B_QKV) | (1u << B_X2);
static const unsigned WGRAD_MASK = (1u << B_DY) | (1u << B_DGU) | (1u << B_DX2) | (1u << B_DQKV);

enum ParamId { P_NORM1_G = 0, P_NORM1_B, P_WQKV, P_WO, P_NORM2_G, P_NORM2_B, P_W1, P_W2, P_COUNT };
// stage-level parameters of a first / last pipeline stage (ELF_P_EMBED .. ELF_P_HEAD - ELF_P_EMBED)
enum EndParamId { XP_EMBED = 0, XP_FNORM_G, XP_FNORM_B, XP_HEAD, XP_COUNT };

struct Buf {
	void* p = nullptr;
	size_t bytes = 0;
	bool owned = false;
	PinnedPool::Block host;  // valid while offloaded
	bool offloaded = false;
	bool dropped = false;  // REFORM_MASK buffer of an offloaded micro-batch: B forms it again
};

struct BlockState {
	Buf b[B_COUNT];
	// offload copies run block by block: this block's device->host copies are done at off_ev; its host->device copies
	// come in the order B needs them: the FFN pre-activation in row chunks (pre_gu[c] after chunk c: B's activation
	// backward and the GEMM behind it run chunk by chunk while the rest is still on the link), then everything else (pre_ev)
	static constexpr int MAX_GU_CHUNKS = 4;
	hipEvent_t off_ev = nullptr, pre_ev = nullptr, pre_gu[MAX_GU_CHUNKS] = {};
	int gu_chunks = 1;  // row chunks of the last restore
};

struct MbState {
	std::vector<BlockState> blk;
	// last stage: the output head.  B_X / B_ST1 = input and statistics of the final norm, B_H1 = input
	// of the head linear (the last block's output when there is no final norm), B_DQKV = gradient of
	// the logits (caller-owned, like the stage's dY)
	BlockState head;
	const void* ids = nullptr;  // first stage: the token ids of the micro-batch (caller-owned)
	bool has_acts = false, has_win = false, has_wgrad = false;
	bool remat_root = false;  // forward kept nothing: B re-runs it
	bool offloaded = false, prefetched = false;
};

struct BlockParams {
	void* w[P_COUNT] = {};
	float* g[P_COUNT] = {};
	void* g16[P_COUNT] = {};  // bf16 copies of the scaled gradients (elf_stage_bind_grad_bf16), linear layers only
};

enum FwdMode { SAVE_ALL, SAVE_WIN, SAVE_NONE };

struct Stage {
	elf_stage_cfg cfg;
	int T, d, Hq, Hkv, D, F, S, B, nqkv, ffn_in;
	bool llama;
	std::vector<BlockParams> params;
	// first / last stage of a pipeline (elf_stage_set_ends): token embedding in front of block 0,
	// optional final norm + output head behind the last block (logits [T, vld], vld >= vocab_out)
	int vocab_in = 0, vocab_out = 0, vld = 0;
	bool final_norm = false;
	int lean = 0;  // elf_stage_set_lean_stash: F keeps no REFORM_MASK (1) / OFFLOAD_REFORM_MASK (2) buffer, B forms them again
	void* xw[XP_COUNT] = {};
	float* xg[XP_COUNT] = {};
	void* xg16[XP_COUNT] = {};
	std::map<int, MbState> mbs;
	// micro-batches with fewer sequences than cfg.mb (the last one of a batch the split size does not
	// divide): T and B above are set from here at every entry point (one host thread per stage)
	std::map<int, int> mb_samples;
	DevicePool pool;
	std::unique_ptr<PinnedPool> pinned;
	hipStream_t offload_stream = nullptr, prefetch_stream = nullptr;
	void* rope_cs = nullptr;
	float* norm_ws = nullptr;
	void* attn_ws = nullptr;
	int64_t ws_bytes = 0;  // fixed device workspaces of the stage (norm / attention backward scratch, rope table, gradient sink)
	float* dummy_grad = nullptr;  // sink for norm weight gradients during gradient recompute
	// pinned blocks of released micro-batches whose last copy may still be in flight: they go back to the arena
	// when their event has fired (polled, never waited for inside a step unless the arena would have to grow)
	struct HostPending {
		hipEvent_t ev;
		std::vector<void*> ptrs;
	};
	std::vector<HostPending> host_pending;
	int64_t d2h_bytes = 0, h2d_bytes = 0;

	size_t buf_bytes(int id) const {
		switch (id) {
			case B_X: case B_H1: case B_X2: case B_H2: case B_DY: case B_DX2: return (size_t)T * d * 2;
			case B_ST1: case B_ST2: return (size_t)T * 2 * 4;
			case B_QKV: case B_DQKV: return (size_t)T * nqkv * 2;
			case B_O: return (size_t)T * Hq * D * 2;
			case B_LSE: return (size_t)B * Hq * S * 4;
			case B_GU: case B_DGU: return (size_t)T * ffn_in * 2;
			case B_A: return (size_t)T * F * 2;
		}
		return 0;
	}
};

#define ELF_TRY(expr)            \
	do {                         \
		int _rc = (expr);        \
		if (_rc) return _rc;     \
	} while (0)

// A pool temporary of one function: returned on every path out of it (release() hands it back early).
struct PoolTmp {
	DevicePool& pool;
	void* p;
	PoolTmp(DevicePool& pl, size_t bytes) : pool(pl), p(bytes ? pl.alloc(bytes) : nullptr) {}
	~PoolTmp() { pool.free(p); }
	PoolTmp(const PoolTmp&) = delete;
	PoolTmp& operator=(const PoolTmp&) = delete;
	void release() {
		pool.free(p);
		p = nullptr;
	}
};

static int buf_alloc(Stage* s, BlockState& bs, int id) {
	Buf& b = bs.b[id];
	if (b.p && b.owned) return 0;
	b.dropped = false;
	b.bytes = s->buf_bytes(id);
	b.p = s->pool.alloc(b.bytes);
	if (!b.p) return -3;
	b.owned = true;
	return 0;
}
static void buf_free(Stage* s, BlockState& bs, int id) {
	Buf& b = bs.b[id];
	if (b.p && b.owned) s->pool.free(b.p);  // a pinned copy, if any, stays until release
	b.p = nullptr;
	b.owned = false;
}
static void free_mask(Stage* s, MbState& m, unsigned mask) {
	for (int id = 0; id < B_COUNT; id++)
		if (mask & (1u << id)) buf_free(s, m.head, id);
	for (auto& bs : m.blk)
		for (int id = 0; id < B_COUNT; id++)
			if (mask & (1u << id)) buf_free(s, bs, id);
}

static MbState& mb_state(Stage* s, int mb) {
	MbState& m = s->mbs[mb];
	if (m.blk.empty()) m.blk.resize(s->cfg.n_blocks);
	return m;
}

static void use_mb(Stage* s, int mb) {
	auto it = s->mb_samples.find(mb);
	s->B = it == s->mb_samples.end() ? s->cfg.mb : it->second;
	s->T = s->B * s->S;
}

static void destroy_events(MbState& m) {
	for (auto& bs : m.blk) {
		if (bs.off_ev) (void)hipEventDestroy(bs.off_ev);
		if (bs.pre_ev) (void)hipEventDestroy(bs.pre_ev);
		for (auto& ev : bs.pre_gu) {
			if (ev) (void)hipEventDestroy(ev);
			ev = nullptr;
		}
		bs.off_ev = bs.pre_ev = nullptr;
	}
}

static int do_offload_block(Stage* s, BlockState& bs, hipStream_t st);

// Return the pinned blocks whose guarding event has fired (all of them, waiting, when `wait`).
static void poll_host_pending(Stage* s, bool wait) {
	for (size_t i = 0; i < s->host_pending.size();) {
		auto& hp = s->host_pending[i];
		const hipError_t e = wait ? hipEventSynchronize(hp.ev) : hipEventQuery(hp.ev);
		if (e == hipSuccess) {
			for (void* p : hp.ptrs) s->pinned->free(p);
			(void)hipEventDestroy(hp.ev);
			s->host_pending[i] = std::move(s->host_pending.back());
			s->host_pending.pop_back();
		} else {
			(void)hipGetLastError();
			i++;
		}
	}
}

// ---------------------------------------------------------------------------------------------
// remat: ELF_FWD_REMAT_ATTN / ELF_FWD_REMAT_NORM of a forward that keeps its stash: the buffers those module
// checkpoints stand for are dropped block by block and run_backward forms them again.
static int run_forward(Stage* s, MbState& m, const void* x, void* y, FwdMode mode, hipStream_t st, bool offload = false, unsigned remat = 0) {
	unsigned remat_drop = 0;
	if (mode == SAVE_ALL && (remat & ELF_FWD_REMAT_ATTN)) remat_drop |= (1u << B_O) | (1u << B_LSE);
	if (mode == SAVE_ALL && (remat & ELF_FWD_REMAT_NORM)) remat_drop |= (1u << B_ST1) | (1u << B_ST2);
	auto drop = [&](BlockState& bs, unsigned mask) {
		for (int id = 0; id < B_COUNT; id++)
			if ((mask & (1u << id)) && bs.b[id].p && bs.b[id].owned) {
				buf_free(s, bs, id);
				bs.b[id].dropped = true;
			}
	};
	const int nb = s->cfg.n_blocks;
	const int T = s->T, d = s->d, F = s->F;
	const int norm_kind = s->llama ? NORM_RMS : NORM_LAYER;
	const float scale = 1.0f / sqrtf((float)s->D);
	for (int i = 0; i < nb; i++) {
		BlockState& bs = m.blk[i];
		const BlockParams& p = s->params[i];
		if (i == 0) {
			if (s->vocab_in) {
				m.ids = x;
				ELF_TRY(buf_alloc(s, bs, B_X));
				ELF_TRY(embedding_fwd(x, s->xw[XP_EMBED], bs.b[B_X].p, T, d, s->vocab_in, st));
			} else {
				bs.b[B_X].p = const_cast<void*>(x);
				bs.b[B_X].owned = false;
				bs.b[B_X].bytes = s->buf_bytes(B_X);
			}
		}
		const void* xin = bs.b[B_X].p;
		ELF_TRY(buf_alloc(s, bs, B_ST1));
		ELF_TRY(buf_alloc(s, bs, B_H1));
		ELF_TRY(norm_fwd(norm_kind, xin, p.w[P_NORM1_G], p.w[P_NORM1_B], bs.b[B_H1].p, bs.b[B_ST1].p, T, d, s->cfg.eps, st));
		ELF_TRY(buf_alloc(s, bs, B_QKV));
		// the packed projection, with the rotary embedding of the q and k heads in the GEMM's epilogue where the shape allows
		if (s->llama) ELF_TRY(gemm_rope_bf16(T, s->nqkv, d, bs.b[B_H1].p, d, p.w[P_WQKV], d, bs.b[B_QKV].p, s->nqkv, s->rope_cs, s->S, s->Hq + s->Hkv, s->D, st));
		else ELF_TRY(gemm_bf16(0, 0, T, s->nqkv, d, bs.b[B_H1].p, d, p.w[P_WQKV], d, bs.b[B_QKV].p, s->nqkv, EPI_BF16, nullptr, 0, 0, 0, st));
		ELF_TRY(buf_alloc(s, bs, B_O));
		ELF_TRY(buf_alloc(s, bs, B_LSE));
		{
			const bf16_t* q = (const bf16_t*)bs.b[B_QKV].p;
			ELF_TRY(attn_fwd(q, q + s->Hq * s->D, q + (s->Hq + s->Hkv) * s->D, bs.b[B_O].p, bs.b[B_LSE].p, s->nqkv, s->nqkv, s->nqkv,
			                 s->Hq * s->D, s->B, s->S, s->Hq, s->Hkv, s->D, s->cfg.causal, scale, st));
		}
		ELF_TRY(buf_alloc(s, bs, B_X2));
		ELF_TRY(gemm_bf16(0, 0, T, d, s->Hq * s->D, bs.b[B_O].p, s->Hq * s->D, p.w[P_WO], s->Hq * s->D, bs.b[B_X2].p, d, EPI_BF16_RESID, xin, d, 0, 0, st));
		ELF_TRY(buf_alloc(s, bs, B_ST2));
		ELF_TRY(buf_alloc(s, bs, B_H2));
		ELF_TRY(norm_fwd(norm_kind, bs.b[B_X2].p, p.w[P_NORM2_G], p.w[P_NORM2_B], bs.b[B_H2].p, bs.b[B_ST2].p, T, d, s->cfg.eps, st));
		ELF_TRY(buf_alloc(s, bs, B_GU));
		ELF_TRY(buf_alloc(s, bs, B_A));
		ELF_TRY(gemm_act_bf16(s->llama ? ACT_SWIGLU : ACT_GELU, T, F, d, bs.b[B_H2].p, d, p.w[P_W1], d, bs.b[B_GU].p, s->ffn_in, bs.b[B_A].p, F, st));
		void* yout;
		if (i == nb - 1 && s->vocab_out) {
			const int id = s->final_norm ? B_X : B_H1;
			ELF_TRY(buf_alloc(s, m.head, id));
			yout = m.head.b[id].p;
		} else if (i == nb - 1) {
			yout = y;
		} else {
			BlockState& nx = m.blk[i + 1];
			ELF_TRY(buf_alloc(s, nx, B_X));
			yout = nx.b[B_X].p;
		}
		// (a recompute passes no y: the stage's output went downstream the first time and no backward reads it)
		if (yout) ELF_TRY(gemm_bf16(0, 0, T, d, F, bs.b[B_A].p, F, p.w[P_W2], F, yout, d, EPI_BF16_RESID, bs.b[B_X2].p, d, 0, 0, st));
		// drop what this mode does not keep (the block input is needed until here)
		if (mode != SAVE_ALL) {
			const unsigned keep = mode == SAVE_WIN ? WIN_MASK : 0u;
			for (int id = 0; id < B_COUNT; id++)
				if ((ACT_MASK & (1u << id)) && !(keep & (1u << id))) buf_free(s, bs, id);
		}
		if (remat_drop) drop(bs, remat_drop);
		// the block's stash starts its way to the host while the next block computes
		if (offload && mode == SAVE_ALL) ELF_TRY(do_offload_block(s, bs, st));
		else if (s->lean && mode == SAVE_ALL) drop(bs, s->lean >= 2 ? OFFLOAD_REFORM_MASK : REFORM_MASK);
	}
	if (s->vocab_out) {
		// last stage: (final norm,) logits = h W_head^T   (benchmarks/models/simple.py:497, 508)
		BlockState& hd = m.head;
		if (s->final_norm) {
			ELF_TRY(buf_alloc(s, hd, B_ST1));
			ELF_TRY(buf_alloc(s, hd, B_H1));
			ELF_TRY(norm_fwd(norm_kind, hd.b[B_X].p, s->xw[XP_FNORM_G], s->xw[XP_FNORM_B], hd.b[B_H1].p, hd.b[B_ST1].p, T, d, s->cfg.eps, st));
		}
		if (y) ELF_TRY(gemm_bf16(0, 0, T, s->vld, d, hd.b[B_H1].p, d, s->xw[XP_HEAD], d, y, s->vld, EPI_BF16, nullptr, 0, 0, 0, st));
		if (remat_drop) drop(hd, remat_drop & (1u << B_ST1));
		if (mode != SAVE_ALL) {
			const unsigned keep = mode == SAVE_WIN ? WIN_MASK : 0u;
			for (int id = 0; id < B_COUNT; id++)
				if ((ACT_MASK & (1u << id)) && !(keep & (1u << id))) buf_free(s, hd, id);
		}
	}
	m.has_acts = mode == SAVE_ALL;
	m.has_win = mode != SAVE_NONE;
	if (offload && mode == SAVE_ALL) {
		m.offloaded = true;
		m.prefetched = false;
	}
	return 0;
}

// grads_only: recompute of the W stash gradients (RECOMPUTE_BACKWARD_INPUTS): no norm weight
// gradients, and the chain stops once the first block's QKV output gradient is known
// (elf/zb_utils.py:584-604, elf/execution/block.py:340-374).
static int run_backward(Stage* s, MbState& m, const void* dy, void* dx, bool grads_only, hipStream_t st, bool reform = true) {
	const int nb = s->cfg.n_blocks;
	const int T = s->T, d = s->d, F = s->F;
	const int norm_kind = s->llama ? NORM_RMS : NORM_LAYER;
	const float scale = 1.0f / sqrtf((float)s->D);
	if (s->vocab_out) {
		// last stage: dy is the gradient of the logits; it is the dY of the head linear's W stash
		BlockState& hd = m.head;
		hd.b[B_DQKV].p = const_cast<void*>(dy);
		hd.b[B_DQKV].owned = false;
		hd.b[B_DQKV].bytes = (size_t)T * s->vld * 2;
		BlockState& last = m.blk[nb - 1];
		ELF_TRY(buf_alloc(s, last, B_DY));
		if (s->final_norm) {
			if (hd.b[B_ST1].dropped) {  // the final norm was checkpointed: run it again for its statistics
				ELF_TRY(buf_alloc(s, hd, B_ST1));
				ELF_TRY(norm_fwd(norm_kind, hd.b[B_X].p, s->xw[XP_FNORM_G], s->xw[XP_FNORM_B], hd.b[B_H1].p, hd.b[B_ST1].p, T, d, s->cfg.eps, st));
			}
			PoolTmp d_hn(s->pool, (size_t)T * d * 2);
			if (!d_hn.p) return -3;
			ELF_TRY(gemm_bf16(0, 1, T, d, s->vld, dy, s->vld, s->xw[XP_HEAD], d, d_hn.p, d, EPI_BF16, nullptr, 0, 0, 0, st));
			ELF_TRY(norm_bwd(norm_kind, d_hn.p, hd.b[B_X].p, s->xw[XP_FNORM_G], hd.b[B_ST1].p, nullptr, last.b[B_DY].p,
			                 grads_only ? s->dummy_grad : s->xg[XP_FNORM_G], grads_only ? s->dummy_grad + d : s->xg[XP_FNORM_B], s->norm_ws, T, d, st));
		} else {
			ELF_TRY(gemm_bf16(0, 1, T, d, s->vld, dy, s->vld, s->xw[XP_HEAD], d, last.b[B_DY].p, d, EPI_BF16, nullptr, 0, 0, 0, st));
		}
		for (int id = 0; id < B_COUNT; id++)
			if ((ACT_MASK & (1u << id)) && !(WIN_MASK & (1u << id))) buf_free(s, hd, id);
	}
	for (int i = nb - 1; i >= 0; i--) {
		BlockState& bs = m.blk[i];
		const BlockParams& p = s->params[i];
		if (i == nb - 1 && !s->vocab_out) {
			bs.b[B_DY].p = const_cast<void*>(dy);
			bs.b[B_DY].owned = false;
			bs.b[B_DY].bytes = s->buf_bytes(B_DY);
		}
		const void* dyin = bs.b[B_DY].p;
		// a prefetched micro-batch: B waits for each group of buffers where it first reads one, and forms what the
		// offload dropped again from them (norm_fwd rewrites the statistics with the same values)
		const bool pre = m.offloaded && m.prefetched && bs.pre_ev;
		// FFN: dY W2 and the activation's backward, in one kernel for SwiGLU where the shape allows (a prefetched
		// micro-batch keeps them apart: the GEMM then runs while the gate/up product is still on the link)
		ELF_TRY(buf_alloc(s, bs, B_DGU));
		PoolTmp d_h(s->pool, (size_t)T * d * 2);
		if (!d_h.p) return -3;
		if (s->llama && !pre && gemm_swiglu_bwd_fused(T, F, d)) {
			// a dropped FFN activation (lean stash) is formed again by the same kernel, from the gate/up values its epilogue reads
			const bool form_a = reform && bs.b[B_A].dropped;
			if (form_a) ELF_TRY(buf_alloc(s, bs, B_A));
			ELF_TRY(gemm_swiglu_bwd_bf16(T, F, d, dyin, d, p.w[P_W2], F, bs.b[B_GU].p, s->ffn_in, bs.b[B_DGU].p, s->ffn_in, nullptr, st,
			                             form_a ? bs.b[B_A].p : nullptr, F));
			ELF_TRY(gemm_bf16(0, 1, T, d, s->ffn_in, bs.b[B_DGU].p, s->ffn_in, p.w[P_W1], d, d_h.p, d, EPI_BF16, nullptr, 0, 0, 0, st));
		} else {
			PoolTmp d_a(s->pool, (size_t)T * F * 2);
			if (!d_a.p) return -3;
			ELF_TRY(gemm_bf16(0, 1, T, F, d, dyin, d, p.w[P_W2], F, d_a.p, F, EPI_BF16, nullptr, 0, 0, 0, st));
			const bool form_a = reform && bs.b[B_A].dropped;
			if (form_a) ELF_TRY(buf_alloc(s, bs, B_A));
			// a prefetched micro-batch: row chunk by row chunk as the pre-activation arrives (elementwise kernels and a
			// GEMM whose rows are independent: the same bits as in one piece)
			const int nch = pre ? bs.gu_chunks : 1;
			const int Tc = T / nch;
			for (int c = 0; c < nch; c++) {
				if (pre) ELF_CHECK_HIP(hipStreamWaitEvent(st, bs.pre_gu[c], 0));
				const bf16_t* gu_c = (const bf16_t*)bs.b[B_GU].p + (size_t)c * Tc * s->ffn_in;
				bf16_t* dgu_c = (bf16_t*)bs.b[B_DGU].p + (size_t)c * Tc * s->ffn_in;
				const bf16_t* da_c = (const bf16_t*)d_a.p + (size_t)c * Tc * F;
				bf16_t* a_c = form_a ? (bf16_t*)bs.b[B_A].p + (size_t)c * Tc * F : nullptr;
				if (s->llama) {
					ELF_TRY(swiglu_bwd(da_c, gu_c, dgu_c, Tc, F, st, a_c));  // the activation, when dropped, from the same pass over g and u
				} else {
					ELF_TRY(gelu_bwd(da_c, gu_c, dgu_c, (int64_t)Tc * F, st));
					if (form_a) ELF_TRY(gelu_fwd(gu_c, a_c, (int64_t)Tc * F, st));
				}
				ELF_TRY(gemm_bf16(0, 1, Tc, d, s->ffn_in, dgu_c, s->ffn_in, p.w[P_W1], d, (bf16_t*)d_h.p + (size_t)c * Tc * d, d, EPI_BF16, nullptr, 0, 0, 0, st));
			}
		}
		ELF_TRY(buf_alloc(s, bs, B_DX2));
		if (pre) ELF_CHECK_HIP(hipStreamWaitEvent(st, bs.pre_ev, 0));  // the rest of the block's stash
		// what the attention backward reads and the offload / lean stash / module checkpoints dropped, formed again with the
		// forward's own calls: the first norm's output and statistics, the QKV projection, the attention output and log-sum-exp
		// the first norm's output, when only W reads it (projection kept, statistics kept), comes out of that norm's backward
		// at the end of the block (the recompute of a first block's W stash stops before that norm: forward again there)
		const bool h1_from_bwd = reform && bs.b[B_H1].dropped && !bs.b[B_QKV].dropped && !bs.b[B_ST1].dropped && norm_bwd_forms_output(d) && !(grads_only && i == 0);
		auto reform_attention_inputs = [&]() -> int {
			if (!h1_from_bwd && ((bs.b[B_H1].dropped && (reform || bs.b[B_QKV].dropped)) || bs.b[B_ST1].dropped)) {
				ELF_TRY(buf_alloc(s, bs, B_H1));
				ELF_TRY(buf_alloc(s, bs, B_ST1));
				ELF_TRY(norm_fwd(norm_kind, bs.b[B_X].p, p.w[P_NORM1_G], p.w[P_NORM1_B], bs.b[B_H1].p, bs.b[B_ST1].p, T, d, s->cfg.eps, st));
			}
			if (bs.b[B_QKV].dropped) {
				ELF_TRY(buf_alloc(s, bs, B_QKV));
				if (s->llama) ELF_TRY(gemm_rope_bf16(T, s->nqkv, d, bs.b[B_H1].p, d, p.w[P_WQKV], d, bs.b[B_QKV].p, s->nqkv, s->rope_cs, s->S, s->Hq + s->Hkv, s->D, st));
				else ELF_TRY(gemm_bf16(0, 0, T, s->nqkv, d, bs.b[B_H1].p, d, p.w[P_WQKV], d, bs.b[B_QKV].p, s->nqkv, EPI_BF16, nullptr, 0, 0, 0, st));
			}
			if (bs.b[B_LSE].dropped) {  // checkpointed attention core: its output and log-sum-exp are formed again
				ELF_TRY(buf_alloc(s, bs, B_O));
				ELF_TRY(buf_alloc(s, bs, B_LSE));
				const bf16_t* q = (const bf16_t*)bs.b[B_QKV].p;
				ELF_TRY(attn_fwd(q, q + s->Hq * s->D, q + (s->Hq + s->Hkv) * s->D, bs.b[B_O].p, bs.b[B_LSE].p, s->nqkv, s->nqkv, s->nqkv,
				                 s->Hq * s->D, s->B, s->S, s->Hq, s->Hkv, s->D, s->cfg.causal, scale, st));
			}
			return 0;
		};
		bool attention_inputs_ready = false;
		if (bs.b[B_X2].dropped && bs.b[B_LSE].dropped) {  // x2 needs the attention output, which a checkpointed attention core dropped as well
			ELF_TRY(reform_attention_inputs());
			attention_inputs_ready = true;
		}
		if (bs.b[B_X2].dropped) {  // not moved over the host link: x2 = x + o Wo^T, the forward's own call
			ELF_TRY(buf_alloc(s, bs, B_X2));
			ELF_TRY(gemm_bf16(0, 0, T, d, s->Hq * s->D, bs.b[B_O].p, s->Hq * s->D, p.w[P_WO], s->Hq * s->D, bs.b[B_X2].p, d, EPI_BF16_RESID, bs.b[B_X].p, d, 0, 0, st));
		}
		// A norm output that the lean stash / offload dropped is only read by W (the FFN's first linear layer): the norm's
		// backward writes it again from the row it holds anyway.  A checkpointed norm has no statistics either: forward again.
		void* h2_out = nullptr;
		if (reform && bs.b[B_H2].dropped && !bs.b[B_ST2].dropped && norm_bwd_forms_output(d)) {
			ELF_TRY(buf_alloc(s, bs, B_H2));
			h2_out = bs.b[B_H2].p;
		} else if ((reform && bs.b[B_H2].dropped) || bs.b[B_ST2].dropped) {
			ELF_TRY(buf_alloc(s, bs, B_H2));
			ELF_TRY(buf_alloc(s, bs, B_ST2));
			ELF_TRY(norm_fwd(norm_kind, bs.b[B_X2].p, p.w[P_NORM2_G], p.w[P_NORM2_B], bs.b[B_H2].p, bs.b[B_ST2].p, T, d, s->cfg.eps, st));
		}
		ELF_TRY(norm_bwd(norm_kind, d_h.p, bs.b[B_X2].p, p.w[P_NORM2_G], bs.b[B_ST2].p, dyin, bs.b[B_DX2].p,
		                 grads_only ? s->dummy_grad : p.g[P_NORM2_G], grads_only ? s->dummy_grad + d : p.g[P_NORM2_B], s->norm_ws, T, d, st,
		                 p.w[P_NORM2_B], h2_out));
		// attention
		PoolTmp d_o(s->pool, (size_t)T * s->Hq * s->D * 2);
		if (!d_o.p) return -3;
		ELF_TRY(gemm_bf16(0, 1, T, s->Hq * s->D, d, bs.b[B_DX2].p, d, p.w[P_WO], s->Hq * s->D, d_o.p, s->Hq * s->D, EPI_BF16, nullptr, 0, 0, 0, st));
		ELF_TRY(buf_alloc(s, bs, B_DQKV));
		if (!attention_inputs_ready) ELF_TRY(reform_attention_inputs());
		{
			const bf16_t* q = (const bf16_t*)bs.b[B_QKV].p;
			bf16_t* dq = (bf16_t*)bs.b[B_DQKV].p;
			const int ko = s->Hq * s->D, vo = (s->Hq + s->Hkv) * s->D;
			// the llama block's q and k carry the rotary embedding: its backward is applied to dQ and dK where they are stored
			ELF_TRY(attn_bwd(q, q + ko, q + vo, bs.b[B_O].p, d_o.p, bs.b[B_LSE].p, dq, dq + ko, dq + vo, s->attn_ws, s->nqkv, s->nqkv, s->nqkv,
			                 s->Hq * s->D, s->Hq * s->D, s->nqkv, s->nqkv, s->nqkv, s->B, s->S, s->Hq, s->Hkv, s->D, s->cfg.causal, scale, st,
			                 s->llama ? s->rope_cs : nullptr));
		}
		d_o.release();
		if (!(grads_only && i == 0)) {
			ELF_TRY(gemm_bf16(0, 1, T, d, s->nqkv, bs.b[B_DQKV].p, s->nqkv, p.w[P_WQKV], d, d_h.p, d, EPI_BF16, nullptr, 0, 0, 0, st));
			void* dxout;
			PoolTmp d_emb(s->pool, i == 0 && s->vocab_in ? (size_t)T * d * 2 : 0);
			if (i == 0 && s->vocab_in) {
				if (!d_emb.p) return -3;
				dxout = d_emb.p;
			} else if (i == 0) {
				dxout = dx;
			} else {
				BlockState& pv = m.blk[i - 1];
				ELF_TRY(buf_alloc(s, pv, B_DY));
				dxout = pv.b[B_DY].p;
			}
			if (h1_from_bwd) ELF_TRY(buf_alloc(s, bs, B_H1));
			ELF_TRY(norm_bwd(norm_kind, d_h.p, bs.b[B_X].p, p.w[P_NORM1_G], bs.b[B_ST1].p, bs.b[B_DX2].p, dxout,
			                 grads_only ? s->dummy_grad : p.g[P_NORM1_G], grads_only ? s->dummy_grad + d : p.g[P_NORM1_B], s->norm_ws, T, d, st,
			                 p.w[P_NORM1_B], h1_from_bwd ? bs.b[B_H1].p : nullptr));
			if (i == 0 && s->vocab_in) {
				// first stage: the embedding is not a split layer, its gradient accumulates inside B
				if (!grads_only) ELF_TRY(embedding_bwd(m.ids, d_emb.p, s->xg[XP_EMBED], T, d, s->vocab_in, st));
			}
		}
		// B consumed the activation stash; what is left is the W stash
		for (int id = 0; id < B_COUNT; id++)
			if ((ACT_MASK & (1u << id)) && !(WIN_MASK & (1u << id))) buf_free(s, bs, id);
	}
	m.has_acts = false;
	m.has_win = true;
	m.has_wgrad = true;
	return 0;
}

// scale != 0: the step's last W pass; every linear layer's accumulator leaves it multiplied by `scale`, with its bf16
// copy written (PipelineBlock.scale_grads, elf/execution/block.py:518-527, folded into the pass that holds the tiles).
static int run_backward_params(Stage* s, MbState& m, hipStream_t st, float scale = 0.f) {
	const int T = s->T, d = s->d, F = s->F;
	// dW[N_out, K_in] += dY[T, N_out]^T X[T, K_in] for every linear layer of the stage: the layers whose shapes fit go
	// into launches of up to 16 (their workgroups fill the chip together), in the stage's layer order; the others
	// (a head whose vocabulary is not a multiple of 256) run one by one.  Which way a layer goes depends on its shape
	// alone, so every stream that reaches this W pass accumulates its gradients in the same order of roundings.
	DwProblem group[16];
	int ng = 0;
	static const bool no_group = getenv("ELF_NO_DW_GROUP") != nullptr;  // one launch per layer instead (for comparisons)
	auto flush = [&]() -> int {
		const int n = ng;
		ng = 0;
		return n ? gemm_dw_group(n, group, T, scale, st) : 0;
	};
	auto dw = [&](int M, int N, const void* dy, int64_t lddy, const void* x, int64_t ldx, float* acc, void* g16) -> int {
		if (!no_group && gemm_dw_groupable(M, N, T, dy, lddy, x, ldx, acc) && (scale == 0.f || g16)) {
			group[ng++] = DwProblem{dy, lddy, x, ldx, acc, g16, M, N};
			return ng == 16 ? flush() : 0;
		}
		if (scale != 0.f) return gemm_dw_final(M, N, T, dy, lddy, x, ldx, acc, g16, scale, st);
		return gemm_bf16(1, 1, M, N, T, dy, lddy, x, ldx, acc, N, EPI_F32_ACC, nullptr, 0, 0, 0, st);
	};
	for (int i = 0; i < s->cfg.n_blocks; i++) {
		BlockState& bs = m.blk[i];
		const BlockParams& p = s->params[i];
		const int hd = s->Hq * s->D;
		ELF_TRY(dw(d, F, bs.b[B_DY].p, d, bs.b[B_A].p, F, p.g[P_W2], p.g16[P_W2]));
		ELF_TRY(dw(s->ffn_in, d, bs.b[B_DGU].p, s->ffn_in, bs.b[B_H2].p, d, p.g[P_W1], p.g16[P_W1]));
		ELF_TRY(dw(d, hd, bs.b[B_DX2].p, d, bs.b[B_O].p, hd, p.g[P_WO], p.g16[P_WO]));
		ELF_TRY(dw(s->nqkv, d, bs.b[B_DQKV].p, s->nqkv, bs.b[B_H1].p, d, p.g[P_WQKV], p.g16[P_WQKV]));
	}
	if (s->vocab_out) ELF_TRY(dw(s->vld, d, m.head.b[B_DQKV].p, s->vld, m.head.b[B_H1].p, d, s->xg[XP_HEAD], s->xg16[XP_HEAD]));
	ELF_TRY(flush());
	free_mask(s, m, WIN_MASK | WGRAD_MASK);
	m.has_win = m.has_wgrad = false;
	return 0;
}

// ---------------------------------------------------------------------------------------------
// Offload (elf/execution/offload.py:228-268, 330-390): every stage-owned activation buffer of
// more than 1 MiB goes to the pinned arena on the offload stream; the device copy returns to the
// pool once that copy has finished.  The OFFLOAD_REFORM_MASK buffers are not copied: they go back to the pool at
// once and run_backward forms them again.
static int do_offload_block(Stage* s, BlockState& bs, hipStream_t st) {
	hipEvent_t ready;
	ELF_CHECK_HIP(hipEventCreateWithFlags(&ready, hipEventDisableTiming));
	ELF_CHECK_HIP(hipEventRecord(ready, st));
	ELF_CHECK_HIP(hipStreamWaitEvent(s->offload_stream, ready, 0));
	ELF_CHECK_HIP(hipEventDestroy(ready));
	if (!bs.off_ev) ELF_CHECK_HIP(hipEventCreateWithFlags(&bs.off_ev, hipEventDisableTiming));
	std::vector<void*> to_free;
	for (int id = 0; id < B_COUNT; id++) {
		Buf& b = bs.b[id];
		if (!(ACT_MASK & (1u << id)) || !b.p || !b.owned || b.bytes <= (size_t(1) << 20)) continue;
		if (OFFLOAD_REFORM_MASK & (1u << id)) {
			s->pool.free(b.p);  // F's kernels are queued: the pool hands it out again in stream order
			b.p = nullptr;
			b.owned = false;
			b.dropped = true;
			continue;
		}
		// blocks of released micro-batches first; the arena only grows when waiting for them does not make room
		if (!s->host_pending.empty()) {
			poll_host_pending(s, false);
			if (!s->pinned->fits((int64_t)(b.bytes / 2), 1)) poll_host_pending(s, true);
		}
		if (!s->pinned->allocate((int64_t)(b.bytes / 2), 2, /*bf16*/ 1, &b.host)) return -3;
		ELF_CHECK_HIP(hipMemcpyAsync(b.host.ptr, b.p, b.bytes, hipMemcpyDeviceToHost, s->offload_stream));
		s->d2h_bytes += (int64_t)b.bytes;
		to_free.push_back(b.p);
		b.p = nullptr;
		b.owned = false;
		b.offloaded = true;
	}
	ELF_CHECK_HIP(hipEventRecord(bs.off_ev, s->offload_stream));
	for (void* p : to_free) s->pool.free_after(p, bs.off_ev);
	return 0;
}

static int do_offload(Stage* s, MbState& m, hipStream_t st) {
	if (!m.has_acts || m.offloaded) return 0;
	for (auto& bs : m.blk) ELF_TRY(do_offload_block(s, bs, st));
	m.offloaded = true;
	m.prefetched = false;
	return 0;
}

// Bring offloaded buffers back: on the prefetch stream (async = true, PREFETCH_ACTIVATIONS) or on
// the compute stream when B finds them still on the host (the reference restores synchronously
// in that case, offload.py:281-283).  Blocks come back in the order B walks them (last first),
// each with its own event, so B starts on the last block while the first is still on the link.
static int do_restore(Stage* s, MbState& m, bool async, hipStream_t st) {
	if (!m.offloaded || m.prefetched) return 0;
	hipStream_t cs = async ? s->prefetch_stream : st;
	// device buffers are taken from the pool in compute-stream order
	for (auto& bs : m.blk)
		for (int id = 0; id < B_COUNT; id++) {
			Buf& b = bs.b[id];
			if (!b.offloaded) continue;
			b.p = s->pool.alloc(b.bytes);
			if (!b.p) return -3;
			b.owned = true;
		}
	if (async) {
		hipEvent_t now;
		ELF_CHECK_HIP(hipEventCreateWithFlags(&now, hipEventDisableTiming));
		ELF_CHECK_HIP(hipEventRecord(now, st));
		ELF_CHECK_HIP(hipStreamWaitEvent(cs, now, 0));
		ELF_CHECK_HIP(hipEventDestroy(now));
	}
	// Row chunks of the FFN pre-activation (by far the largest buffer: 940 of 1210 MB per block at the 70B shape): as
	// many as keep each chunk's GEMM in B on the tiles the whole GEMM uses (at least 192 tiles of 256 x 256), so that
	// chunked and whole give the same bits.
	int nch = 1;
	for (int n : {4, 2})
		if (nch == 1 && n <= BlockState::MAX_GU_CHUNKS && s->T % (n * 256) == 0 && s->d % 256 == 0 && (int64_t)(s->T / n / 256) * (s->d / 256) >= 192) nch = n;
	for (int i = (int)m.blk.size() - 1; i >= 0; i--) {
		BlockState& bs = m.blk[i];
		if (bs.off_ev) ELF_CHECK_HIP(hipStreamWaitEvent(cs, bs.off_ev, 0));
		// in the order B reads them: the gate/up product (activation backward, after one GEMM), then the block input and
		// the attention's buffers (x2, the norm outputs and the QKV projection are formed again from these)
		static const int order[] = {B_GU, B_X, B_ST1, B_ST2, B_O, B_LSE, B_X2, B_QKV};
		static_assert(sizeof(order) / sizeof(order[0]) == 8, "every ACT_MASK buffer outside REFORM_MASK is listed");
		bs.gu_chunks = async ? nch : 1;
		for (int id : order) {
			Buf& b = bs.b[id];
			if (id == B_GU && b.offloaded && async) {
				const size_t piece = b.bytes / nch;  // whole rows: bytes = T * ffn_in * 2 and T % nch == 0
				for (int c = 0; c < nch; c++) {
					ELF_CHECK_HIP(hipMemcpyAsync((char*)b.p + c * piece, (const char*)b.host.ptr + c * piece, piece, hipMemcpyHostToDevice, cs));
					if (!bs.pre_gu[c]) ELF_CHECK_HIP(hipEventCreateWithFlags(&bs.pre_gu[c], hipEventDisableTiming));
					ELF_CHECK_HIP(hipEventRecord(bs.pre_gu[c], cs));
				}
				s->h2d_bytes += (int64_t)b.bytes;
				continue;
			}
			if (b.offloaded) {
				ELF_CHECK_HIP(hipMemcpyAsync(b.p, b.host.ptr, b.bytes, hipMemcpyHostToDevice, cs));
				s->h2d_bytes += (int64_t)b.bytes;
			}
			if (id == B_GU && async) {  // nothing to copy (the buffer was small enough to stay): its events fire at once
				for (int c = 0; c < nch; c++) {
					if (!bs.pre_gu[c]) ELF_CHECK_HIP(hipEventCreateWithFlags(&bs.pre_gu[c], hipEventDisableTiming));
					ELF_CHECK_HIP(hipEventRecord(bs.pre_gu[c], cs));
				}
			}
		}
		if (async) {
			if (!bs.pre_ev) ELF_CHECK_HIP(hipEventCreateWithFlags(&bs.pre_ev, hipEventDisableTiming));
			ELF_CHECK_HIP(hipEventRecord(bs.pre_ev, cs));
		} else if (bs.pre_ev) {
			(void)hipEventDestroy(bs.pre_ev);
			bs.pre_ev = nullptr;
		}
	}
	m.prefetched = true;
	return 0;
}

// RELEASE of an offloaded micro-batch (offload.py:392-411): its pinned blocks go back to the arena once the copies
// that use them are done.  The host does not wait: an event recorded now on the stream those copies were issued on
// guards the blocks (poll_host_pending).
static int do_release(Stage* s, MbState& m) {
	if (!m.offloaded) return 0;
	Stage::HostPending hp;
	hp.ev = nullptr;
	for (auto& bs : m.blk)
		for (int id = 0; id < B_COUNT; id++) {
			Buf& b = bs.b[id];
			if (b.offloaded) {
				hp.ptrs.push_back(b.host.ptr);
				b.offloaded = false;
			}
		}
	if (!hp.ptrs.empty()) {
		// asynchronous prefetch: the host-to-device copies ran on the prefetch stream; otherwise the last user of the
		// blocks is the offload stream's device-to-host copy (a restore on the compute stream is ordered before any
		// later offload by that offload's own wait on the compute stream)
		bool async_restore = false;
		for (auto& bs : m.blk) async_restore = async_restore || (m.prefetched && bs.pre_ev);
		ELF_CHECK_HIP(hipEventCreateWithFlags(&hp.ev, hipEventDisableTiming));
		ELF_CHECK_HIP(hipEventRecord(hp.ev, async_restore ? s->prefetch_stream : s->offload_stream));
		s->host_pending.push_back(std::move(hp));
	}
	m.offloaded = false;
	m.prefetched = false;
	poll_host_pending(s, false);
	return 0;
}

}  // namespace elf

using namespace elf;

extern "C" {

int elf_stage_create(const elf_stage_cfg* cfg, elf_stage_t** out) {
	ELF_REQUIRE(cfg && out, "elf_stage_create: null argument");
	ELF_REQUIRE(cfg->arch == ELF_ARCH_GPT || cfg->arch == ELF_ARCH_LLAMA, "elf_stage_create: unknown arch %d", cfg->arch);
	ELF_REQUIRE(cfg->n_blocks > 0 && cfg->d_model > 0 && cfg->n_heads > 0 && cfg->n_kv_heads > 0 && cfg->ffn > 0 && cfg->seq > 0 && cfg->mb > 0,
	            "elf_stage_create: sizes must be positive");
	ELF_REQUIRE(cfg->n_heads % cfg->n_kv_heads == 0, "elf_stage_create: n_heads must be a multiple of n_kv_heads");
	ELF_REQUIRE(cfg->head_dim == 64 || cfg->head_dim == 128, "elf_stage_create: head_dim must be 64 or 128");
	ELF_REQUIRE(cfg->seq % 128 == 0, "elf_stage_create: seq must be a multiple of 128");
	ELF_REQUIRE(cfg->d_model % 64 == 0 && cfg->ffn % 64 == 0 && cfg->d_model <= 8192, "elf_stage_create: d_model and ffn must be multiples of 64, d_model <= 8192");
	ELF_REQUIRE(cfg->arch == ELF_ARCH_LLAMA || cfg->n_heads == cfg->n_kv_heads, "elf_stage_create: the GPT block has no grouped-query attention");
	Stage* s = new Stage();
	s->cfg = *cfg;
	s->llama = cfg->arch == ELF_ARCH_LLAMA;
	s->d = cfg->d_model;
	s->Hq = cfg->n_heads;
	s->Hkv = cfg->n_kv_heads;
	s->D = cfg->head_dim;
	s->F = cfg->ffn;
	s->S = cfg->seq;
	s->B = cfg->mb;
	s->T = cfg->mb * cfg->seq;
	s->nqkv = (s->Hq + 2 * s->Hkv) * s->D;
	s->ffn_in = s->llama ? 2 * s->F : s->F;
	s->params.resize(cfg->n_blocks);
	s->pinned.reset(new PinnedPool(false));
	auto fail = [&](const char* what) {
		set_error("elf_stage_create: %s failed", what);
		elf_stage_destroy((elf_stage_t*)s);
		return -2;
	};
	if (hipStreamCreateWithFlags(&s->offload_stream, hipStreamNonBlocking) != hipSuccess) return fail("offload stream");
	if (hipStreamCreateWithFlags(&s->prefetch_stream, hipStreamNonBlocking) != hipSuccess) return fail("prefetch stream");
	const size_t norm_ws_bytes = (size_t)norm_bwd_workspace_floats(s->T, s->d) * 4;
	const size_t attn_ws_bytes = (size_t)attn_bwd_workspace_bytes(s->B, s->S, s->Hq, s->D, s->cfg.causal);
	const size_t rope_bytes = s->llama ? (size_t)s->S * (s->D / 2) * 8 : 0;
	s->ws_bytes = (int64_t)(norm_ws_bytes + attn_ws_bytes + rope_bytes + (size_t)2 * s->d * 4);
	if (hipMalloc((void**)&s->norm_ws, norm_ws_bytes) != hipSuccess) return fail("norm workspace");
	if (hipMalloc(&s->attn_ws, attn_ws_bytes) != hipSuccess) return fail("attention workspace");
	if (hipMalloc((void**)&s->dummy_grad, (size_t)2 * s->d * 4) != hipSuccess) return fail("gradient sink");
	if (hipMemset(s->dummy_grad, 0, (size_t)2 * s->d * 4) != hipSuccess) return fail("gradient sink clear");
	if (s->llama) {
		if (hipMalloc(&s->rope_cs, rope_bytes) != hipSuccess) return fail("rope table");
		if (rope_table(s->rope_cs, s->S, s->D, cfg->rope_theta, nullptr) != 0) return fail("rope table fill");
		if (hipStreamSynchronize(nullptr) != hipSuccess) return fail("rope table sync");
	}
	*out = (elf_stage_t*)s;
	return 0;
}

void elf_stage_destroy(elf_stage_t* h) {
	if (!h) return;
	Stage* s = (Stage*)h;
	(void)hipDeviceSynchronize();
	s->pool.drain();  // blocks waiting on per-block copy events go back before those events are destroyed
	for (auto& kv : s->mbs) {
		do_release(s, kv.second);
		free_mask(s, kv.second, ~0u);
		destroy_events(kv.second);
	}
	s->mbs.clear();
	poll_host_pending(s, true);
	if (s->offload_stream) (void)hipStreamDestroy(s->offload_stream);
	if (s->prefetch_stream) (void)hipStreamDestroy(s->prefetch_stream);
	if (s->norm_ws) (void)hipFree(s->norm_ws);
	if (s->attn_ws) (void)hipFree(s->attn_ws);
	if (s->dummy_grad) (void)hipFree(s->dummy_grad);
	if (s->rope_cs) (void)hipFree(s->rope_cs);
	delete s;
}

int elf_stage_bind_param(elf_stage_t* h, int block, int which, void* weight_bf16, void* grad_f32) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s, "elf_stage_bind_param: null stage");
	ELF_REQUIRE(weight_bf16 && grad_f32, "elf_stage_bind_param: null pointer");
	ELF_REQUIRE(((uintptr_t)weight_bf16 % 16) == 0 && ((uintptr_t)grad_f32 % 16) == 0, "elf_stage_bind_param: pointers must be 16-byte aligned");
	if (block == -1) {
		ELF_REQUIRE(which >= ELF_P_EMBED && which <= ELF_P_HEAD, "elf_stage_bind_param: stage-level parameter id %d out of range", which);
		s->xw[which - ELF_P_EMBED] = weight_bf16;
		s->xg[which - ELF_P_EMBED] = (float*)grad_f32;
		return 0;
	}
	ELF_REQUIRE(block >= 0 && block < s->cfg.n_blocks, "elf_stage_bind_param: block %d out of range", block);
	ELF_REQUIRE(which >= 0 && which < P_COUNT, "elf_stage_bind_param: parameter id %d out of range", which);
	s->params[block].w[which] = weight_bf16;
	s->params[block].g[which] = (float*)grad_f32;
	return 0;
}

static int check_bound(Stage* s) {
	for (int i = 0; i < s->cfg.n_blocks; i++)
		for (int w = 0; w < P_COUNT; w++) {
			if (s->llama && (w == P_NORM1_B || w == P_NORM2_B)) continue;
			ELF_REQUIRE(s->params[i].w[w] != nullptr, "stage: parameter %d of block %d is not bound", w, i);
		}
	ELF_REQUIRE(!s->vocab_in || s->xw[XP_EMBED], "stage: the embedding table is not bound");
	ELF_REQUIRE(!s->vocab_out || s->xw[XP_HEAD], "stage: the output head is not bound");
	ELF_REQUIRE(!s->final_norm || (s->xw[XP_FNORM_G] && (s->llama || s->xw[XP_FNORM_B])), "stage: the final norm is not bound");
	return 0;
}

int elf_stage_set_ends(elf_stage_t* h, int vocab_in, int vocab_out, int vocab_out_ld, int final_norm) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s, "elf_stage_set_ends: null stage");
	ELF_REQUIRE(s->mbs.empty(), "elf_stage_set_ends: call it before the first forward");
	ELF_REQUIRE(vocab_in >= 0 && vocab_out >= 0, "elf_stage_set_ends: negative vocabulary size");
	ELF_REQUIRE(!vocab_out || (vocab_out_ld >= vocab_out && vocab_out_ld % 64 == 0),
	            "elf_stage_set_ends: the logits row stride must be a multiple of 64 and at least vocab_out (%d, %d)", vocab_out_ld, vocab_out);
	ELF_REQUIRE(!final_norm || vocab_out, "elf_stage_set_ends: a final norm needs an output head");
	s->vocab_in = vocab_in;
	s->vocab_out = vocab_out;
	s->vld = vocab_out ? vocab_out_ld : 0;
	s->final_norm = final_norm != 0;
	return 0;
}

int elf_stage_set_lean_stash(elf_stage_t* h, int level) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s, "elf_stage_set_lean_stash: null stage");
	ELF_REQUIRE(level >= 0 && level <= 2, "elf_stage_set_lean_stash: level must be 0, 1 or 2 (got %d)", level);
	s->lean = level;
	return 0;
}

int elf_stage_set_mb_samples(elf_stage_t* h, int mb, int samples) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s && mb >= 0, "elf_stage_set_mb_samples: bad argument");
	ELF_REQUIRE(samples >= 1 && samples <= s->cfg.mb, "elf_stage_set_mb_samples: micro-batch %d has %d sequences, the stage was created for 1..%d", mb, samples, s->cfg.mb);
	auto it = s->mbs.find(mb);
	if (it != s->mbs.end()) {
		const MbState& m = it->second;
		ELF_REQUIRE(!m.has_acts && !m.has_win && !m.has_wgrad && !m.remat_root, "elf_stage_set_mb_samples: micro-batch %d is in flight", mb);
	}
	if (samples == s->cfg.mb) s->mb_samples.erase(mb);
	else s->mb_samples[mb] = samples;
	return 0;
}

int elf_stage_forward(elf_stage_t* h, int mb, const void* x, void* y, uint32_t flags, void* stream) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s && x && y && mb >= 0, "elf_stage_forward: bad argument");
	ELF_TRY(check_bound(s));
	MbState& m = mb_state(s, mb);
	ELF_REQUIRE(!m.has_acts && !m.has_win && !m.has_wgrad && !m.remat_root, "elf_stage_forward: micro-batch %d is already in flight", mb);
	use_mb(s, mb);
	ELF_REQUIRE(!(flags & ~(ELF_FWD_REMAT_ROOT | ELF_FWD_REMAT_ATTN | ELF_FWD_OFFLOAD | ELF_FWD_REMAT_NORM)), "elf_stage_forward: unknown flag bits 0x%x", flags);
	const bool root = flags & ELF_FWD_REMAT_ROOT;
	ELF_TRY(run_forward(s, m, x, y, root ? SAVE_NONE : SAVE_ALL, (hipStream_t)stream, (flags & ELF_FWD_OFFLOAD) && !root, root ? 0u : flags));
	m.remat_root = root;
	if (root) m.has_win = false;
	return 0;
}

int elf_stage_backward_inputs(elf_stage_t* h, int mb, const void* x, const void* dy, void* dx, uint32_t flags, void* stream) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s && dy && (dx || s->vocab_in) && mb >= 0, "elf_stage_backward_inputs: bad argument");
	auto it = s->mbs.find(mb);
	ELF_REQUIRE(it != s->mbs.end(), "elf_stage_backward_inputs: no forward was run for micro-batch %d", mb);
	MbState& m = it->second;
	hipStream_t st = (hipStream_t)stream;
	use_mb(s, mb);
	if (m.remat_root) {
		// the forward kept only the stage input: re-run it, this time keeping the stash
		ELF_REQUIRE(x != nullptr, "elf_stage_backward_inputs: micro-batch %d was checkpointed, the stage input is needed", mb);
		ELF_TRY(run_forward(s, m, x, nullptr, SAVE_ALL, st));
		m.remat_root = false;
	}
	ELF_REQUIRE(m.has_acts, "elf_stage_backward_inputs: micro-batch %d has no saved activations", mb);
	if (m.offloaded) {
		if (!m.prefetched) ELF_TRY(do_restore(s, m, false, st));  // run_backward waits block by block otherwise
	}
	if (x && s->vocab_in) m.ids = x;
	else if (x) m.blk[0].b[B_X].p = const_cast<void*>(x);
	// the W-stash inputs are dropped below: no point in forming the ones F or the offload left out
	if (int rc = run_backward(s, m, dy, dx, false, st, !(flags & ELF_BWD_RECOMPUTE_ACTIVATIONS))) {
		free_mask(s, m, WGRAD_MASK);  // half-written output gradients are of no use to W
		m.has_wgrad = false;
		return rc;
	}
	if (flags & ELF_BWD_RECOMPUTE_GRADIENTS) free_mask(s, m, WGRAD_MASK), m.has_wgrad = false;
	if (flags & ELF_BWD_RECOMPUTE_ACTIVATIONS) free_mask(s, m, WIN_MASK), m.has_win = false;
	return 0;
}

int elf_stage_bind_grad_bf16(elf_stage_t* h, int block, int which, void* grad_bf16) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s && grad_bf16 && ((uintptr_t)grad_bf16 % 16) == 0, "elf_stage_bind_grad_bf16: null stage or null / misaligned pointer");
	if (block == -1) {
		ELF_REQUIRE(which == ELF_P_HEAD, "elf_stage_bind_grad_bf16: of the stage-level parameters only the output head (%d) is a linear layer", ELF_P_HEAD);
		s->xg16[XP_HEAD] = grad_bf16;
		return 0;
	}
	ELF_REQUIRE(block >= 0 && block < s->cfg.n_blocks, "elf_stage_bind_grad_bf16: block %d out of range", block);
	ELF_REQUIRE(which == P_WQKV || which == P_WO || which == P_W1 || which == P_W2, "elf_stage_bind_grad_bf16: parameter %d is not a linear layer's weight", which);
	s->params[block].g16[which] = grad_bf16;
	return 0;
}

static int backward_params_entry(elf_stage_t* h, int mb, float scale, void* stream, const char* who);

int elf_stage_backward_params_scaled(elf_stage_t* h, int mb, float scale, void* stream) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s && scale != 0.f && scale == scale, "elf_stage_backward_params_scaled: null stage or a scale that is zero or not a number");
	for (int i = 0; i < s->cfg.n_blocks; i++)
		for (int w : {P_WQKV, P_WO, P_W1, P_W2}) ELF_REQUIRE(s->params[i].g16[w] != nullptr, "elf_stage_backward_params_scaled: bf16 gradient buffer %d of block %d not bound", w, i);
	ELF_REQUIRE(!s->vocab_out || s->xg16[XP_HEAD], "elf_stage_backward_params_scaled: bf16 gradient buffer of the output head not bound");
	return backward_params_entry(h, mb, scale, stream, "elf_stage_backward_params_scaled");
}

int elf_stage_backward_params(elf_stage_t* h, int mb, void* stream) { return backward_params_entry(h, mb, 0.f, stream, "elf_stage_backward_params"); }

static int backward_params_entry(elf_stage_t* h, int mb, float scale, void* stream, const char* who) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s && mb >= 0, "%s: bad argument", who);
	auto it = s->mbs.find(mb);
	ELF_REQUIRE(it != s->mbs.end() && it->second.has_win && it->second.has_wgrad,
	            "elf_stage_backward_params: micro-batch %d has no saved inputs / output gradients (run B, or the recompute ops, first)", mb);
	for (int i = 0; i < s->cfg.n_blocks; i++)
		for (int w : {P_WQKV, P_WO, P_W1, P_W2}) ELF_REQUIRE(s->params[i].g[w] != nullptr, "elf_stage_backward_params: gradient buffer not bound");
	ELF_REQUIRE(!s->vocab_out || s->xg[XP_HEAD], "elf_stage_backward_params: gradient buffer of the output head not bound");
	use_mb(s, mb);
	ELF_TRY(run_backward_params(s, it->second, (hipStream_t)stream, scale));
	return 0;
}

int elf_stage_recompute_forward(elf_stage_t* h, int mb, const void* x, int save, void* stream) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s && x && mb >= 0, "elf_stage_recompute_forward: bad argument");
	auto it = s->mbs.find(mb);
	ELF_REQUIRE(it != s->mbs.end(), "elf_stage_recompute_forward: unknown micro-batch %d", mb);
	MbState& m = it->second;
	ELF_REQUIRE(!m.has_acts && !m.has_win, "elf_stage_recompute_forward: micro-batch %d still holds its activations", mb);
	hipStream_t st = (hipStream_t)stream;
	use_mb(s, mb);
	return run_forward(s, m, x, nullptr, save ? SAVE_ALL : SAVE_WIN, st);
}

int elf_stage_recompute_backward_inputs(elf_stage_t* h, int mb, const void* dy, void* stream) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s && dy && mb >= 0, "elf_stage_recompute_backward_inputs: bad argument");
	auto it = s->mbs.find(mb);
	ELF_REQUIRE(it != s->mbs.end() && it->second.has_acts,
	            "elf_stage_recompute_backward_inputs: micro-batch %d has no saved graph (run recompute_forward with save first)", mb);
	use_mb(s, mb);
	return run_backward(s, it->second, dy, nullptr, true, (hipStream_t)stream);
}

int elf_stage_offload(elf_stage_t* h, int mb, void* stream) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s, "elf_stage_offload: null stage");
	auto it = s->mbs.find(mb);
	ELF_REQUIRE(it != s->mbs.end(), "elf_stage_offload: unknown micro-batch %d", mb);
	return do_offload(s, it->second, (hipStream_t)stream);
}

int elf_stage_prefetch(elf_stage_t* h, int mb, void* stream) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s, "elf_stage_prefetch: null stage");
	auto it = s->mbs.find(mb);
	if (it == s->mbs.end()) return 0;  // nothing offloaded (the offloader of the reference is empty then)
	return do_restore(s, it->second, true, (hipStream_t)stream);
}

int elf_stage_release(elf_stage_t* h, int mb) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s, "elf_stage_release: null stage");
	auto it = s->mbs.find(mb);
	if (it == s->mbs.end()) return 0;
	return do_release(s, it->second);
}

int elf_stage_reserve_pinned(elf_stage_t* h, int64_t bytes) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s && bytes > 0, "elf_stage_reserve_pinned: bad argument");
	return s->pinned->reserve(bytes, 2, /*bf16*/ 1) ? 0 : -3;
}

int elf_stage_clear(elf_stage_t* h) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s, "elf_stage_clear: null stage");
	ELF_CHECK_HIP(hipDeviceSynchronize());
	s->pool.drain();  // blocks waiting on per-block copy events go back before those events are destroyed
	for (auto& kv : s->mbs) {
		ELF_TRY(do_release(s, kv.second));
		free_mask(s, kv.second, ~0u);
		destroy_events(kv.second);
	}
	s->mbs.clear();
	s->mb_samples.clear();
	poll_host_pending(s, true);
	return 0;
}

int elf_stage_mem_stats(elf_stage_t* h, elf_mem_stats* out) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s && out, "elf_stage_mem_stats: null argument");
	s->pool.poll();  // buffers whose copy to the host has finished no longer count as live
	poll_host_pending(s, false);
	out->live_bytes = (int64_t)s->pool.live_bytes();
	out->peak_bytes = (int64_t)s->pool.peak_bytes();
	out->reserved_bytes = (int64_t)s->pool.reserved_bytes();
	out->pinned_bytes = s->pinned->size_bytes();
	out->d2h_bytes = s->d2h_bytes;
	out->h2d_bytes = s->h2d_bytes;
	out->workspace_bytes = s->ws_bytes;
	return 0;
}

int elf_stage_reset_peak(elf_stage_t* h) {
	Stage* s = (Stage*)h;
	ELF_REQUIRE(s, "elf_stage_reset_peak: null stage");
	s->pool.reset_peak();
	return 0;
}

// Pinned arena exposed on its own so that its placement policy can be checked against the
// reference's rules without a GPU (host_backing = 1 uses malloc).
int elf_pinned_pool_create(int host_backing, elf_pinned_pool_t** out) {
	ELF_REQUIRE(out, "elf_pinned_pool_create: null argument");
	*out = (elf_pinned_pool_t*)new PinnedPool(host_backing != 0);
	return 0;
}
void elf_pinned_pool_destroy(elf_pinned_pool_t* p) { delete (PinnedPool*)p; }
int elf_pinned_pool_allocate(elf_pinned_pool_t* p, int64_t elems, int elem_size, int dtype_key, void** ptr, int* parent, int64_t* offset) {
	ELF_REQUIRE(p && ptr, "elf_pinned_pool_allocate: null argument");
	ELF_REQUIRE(elem_size > 0, "elf_pinned_pool_allocate: element size must be positive");
	PinnedPool::Block b;
	if (!((PinnedPool*)p)->allocate(elems, elem_size, dtype_key, &b)) return -3;
	*ptr = b.ptr;
	if (parent) *parent = b.parent;
	if (offset) *offset = b.offset;
	return 0;
}
int elf_pinned_pool_free(elf_pinned_pool_t* p, void* ptr) {
	ELF_REQUIRE(p, "elf_pinned_pool_free: null pool");
	return ((PinnedPool*)p)->free(ptr) ? 0 : 1;  // 1: not a block of this pool (ignored, as in the reference)
}
int elf_pinned_pool_reserve(elf_pinned_pool_t* p, int64_t bytes, int elem_size, int dtype_key) {
	ELF_REQUIRE(p && elem_size > 0 && bytes > 0, "elf_pinned_pool_reserve: bad argument");
	return ((PinnedPool*)p)->reserve(bytes, elem_size, dtype_key) ? 0 : -3;
}
int64_t elf_pinned_pool_size(elf_pinned_pool_t* p) { return p ? ((PinnedPool*)p)->size_bytes() : 0; }
int elf_pinned_pool_n_parents(elf_pinned_pool_t* p) { return p ? ((PinnedPool*)p)->n_parents() : 0; }
int elf_pinned_pool_n_free(elf_pinned_pool_t* p, int parent) {
	PinnedPool* pp = (PinnedPool*)p;
	if (!pp || parent < 0 || parent >= pp->n_parents()) return -1;
	return pp->n_free_segments(parent);
}
int elf_pinned_pool_free_segment(elf_pinned_pool_t* p, int parent, int i, int64_t* offset, int64_t* length) {
	PinnedPool* pp = (PinnedPool*)p;
	ELF_REQUIRE(pp && parent >= 0 && parent < pp->n_parents() && i >= 0 && i < pp->n_free_segments(parent) && offset && length,
	            "elf_pinned_pool_free_segment: index out of range");
	auto seg = pp->free_segment(parent, i);
	*offset = seg.first;
	*length = seg.second;
	return 0;
}

}  // extern "C"
