"""F / B / W of a whole stage through the C ABI (HipStageBlock) against the oracle stage
(oracle/stage_ref.py, fp32 from the same bf16-rounded weights and boundary tensors).
Tolerance: rel 2e-2 of the tensor's max magnitude (the path's stated bf16 bar), plus a 1e-2
relative Frobenius bound; weight gradients are accumulated in fp32 over several micro-batches."""

import pytest
import torch

from tests.helpers import assert_close, cfg_from_stage, oracle_params_from_stage, perturb_norms, product_grads

pytestmark = pytest.mark.gpu

N_MB = 3


def _stage(kind):
	from elf_amd import models

	if kind == "gpt":
		st = models.gpt_stage(2, 256, 4, 512, 128, causal=False, seed=3)
	elif kind == "gpt_causal":
		st = models.gpt_stage(1, 128, 2, 256, 256, causal=True, seed=4)
	else:
		st = models.llama_stage(2, 512, 4, 2, 768, 256, head_dim=128, seed=5)
	perturb_norms(st)
	return st


def _block(stage, mb, **kw):
	from elf_amd.execution import HipStageBlock
	from elf_amd.partitioners.utils import sequential_signatures

	placement = [0, 1, 2, 3]
	return HipStageBlock(stage, 1, placement, sequential_signatures(placement)[1], mb_size=mb, **kw)


def _oracle(stage, mb, **kw):
	from oracle import stage_ref as R

	cfg = cfg_from_stage(stage, mb)
	return R, cfg, R.RefStage(cfg, oracle_params_from_stage(stage), device="cuda", **kw)


@pytest.mark.parametrize("kind", ["gpt", "gpt_causal", "llama"])
def test_fbw_matches_oracle(kind):
	mb = 2
	stage = _stage(kind)
	R, cfg, ref = _oracle(stage, mb)
	blk = _block(stage, mb)
	xs, dys = R.make_boundary(cfg, N_MB, seed=11)
	blk.set_boundary(inputs=[x.cuda() for x in xs], grads=[d.cuda() for d in dys], keep_sent=True)
	# all forwards first, then B, then W (queues hold several micro-batches at once)
	for m in range(N_MB):
		blk.recv_forward(m, mb, src=0)
		blk.forward(m)
		blk.send_forward(m, dst=2)
		assert_close(blk.sent_forward[m], ref.forward(m, xs[m]), f"{kind} y[{m}]")
	for m in range(N_MB):
		blk.recv_backward(m, mb, src=2)
		blk.backward_inputs(m)
		blk.send_backward(m, dst=0)
		assert_close(blk.sent_backward[m], ref.backward_inputs(m, dys[m]), f"{kind} dx[{m}]")
	for m in range(N_MB):
		blk.backward_params(m)
		ref.backward_params(m)
	got, want = product_grads(stage), ref.grads()
	assert set(got) == set(want)
	for name in sorted(want):
		assert_close(got[name], want[name], f"{kind} grad {name}")
	# scale_grads: main_grad /= batch and bf16 .grad appears (block.py:518-527)
	blk.scale_grads(mb * N_MB)
	ref.scale_grads(mb * N_MB)
	got_bf16, got32, want = product_grads(stage, "grad"), product_grads(stage), ref.grads()
	for name in sorted(want):
		assert got_bf16[name].dtype == torch.bfloat16
		assert_close(got32[name], want[name], f"{kind} scaled grad {name}")
		assert torch.equal(got_bf16[name], got32[name].to(torch.bfloat16))
	st = blk.mem_stats()
	assert st["live_bytes"] == 0, "every stash must be gone after W"
	assert st["peak_bytes"] > 0
	# fixed scratch allocated at creation: at least the attention backward's workspace
	from elf_amd import _lib

	c = blk.cfg
	attn_ws = _lib.load().elf_attn_bwd_workspace_bytes(c.mb, c.seq, c.n_heads, c.head_dim, int(c.causal))
	assert attn_ws <= st["workspace_bytes"] <= attn_ws + (64 << 20)


@pytest.mark.parametrize("kind", ["gpt", "llama"])
def test_short_micro_batches_share_a_stage(kind):
	"""Micro-batches of 3, 1 and 2 sequences on a stage sized for 3 (an uneven split of the batch,
	elf/pipeline.py:497-503): each against the oracle, with a recompute of the 1-sequence one, an offload
	round trip of the 2-sequence one, and the slot
	of the short micro-batch reused by a full one in the next step."""
	mb, sizes = 3, [3, 1, 2]
	stage = _stage(kind)
	R, cfg, ref = _oracle(stage, mb)
	blk = _block(stage, mb)
	xs, dys = R.make_boundary(cfg, len(sizes), seed=13)
	xs = [x[:n].contiguous() for x, n in zip(xs, sizes)]
	dys = [d[:n].contiguous() for d, n in zip(dys, sizes)]
	blk.set_boundary(inputs=[x.cuda() for x in xs], grads=[d.cuda() for d in dys], keep_sent=True)
	for m, n in enumerate(sizes):
		blk.recv_forward(m, n, src=0)
		blk.forward(m, **({"remat_strategy": (lambda name, module: name == "")} if m == 1 else {}))
		blk.send_forward(m, dst=2)
		assert_close(blk.sent_forward[m], ref.forward(m, xs[m]), f"{kind} y[{m}] ({n} sequences)")
	blk.offload(2)  # the 2-sequence micro-batch goes to the pinned arena and comes back before its B
	for m, n in enumerate(sizes):
		blk.recv_backward(m, n, src=2)
		if m == 2:
			blk.prefetch(2)
		blk.backward_inputs(m)
		if m == 2:
			blk.release(2)
		blk.send_backward(m, dst=0)
		assert_close(blk.sent_backward[m], ref.backward_inputs(m, dys[m]), f"{kind} dx[{m}] ({n} sequences)")
		blk.backward_params(m)
		ref.backward_params(m)
	got, want = product_grads(stage), ref.grads()
	for name in sorted(want):
		assert_close(got[name], want[name], f"{kind} grad {name}")
	assert blk.mem_stats()["live_bytes"] == 0
	# next step: slot 1 now carries a full micro-batch
	full = R.make_boundary(cfg, 1, seed=14)[0][0]
	blk.set_boundary(inputs={1: full.cuda()}.__getitem__, keep_sent=True)
	blk.recv_forward(1, mb, src=0)
	blk.forward(1)
	blk.send_forward(1, dst=2)
	assert_close(blk.sent_forward[1], R.RefStage(cfg, oracle_params_from_stage(stage), device="cuda").forward(1, full), f"{kind} full micro-batch in a slot that was short")
	blk.clear()


@pytest.mark.parametrize("kind", ["gpt", "llama"])
@pytest.mark.parametrize("lean", [0, 1, 2])
@pytest.mark.parametrize("variant", ["full_fwd", "activations_bwd", "full_bwd", "offload", "offload_no_prefetch", "lean_stash"])
def test_remat_and_offload_variants_equal_plain(kind, variant, lean):
	"""Every remat / offload variant must give the results of the plain F-B-W sequence bit for bit: the
	same kernels on the same data, and every accumulation in a fixed order (the attention backward sums its
	dQ partials in tile order, the K splits of a weight-gradient tile add in turn, the norm gradients are
	folded by one writer per column)."""
	from elf_amd.scheduling import OpOptions

	if not lean and variant == "lean_stash":
		pytest.skip("the lean stash alone needs a level")
	mb = 16 if variant.startswith("offload") else 2  # only buffers above 1 MiB are offloaded
	stage = _stage(kind)
	R, cfg, _ = _oracle(stage, mb)
	xs, dys = R.make_boundary(cfg, 2, seed=21)
	xs, dys = [x.cuda() for x in xs], [d.cuda() for d in dys]

	held_after_f = {}

	def run(variant):
		blk = _block(stage, mb, lean_stash=0 if variant == "plain" else lean)
		blk.zero_grad()
		blk.set_boundary(inputs=xs, grads=dys, keep_sent=True)
		root = lambda name, module: name == ""
		for m in range(2):
			blk.recv_forward(m, mb, src=0)
			if variant == "full_fwd":
				blk.forward(m, **{OpOptions.REMAT_STRATEGY: root})
				assert blk.mem_stats()["live_bytes"] == 0, "a checkpointed forward keeps nothing"
			elif variant.startswith("offload"):
				blk.forward(m)
				blk.offload(m)
			else:
				blk.forward(m)
			blk.send_forward(m, dst=2)
		held_after_f[variant] = blk.mem_stats()["live_bytes"]
		if variant.startswith("offload"):
			torch.cuda.synchronize()
			st = blk.mem_stats()
			assert st["d2h_bytes"] > 0 and st["pinned_bytes"] >= st["d2h_bytes"]
			# what crosses the link: the stage-owned buffers above 1 MiB minus the two norm outputs, the FFN activation,
			# the QKV projection's output and the attention residual, which B forms again from the restored buffers:
			# per block the attention output, its log-sum-exp and the FFN pre-activation, plus the inputs of the blocks
			# behind the first
			T, d, hq, hkv, hd = mb * cfg["seq"], cfg["d_model"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
			ffn_in = cfg["ffn"] * (2 if kind == "llama" else 1)
			per_block = [T * hq * hd * 2, mb * hq * cfg["seq"] * 4, T * ffn_in * 2]
			moved = sum(b for b in per_block if b > 1 << 20) * cfg["n_blocks"] + (T * d * 2 if T * d * 2 > 1 << 20 else 0) * (cfg["n_blocks"] - 1)
			assert st["d2h_bytes"] == 2 * moved
		for m in range(2):
			blk.recv_backward(m, mb, src=2)
			if variant == "activations_bwd":
				blk.backward_inputs(m, **{OpOptions.RECOMPUTE_ACTIVATIONS: True})
				blk.recompute_forward(m)
			elif variant == "full_bwd":
				blk.backward_inputs(m, **{OpOptions.RECOMPUTE_ACTIVATIONS: True, OpOptions.RECOMPUTE_GRADIENTS: True})
				if m == 1:  # no other micro-batch in flight any more
					assert blk.mem_stats()["live_bytes"] == 0, "full_bwd drops both halves of the W stash"
				blk.recompute_forward(m, **{OpOptions.SAVE: True})
				blk.recompute_backward_inputs(m)
			elif variant == "offload":
				blk.prefetch(m)
				blk.backward_inputs(m)
				blk.release(m)
			elif variant == "offload_no_prefetch":
				blk.backward_inputs(m)
				blk.release(m)
			else:
				blk.backward_inputs(m)
			blk.send_backward(m, dst=0)
			blk.backward_params(m)
		torch.cuda.synchronize()
		assert blk.mem_stats()["live_bytes"] == 0
		if variant.startswith("offload"):
			assert blk.mem_stats()["h2d_bytes"] == blk.mem_stats()["d2h_bytes"]
		grads = {k: v.clone() for k, v in product_grads(stage).items()}
		return dict(blk.sent_forward), dict(blk.sent_backward), grads

	y0, dx0, g0 = run("plain")
	y1, dx1, g1 = run(variant)
	if variant == "lean_stash":
		# two micro-batches after F: per block the two norm outputs and the FFN activation less; at level 2 the QKV
		# projection's output and the attention residual as well
		T = mb * cfg["seq"]

		def pooled(elements):  # what the device pool holds for a bf16 buffer: 512-byte granules, 2 MiB ones from 1 MiB on
			b = 2 * elements
			gran = 2 << 20 if b >= 1 << 20 else 512
			return (b + gran - 1) // gran * gran

		less = 2 * pooled(T * cfg["d_model"]) + pooled(T * cfg["ffn"])
		if lean == 2:
			less += pooled(T * (cfg["n_heads"] + 2 * cfg["n_kv_heads"]) * cfg["head_dim"]) + pooled(T * cfg["d_model"])
		assert held_after_f["plain"] - held_after_f["lean_stash"] == 2 * cfg["n_blocks"] * less
	for m in range(2):
		assert torch.equal(y0[m], y1[m]), "forward outputs must be bit-identical"
		assert torch.equal(dx1[m], dx0[m]), f"{variant} dx[{m}] must be bit-identical"
	for name in g0:
		assert torch.equal(g1[name], g0[name]), f"{variant} grad {name} must be bit-identical"


def _pool_round(nbytes):
	"""Size the stage's device pool charges for a buffer (2 MiB steps from 1 MiB up, 512 B below)."""
	gran = (2 << 20) if nbytes >= (1 << 20) else 512
	return -(-nbytes // gran) * gran


@pytest.mark.parametrize("kind", ["gpt", "llama"])
@pytest.mark.parametrize("strategy_kind", ["simple", "selective", "norms_and_cores"])
@pytest.mark.parametrize("offload", [False, True])
def test_module_remat_strategies_match_the_oracle(kind, strategy_kind, offload):
	"""remat_strategy functions that select sub-modules (benchmarks/benchmark_utils.py:311-321: "simple" =
	GELU / LayerNorm / Dropout modules, "selective" = attention cores; plus one that picks every norm of
	either kind and the cores): the forward drops what those modules would have kept (asserted on the
	library's live bytes), B forms it again, and y, dX and every gradient match the oracle run with
	checkpoint() around the same sub-modules, and the plain run of this library."""
	from elf_amd.benchmark_utils import _strategy
	from elf_amd.scheduling import OpOptions

	mb = 16 if offload else 2  # only buffers above 1 MiB are offloaded
	stage = _stage(kind)
	R, cfg, ref = _oracle(stage, mb)
	if strategy_kind == "norms_and_cores":
		strategy = lambda name, module: type(module).__name__ in ("LayerNorm", "RMSNorm", "Attention")
	else:
		strategy = _strategy(strategy_kind)
	# what the strategy selects in this stage, in the oracle's terms
	picked = {type(m).__name__ for n, m in stage.named_modules() if strategy(n, m)}
	kinds = tuple(k for k, names in (("norm", {"LayerNorm", "RMSNorm"}), ("attn", {"Attention"}), ("act", {"GELU"})) if picked & names)
	if strategy_kind == "simple":
		assert kinds == (("norm", "act") if kind == "gpt" else ()), "the llama block has no LayerNorm / GELU module: nothing is selected"
	xs, dys = R.make_boundary(cfg, 1, seed=23)
	x, dy = xs[0].cuda(), dys[0].cuda()

	def run(strategy):
		blk = _block(stage, mb)
		blk.zero_grad()
		blk.set_boundary(inputs=[x], grads=[dy], keep_sent=True)
		blk.recv_forward(0, mb, src=0)
		blk.forward(0, **({OpOptions.REMAT_STRATEGY: strategy} if strategy else {}))
		held = blk.mem_stats()["live_bytes"]
		if offload:
			blk.offload(0)
		blk.send_forward(0, dst=2)
		blk.recv_backward(0, mb, src=2)
		if offload:
			blk.prefetch(0)
		blk.backward_inputs(0)
		if offload:
			blk.release(0)
		blk.send_backward(0, dst=0)
		blk.backward_params(0)
		torch.cuda.synchronize()
		assert blk.mem_stats()["live_bytes"] == 0
		return blk.sent_forward[0], blk.sent_backward[0], {k: v.clone() for k, v in product_grads(stage).items()}, held

	y0, dx0, g0, held0 = run(None)
	y1, dx1, g1, held1 = run(strategy)
	T = mb * cfg["seq"]
	saved = 0
	if "norm" in kinds:
		saved += 2 * _pool_round(T * 2 * 4)
	if "attn" in kinds:
		saved += _pool_round(T * cfg["n_heads"] * cfg["head_dim"] * 2) + _pool_round(mb * cfg["n_heads"] * cfg["seq"] * 4)
	assert held0 - held1 == cfg["n_blocks"] * saved
	assert torch.equal(y1, y0) and torch.equal(dx1, dx0), "the re-formed buffers are bit-identical, so are y and dX"
	want_y = ref.forward(0, xs[0], remat=kinds)
	want_dx = ref.backward_inputs(0, dys[0])
	ref.backward_params(0)
	assert_close(y1, want_y, f"{kind} {strategy_kind} y")
	assert_close(dx1, want_dx, f"{kind} {strategy_kind} dx")
	want = ref.grads()
	for name in sorted(want):
		assert_close(g1[name], want[name], f"{kind} {strategy_kind} grad {name}")
		assert torch.equal(g1[name], g0[name]), f"{kind} {strategy_kind} grad {name} differs from the plain run"


def test_remat_strategies_this_executor_cannot_express_raise():
	from elf_amd._lib import ElfStageError
	from elf_amd.scheduling import OpOptions

	stage = _stage("gpt")
	blk = _block(stage, 2)
	x = torch.zeros(2, 128, 256, dtype=torch.bfloat16, device="cuda")
	for m, strategy in enumerate([
		lambda name, module: type(module).__name__ == "Linear",  # linears are not checkpointable units here
		lambda name, module: name == "0",  # one block of the stage
		lambda name, module: name == "0.norm1",  # one norm of many
	]):
		blk.set_boundary(inputs={m: x}.__getitem__)
		blk.recv_forward(m, 2, src=0)
		with pytest.raises(ElfStageError):
			blk.forward(m, **{OpOptions.REMAT_STRATEGY: strategy})
	# a strategy that selects nothing is a plain forward, as in the reference
	blk.set_boundary(inputs={5: x}.__getitem__)
	blk.recv_forward(5, 2, src=0)
	blk.forward(5, **{OpOptions.REMAT_STRATEGY: lambda name, module: False})
	blk.clear()


def test_engine_runs_1f1b_and_zbh1_streams():
	"""The Engine interprets the filtered op stream of a middle stage (block 1 of pp = 4) and gives
	the same gradients as the oracle stage driven by the same stream."""
	from elf_amd.execution import Engine
	from elf_amd.partitioners.utils import sequential_signatures
	from elf_amd.registry import COMM_SCHEDULERS, SCHEDULERS
	from elf_amd.scheduling import OperationType as T, add_comms

	mb, nmb, placement = 2, 4, [0, 1, 2, 3]
	for sched_name in ("1f1b", "zbh1"):
		stage = _stage("llama")
		R, cfg, ref = _oracle(stage, mb)
		xs, dys = R.make_boundary(cfg, nmb, seed=31)
		blk = _block(stage, mb)
		blk.zero_grad()
		blk.set_boundary(inputs=[x.cuda() for x in xs], grads=[d.cuda() for d in dys])
		schedule = COMM_SCHEDULERS["pipelined"](add_comms(SCHEDULERS[sched_name](placement, nmb), sequential_signatures(placement)))
		stream = [op for op in schedule if op.block_id == 1]
		eng = Engine([blk])
		result, losses, stats, detailed = eng.train_step(None, None, None, stream, [mb] * nmb)
		for op in stream:
			if op.op == T.FORWARD:
				ref.forward(op.mb_id, xs[op.mb_id])
			elif op.op == T.BACKWARD_INPUTS:
				ref.backward_inputs(op.mb_id, dys[op.mb_id])
			elif op.op == T.BACKWARD_PARAMS:
				ref.backward_params(op.mb_id)
			elif op.op == T.ALL_REDUCE_PARAM_GRADS:
				ref.scale_grads(mb * nmb)
		got, want = product_grads(stage), ref.grads()
		for name in sorted(want):
			assert_close(got[name], want[name], f"{sched_name} grad {name}")
		assert list(detailed["memories"]) == [str(op) for op in stream]
		assert set(stats) == {"total", "idle", "start_idle", "end_idle", "bubble"}


def test_gradient_scale_folded_into_the_last_w_equals_the_separate_pass():
	"""The Engine tells the step's last W the scale that ALL_REDUCE_PARAM_GRADS applies behind it; the accumulators and
	the bf16 gradients must be those of the plain order, W then scale_grads (elf/execution/block.py:518-527), bit for
	bit - here at a shape whose weight gradients take the unfused route inside the library; the benchmark shapes, which
	scale in the GEMM epilogue, are compared the same way in tests/test_full_streams_gpu.py."""
	from elf_amd.execution import Engine
	from elf_amd.partitioners.utils import sequential_signatures
	from elf_amd.registry import COMM_SCHEDULERS, SCHEDULERS
	from elf_amd.scheduling import add_comms

	mb, nmb, placement = 2, 4, [0, 1, 2, 3]
	out = {}
	for fold in (True, False):
		stage = _stage("llama")
		R, cfg, _ = _oracle(stage, mb)
		xs, dys = R.make_boundary(cfg, nmb, seed=33)
		blk = _block(stage, mb)
		if not fold:
			blk.folds_grad_scale = False
		blk.zero_grad()
		blk.set_boundary(inputs=[x.cuda() for x in xs], grads=[d.cuda() for d in dys])
		schedule = COMM_SCHEDULERS["pipelined"](add_comms(SCHEDULERS["zbh1"](placement, nmb), sequential_signatures(placement)))
		Engine([blk]).train_step(None, None, None, [op for op in schedule if op.block_id == 1], [mb] * nmb)
		torch.cuda.synchronize()
		out[fold] = ({k: v.clone() for k, v in product_grads(stage).items()}, {k: v.clone() for k, v in product_grads(stage, "grad").items()})
	for k in out[True][0]:
		assert torch.equal(out[True][0][k], out[False][0][k]), f"fp32 accumulator {k}"
		assert out[True][1][k].dtype == torch.bfloat16 and torch.equal(out[True][1][k], out[False][1][k]), f"bf16 gradient {k}"
	# a scale that is not the one the last W folded is refused
	blk = _block(_stage("llama"), mb)
	blk._folded_scale = 0.5  # as if the last W had folded 1 / 2
	from elf_amd._lib import ElfStageError

	with pytest.raises(ElfStageError):
		blk.scale_grads(8)


def test_profile_stage_feeds_the_remat_ilp_and_the_stream_fits_the_budget():
	"""profile_stage on the native executor (reference: elf/scheduling/ilp.py:50-126, 224-254): the
	record is self-consistent, the ILP solved from it picks remat under a budget between the
	full-remat and no-remat peaks, and block 1's rewritten stream runs within that budget with the
	gradients of the plain stream."""
	from elf_amd.execution import Engine
	from elf_amd.partitioners.utils import sequential_signatures
	from elf_amd.registry import COMM_SCHEDULERS, SCHEDULERS
	from elf_amd.scheduling import add_comms
	from elf_amd.scheduling.ilp import RematScheduler, evaluate_remat, build_ilp_params, profile_stage, solve_remat

	mb, nmb, placement = 2, 6, [0, 1, 2, 3]
	stage = _stage("llama")
	blk = _block(stage, mb)
	blk.zero_grad()
	stats, nxt = profile_stage(blk, n_iter=2)
	assert tuple(nxt.shape) == (blk.T, blk.d) and nxt.device.type == "cpu"
	assert all(stats["T"][k] > 0 for k in "fbw")
	assert stats["M"]["w"] == 0.0 and stats["Mpeak"]["f"] >= stats["M"]["f"] > stats["Mpeak_ckpt"] > 0
	assert stats["Mba"] > 0 and stats["Mbg"] > 0 and abs(stats["Mba"] + stats["Mbg"] - stats["M"]["b"]) < 1e-6
	assert all(float(g.abs().max()) == 0.0 for g in blk._fused_g), "profiling must leave the accumulators as it found them"
	assert blk.mem_stats()["live_bytes"] == 0

	base = SCHEDULERS["1f1b"]
	statistics = [stats] * len(placement)
	params = build_ilp_params(statistics, placement, base, nmb, 1e9)
	zeros = {k: [[0.0] * nmb for _ in placement] for k in ("full_fwd", "activations_bwd", "full_bwd")}
	ones = dict(zeros, full_fwd=[[1.0] * nmb for _ in placement])
	peak_plain, peak_remat = max(evaluate_remat(params, zeros)[1]), max(evaluate_remat(params, ones)[1])
	assert peak_remat < peak_plain
	budget = 0.5 * (peak_plain + peak_remat)
	solution = solve_remat(statistics, placement, base, nmb, budget, time_limit=20)
	assert max(solution["peak_mems"]) <= budget + 1e-6
	assert sum(map(sum, solution["full_fwd"])) + sum(map(sum, solution["activations_bwd"])) + sum(map(sum, solution["full_bwd"])) > 0

	def run(scheduler):
		b = _block(_stage("llama"), mb)
		b.zero_grad()
		xs, dys = b_xs
		b.set_boundary(inputs=xs, grads=dys)
		schedule = COMM_SCHEDULERS["pipelined"](add_comms(scheduler(placement, nmb), sequential_signatures(placement)))
		stream = [op for op in schedule if op.block_id == 1]
		b.reset_peak()
		Engine([b]).train_step(None, None, None, stream, [mb] * nmb)
		torch.cuda.synchronize()
		return product_grads(b.model), b.mem_stats()["peak_bytes"]

	from elf_amd.synthetic import make_boundary

	b_xs = make_boundary(mb, stage.seq_len, blk.d, nmb, seed=5, device="cuda")
	g_plain, peak_plain_run = run(base)
	g_remat, peak_remat_run = run(RematScheduler(base, solution))
	assert peak_remat_run < peak_plain_run
	# what the library held at its high-water mark + weights and accumulators stays under the budget
	assert peak_remat_run / 2**20 + 2 * stats["Mparams"] <= budget + 1.0
	for name in sorted(g_plain):
		assert_close(g_remat[name], g_plain[name], f"remat grad {name}", rel_max=2e-3, rel_fro=2e-3)


def test_error_paths():
	from elf_amd._lib import ElfStageError

	stage = _stage("gpt")
	blk = _block(stage, 2)
	with pytest.raises(ElfStageError):
		blk.backward_params(0)  # nothing stashed
	blk.set_boundary(inputs=[torch.zeros(2, 128, 256, dtype=torch.float32, device="cuda")])
	blk.recv_forward(0, 2, src=0)
	with pytest.raises(ElfStageError):
		blk.forward(0)  # wrong dtype
	with pytest.raises(Exception):
		blk.forward(1)  # empty slot
	blk.set_boundary(inputs=[None, None, torch.zeros(3, 128, 256, dtype=torch.bfloat16, device="cuda")])
	blk.recv_forward(2, 3, src=0)
	with pytest.raises(ElfStageError):
		blk.forward(2)  # more sequences than the stage was sized for


def test_preallocate_pool_reserves_the_pinned_arena_before_the_first_step(monkeypatch):
	"""ELF_PREALLOCATE_POOL (elf/execution/engine.py:71-93): the Engine grows the stage's pinned arena by the
	requested size when it is built, so an offloaded micro-batch that fits finds its host blocks there and
	the arena does not grow inside the step."""
	from elf_amd.execution import Engine

	monkeypatch.setenv("ELF_PREALLOCATE_POOL", "bf16:1")
	mb = 16
	stage = _stage("llama")
	blk = _block(stage, mb)
	assert blk.mem_stats()["pinned_bytes"] == 0
	Engine([blk])
	assert blk.mem_stats()["pinned_bytes"] == 1 << 30, "one chunk of exactly the requested size (reserve does not round to a power of two)"
	R, cfg, _ = _oracle(stage, mb)
	xs, dys = R.make_boundary(cfg, 1, seed=3)
	blk.set_boundary(inputs=[xs[0].cuda()], grads=[dys[0].cuda()])
	blk.recv_forward(0, mb, src=0)
	blk.forward(0)
	blk.offload(0)
	torch.cuda.synchronize()
	st = blk.mem_stats()
	assert 0 < st["d2h_bytes"] < (1 << 30) and st["pinned_bytes"] == 1 << 30
	blk.clear()
	monkeypatch.setenv("ELF_PREALLOCATE_POOL", "q4:1")
	with pytest.raises(KeyError):
		Engine([blk])


def test_lean_stash_levels_are_zero_one_or_two():
	from elf_amd._lib import ElfStageError

	blk = _block(_stage("llama"), 2)
	for level in (0, 1, 2, 1, 0):
		blk.set_lean_stash(level)
		assert blk.lean_stash == level
	for bad in (3, -1):
		with pytest.raises(ElfStageError, match="level must be 0, 1 or 2"):
			blk.set_lean_stash(bad)
	assert blk.lean_stash == 0
