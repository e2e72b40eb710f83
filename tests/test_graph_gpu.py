"""A stage step captured as a HIP graph (Engine.capture, Pipeline.capture_step) against the same step
run eagerly: every replay is checked, with eager kernels and device synchronisations between the
replays and with new input data written into the buffers the graph reads.  Outputs, input gradients
and weight gradients are bit-identical: every accumulation of the path has a fixed order."""

import pytest
import torch

from tests.helpers import assert_close, perturb_norms, product_grads

pytestmark = pytest.mark.gpu


def _middle_stage(seed=5):
	from elf_amd import models
	from elf_amd.execution import HipStageBlock
	from elf_amd.partitioners.utils import sequential_signatures

	st = models.llama_stage(2, 512, 4, 2, 768, 256, head_dim=128, seed=seed)
	perturb_norms(st)
	placement = [0, 1, 2, 3]
	return st, HipStageBlock(st, 1, placement, sequential_signatures(placement)[1], mb_size=2)


def _stream(nmb):
	from elf_amd.partitioners.utils import sequential_signatures
	from elf_amd.registry import COMM_SCHEDULERS, SCHEDULERS
	from elf_amd.scheduling import add_comms

	placement = [0, 1, 2, 3]
	schedule = COMM_SCHEDULERS["pipelined"](add_comms(SCHEDULERS["zbh1"](placement, nmb), sequential_signatures(placement)))
	return [op for op in schedule if op.block_id == 1]


def test_captured_stage_stream_replays_like_the_eager_one():
	from elf_amd import kernels as K
	from elf_amd.execution import Engine
	from elf_amd.synthetic import make_boundary

	nmb, mb = 4, 2
	stage, blk = _middle_stage()
	xs, dys = make_boundary(mb, stage.seq_len, blk.d, nmb, seed=3, device="cuda")
	blk.set_boundary(inputs=xs, grads=dys, keep_sent=True)
	stream = _stream(nmb)
	eng = Engine([blk])

	def eager():
		blk.zero_grad()
		blk.set_boundary(inputs=xs, grads=dys, keep_sent=True)
		eng.train_step(None, None, None, stream, [mb] * nmb)
		torch.cuda.synchronize()
		return {m: y.clone() for m, y in blk.sent_forward.items()}, {m: d.clone() for m, d in blk.sent_backward.items()}, {k: v.clone() for k, v in product_grads(stage).items()}

	y0, dx0, g0 = eager()
	blk.set_boundary(inputs=xs, grads=dys, keep_sent=True)
	blk.zero_grad()
	marker = [g.clone().fill_(0.5) for g in blk._fused_g]
	for g, m in zip(blk._fused_g, marker):
		g.copy_(m)
	graphed = eng.capture(None, None, None, stream, [mb] * nmb)
	assert all(torch.equal(g, m) for g, m in zip(blk._fused_g, marker)), "capturing must not change the gradient accumulators"
	sent_y, sent_dx = dict(blk.sent_forward), dict(blk.sent_backward)  # tensors the graph writes
	a = torch.randn(512, 512, device="cuda").to(torch.bfloat16)
	for rep in range(3):
		blk.zero_grad()
		graphed.replay()
		torch.cuda.synchronize()
		for m in range(nmb):
			assert torch.equal(sent_y[m], y0[m]), f"replay {rep}: y[{m}]"
			assert torch.equal(sent_dx[m], dx0[m]), f"replay {rep}: dx[{m}]"
		got = product_grads(stage)
		for name in sorted(g0):
			assert torch.equal(got[name], g0[name]), f"replay {rep}: grad {name}"
		# eager work of the same library and a synchronisation between replays
		K.gemm(a, a)
		K.norm_fwd(K.NORM_RMS, a, torch.ones(512, dtype=torch.bfloat16, device="cuda"), None, 1e-5)
		torch.cuda.synchronize()
	assert blk.mem_stats()["live_bytes"] == 0

	# new data in the buffers the graph reads: the replay follows it
	xs2, dys2 = make_boundary(mb, stage.seq_len, blk.d, nmb, seed=4, device="cuda")
	for dst, src in zip(list(xs) + list(dys), list(xs2) + list(dys2)):
		dst.copy_(src)
	blk.zero_grad()
	graphed.replay()
	torch.cuda.synchronize()
	y_rep = {m: t.clone() for m, t in sent_y.items()}
	g_rep = {k: v.clone() for k, v in product_grads(stage).items()}
	y1, _, g1 = eager()
	for m in range(nmb):
		assert torch.equal(y_rep[m], y1[m]) and not torch.equal(y1[m], y0[m])
	for name in sorted(g1):
		assert torch.equal(g_rep[name], g1[name]), f"new data: grad {name}"


@pytest.mark.parametrize("loss_kind", ["fused", "torch"])
def test_captured_pipeline_step(loss_kind):
	"""Two stages (embedding ... head) on one rank, cross-entropy from elf_amd.losses or torch's under
	autograd: capture_step's replays on new token ids give the loss and gradients of step() on the
	same ids."""
	import torch.nn.functional as F

	from elf_amd import losses, models
	from elf_amd.pipeline import Pipeline

	V, d, S, mb, nmb = 1000, 256, 128, 4, 4

	def torch_loss(pred, target, *args, **kwargs):
		return F.cross_entropy(pred.to(torch.float32).view(-1, V), target.view(-1), *args, **kwargs)

	loss_fn = losses.cross_entropy if loss_kind == "fused" else torch_loss
	first = models.gpt_end_stage(2, d, 4, 1024, S, vocab_in=V, causal=True, seed=41)
	last = models.gpt_end_stage(2, d, 4, 1024, S, vocab_out=V, causal=True, seed=42)
	pipe = Pipeline([first, last], torch.zeros(mb, S, dtype=torch.int64), scheduler="afab", partitioner=False, placement=[0, 0])
	g = torch.Generator().manual_seed(2)
	draw = lambda: (torch.randint(0, V, (mb * nmb, S), generator=g).cuda(), torch.randint(0, V, (mb * nmb, S), generator=g).cuda())
	ids, tgt = draw()
	pipe.zero_grad()
	replay = pipe.capture_step(ids, tgt, loss_fn, split_size=mb)
	for rep in range(3):
		ids, tgt = draw()
		pipe.zero_grad()
		out, loss = replay(ids, tgt)
		torch.cuda.synchronize()
		got_loss = float(loss)
		got_out = [o.clone() for o in out]
		got = [p.main_grad.clone() for p in pipe.parameters()]  # (names repeat across stages)
		pipe.zero_grad()
		want_out, want_loss = pipe(ids, tgt, loss_fn, split_size=mb)
		assert got_loss == pytest.approx(float(want_loss), rel=1e-4), f"replay {rep}"
		for a, b in zip(got_out, want_out):
			assert torch.equal(a.cpu(), b.cpu())
		for have, (n, p) in zip(got, pipe.named_parameters()):
			assert torch.equal(have, p.main_grad), f"replay {rep}: grad {n}"


def test_capture_refuses_offload_schedules():
	from elf_amd.benchmark_utils import get_offloaded_scheduler
	from elf_amd.execution import Engine
	from elf_amd.partitioners.utils import sequential_signatures
	from elf_amd.registry import COMM_SCHEDULERS, SCHEDULERS
	from elf_amd.scheduling import add_comms

	stage, blk = _middle_stage()
	placement = [0, 1, 2, 3]
	sched = get_offloaded_scheduler(SCHEDULERS["1f1b"], 1, 1)
	schedule = COMM_SCHEDULERS["pipelined"](add_comms(sched(placement, 4), sequential_signatures(placement)))
	with pytest.raises(NotImplementedError):
		Engine([blk]).capture(None, None, None, [op for op in schedule if op.block_id == 1], [2] * 4)


def test_capture_with_live_kernel_timing_switched_on():
	"""Kernel timing events travel in the dispatches; a stream under capture must get plain launches all the
	same, and the captured kernels must replay correctly."""
	from elf_amd import _lib
	from elf_amd import kernels as K

	lib = _lib.load()
	g = torch.Generator(device="cuda").manual_seed(11)
	a = torch.randn(512, 256, device="cuda", generator=g).bfloat16()
	w = (torch.randn(768, 256, device="cuda", generator=g) * 0.05).bfloat16()
	out = torch.empty(512, 768, device="cuda", dtype=torch.bfloat16)
	ref = K.gemm(a, w).clone()
	lib.elf_prof_enable(1)
	try:
		K.gemm(a, w, out=out)  # timed, eager
		torch.cuda.synchronize()
		graph = torch.cuda.CUDAGraph()
		side = torch.cuda.Stream()
		side.wait_stream(torch.cuda.current_stream())
		with torch.cuda.stream(side):
			with torch.cuda.graph(graph, stream=side):
				K.gemm(a, w, out=out)
		torch.cuda.current_stream().wait_stream(side)
		for _ in range(3):
			out.zero_()
			graph.replay()
			torch.cuda.synchronize()
			assert torch.equal(out, ref)
	finally:
		lib.elf_prof_enable(0)


def test_kernel_timing_on_a_sample_of_the_launches():
	"""``elf_prof_enable(n)`` lets one launch in n carry events (the same pseudo-random picks every run);
	``elf_prof_launches`` still counts every launch and its work, and the sample gives the rate of all of them."""
	import ctypes

	from elf_amd import _lib
	from elf_amd import kernels as K

	lib = _lib.load()
	g = torch.Generator(device="cuda").manual_seed(12)
	a = torch.randn(1024, 512, device="cuda", generator=g).bfloat16()
	w = (torch.randn(1024, 512, device="cuda", generator=g) * 0.05).bfloat16()
	out = torch.empty(1024, 1024, device="cuda", dtype=torch.bfloat16)
	flops = 2.0 * 1024 * 1024 * 512

	def run(one_in, n=400):
		lib.elf_prof_enable(one_in)
		try:
			for _ in range(n):
				K.gemm(a, w, out=out)
			torch.cuda.synchronize()
			ms, work, all_work = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
			timed = lib.elf_prof_collect(0, ctypes.byref(ms), ctypes.byref(work))
			launches = lib.elf_prof_launches(0, ctypes.byref(all_work))
			return timed, launches, ms.value, work.value, all_work.value
		finally:
			lib.elf_prof_enable(0)

	for _ in range(50):
		K.gemm(a, w, out=out)  # warm
	t1, l1, ms1, w1, aw1 = run(1)
	assert t1 == l1 == 400 and w1 == aw1 == 400 * flops
	t4, l4, ms4, w4, aw4 = run(4)
	assert l4 == 400 and aw4 == 400 * flops and w4 == t4 * flops
	assert 60 <= t4 <= 140  # a quarter of 400, give or take
	assert run(4)[0] == t4  # the same picks every run
	# same kernel, same rate: the sampled mean duration within 15 % or 3 us of the full one (a timed dispatch behind an
	# untimed one stamps its start before the predecessor has drained: 1-2 us on an 8 us kernel)
	assert abs(ms4 / t4 - ms1 / t1) <= max(0.15 * (ms1 / t1), 3e-3)
	assert lib.elf_prof_launches(99, None) == 0
