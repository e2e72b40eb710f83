"""Host logic of the Engine with stand-in blocks (no GPU): dispatch order, slot hand-offs
between same-rank blocks, loss scaling, statistics surface, error paths of the Variable slots."""

import pytest
import torch

from elf_amd.execution import Engine, Variable, compute_loss
from elf_amd.partitioners.utils import sequential_signatures
from elf_amd.registry import COMM_SCHEDULERS, SCHEDULERS
from elf_amd.scheduling import OperationType as T, add_comms


class FakeBlock:
	"""y = 2x forward, dx = 2 dy backward; records what the engine calls."""

	def __init__(self, id_, placement):
		sig = sequential_signatures(placement)[id_]
		self.id, self.rank, self.placement = id_, placement[id_], placement
		self.is_first, self.is_last = id_ == 0, id_ == len(placement) - 1
		self.input_variables = [Variable(n, s) for n, s in zip(sig.inputs, sig.sources)]
		self.output_variables = [[Variable(n, d) for d in dsts] for n, dsts in zip(sig.outputs, sig.targets)]
		self.compute_time, self.calls = [], []
		self.model = torch.nn.Linear(1, 1)

	def forward(self, mb, **opts):
		self.calls.append(("F", mb))
		x = self.input_variables[0].wait_and_pop(mb)
		y = 2 * x
		out = self.output_variables[0][0]
		out.set(out.to_send, mb, y)
		self.input_variables[0].set(self.input_variables[0].saved, mb, x)
		if self.is_last:
			return [out.get(out.to_send, mb)]

	def backward_inputs(self, mb, **opts):
		self.calls.append(("B", mb))
		self.input_variables[0].get(self.input_variables[0].saved, mb)
		dy = self.output_variables[0][0].wait_and_pop(mb)
		self.input_variables[0].set(self.input_variables[0].to_send, mb, 2 * dy)

	def backward_params(self, mb, **opts):
		self.calls.append(("W", mb))

	def scale_grads(self, n):
		self.calls.append(("scale", n))

	def all_reduce_param_grads(self, **opts):
		self.calls.append(("AR", None))

	def send_forward(self, mb, **o): pass
	def send_backward(self, mb, **o): pass
	def recv_forward(self, mb, size, **o): pass
	def recv_backward(self, mb, size, **o): pass


def test_engine_runs_a_two_block_pipeline_on_one_rank():
	placement = [0, 0]
	blocks = [FakeBlock(0, placement), FakeBlock(1, placement)]
	schedule = COMM_SCHEDULERS["pipelined"](add_comms(SCHEDULERS["afab"](placement, 2), sequential_signatures(placement)))
	x = torch.arange(8.0).reshape(4, 2)
	target = torch.zeros(4, 2)
	result, losses, stats, detailed = Engine(blocks).train_step([x], target, torch.nn.functional.mse_loss, schedule, [2, 2])
	assert torch.equal(torch.cat(result), 4 * x)
	# per micro-batch: sum over samples of squared error / elements per sample
	assert torch.allclose(torch.stack(losses), torch.stack([((4 * x[:2]) ** 2).sum() / 2, ((4 * x[2:]) ** 2).sum() / 2]))
	assert blocks[0].calls[-2:] == [("scale", 4), ("AR", None)]
	assert [c for c in blocks[1].calls if c[0] in "FBW"] == [("F", 0), ("F", 1), ("B", 0), ("W", 0), ("B", 1), ("W", 1)]
	assert set(stats) == {"total", "idle", "start_idle", "end_idle", "bubble"}
	assert list(detailed) == ["all_events", "memories", "peak_memory"]
	assert list(detailed["memories"]) == list(dict.fromkeys(str(op) for op in schedule))
	# loss = sum((4x)^2) / 2 per micro-batch -> dL/dy = 4x, then two backwards of y = 2x: dL/dx = 16x.
	# It stays in the first block's outgoing slot (SEND_BACKWARD has no peer there); everything
	# else was consumed.
	left = blocks[0].input_variables[0].to_send
	assert torch.equal(torch.cat(left), 16 * x)
	for b in blocks:
		for v in b.input_variables + [d for var in b.output_variables for d in var]:
			assert all(s is None for s in v.to_process), v._state()
	assert all(s is None for s in blocks[1].input_variables[0].to_send)


def test_engine_skips_other_ranks_and_rejects_unknown_ops():
	blk = FakeBlock(0, [0, 1])
	sched = SCHEDULERS["afab"]([0, 1], 1)
	eng = Engine([blk])
	with pytest.raises(Exception, match="shorter than mb_id|empty"):
		eng.train_step(None, None, None, [op for op in sched if op.op == T.FORWARD], [1])  # no input was received
	class Weird: op, block_id, mb_id, options = "nope", 0, 0, {}
	with pytest.raises(Exception, match="Unknown operation"):
		eng.train_step(None, None, None, [Weird()], [1])


def test_variable_slot_rules():
	v = Variable("x", 3)
	v.set(v.saved, 2, "a")
	assert v.saved == [None, None, "a"]
	with pytest.raises(Exception, match="already set"):
		v.set(v.saved, 2, "b")
	assert v.get(v.saved, 2, delete=False) == "a" and v.get(v.saved, 2) == "a"
	with pytest.raises(Exception, match="empty"):
		v.get(v.saved, 2)
	with pytest.raises(Exception, match="shorter"):
		v.get(v.to_send, 0)

	class Work:
		waited = False
		def wait(self): self.waited = True

	w, t = Work(), torch.ones(2, requires_grad=True) * 2
	v.set(v.to_process, 0, (w, t))
	out = v.wait_and_pop(0)
	assert w.waited and not out.requires_grad
	v.clear()
	assert v.saved == [] and str(v) == "Variable(name=x,peer=3,metadata=None)"


def test_compute_loss_matches_mean_reduction_after_batch_scaling():
	blk = FakeBlock(1, [0, 1])
	out = torch.randn(3, 5, requires_grad=False)
	tgt = torch.randn(3, 5)
	loss, grad_fn = compute_loss(blk, out, tgt, torch.nn.functional.mse_loss)
	(g,) = grad_fn()
	ref_in = out.clone().requires_grad_(True)
	ref = torch.nn.functional.mse_loss(ref_in, tgt)  # mean over 15 elements
	ref.backward()
	assert torch.allclose(loss / 3, ref) and torch.allclose(g / 3, ref_in.grad)
	assert blk.compute_time[0].name == "loss_forward"


@pytest.mark.parametrize("scheduler,placement,nmb", [("1f1b", [0, 1], 4), ("zbh1", [0, 1, 2, 3], 8), ("1f1b", [0, 1, 0, 1], 4), ("afab", [0, 1, 2], 3), ("zbh2", [0, 1, 2, 3], 4)])
@pytest.mark.parametrize("comm", ["pipelined", "topo", "simulation"])
def test_sequential_order_lets_one_process_play_every_rank(scheduler, placement, nmb, comm):
	"""``sequential_order`` (the order ``Pipeline(all_ranks=True)`` runs a multi-rank schedule in): the same ops, every
	rank's own order kept, each FORWARD after the SEND_FORWARD that feeds it and each BACKWARD_INPUTS after the
	SEND_BACKWARD of its consumer; the Engine then runs all blocks of the placement on stand-in blocks and the
	values that come out are those of the chain y = 2^n x."""
	from elf_amd.pipeline import sequential_order

	sigs = sequential_signatures(placement)
	schedule = COMM_SCHEDULERS[comm](add_comms(SCHEDULERS[scheduler](placement, nmb), sigs))
	order = sequential_order(schedule, sigs)
	assert sorted(map(id, order)) == sorted(map(id, schedule))
	for r in set(placement):
		assert [op for op in order if op.rank == r] == [op for op in schedule if op.rank == r]
	pos = {id(op): i for i, op in enumerate(order)}
	for op in order:
		if op.op == T.FORWARD and op.block_id > 0:
			send = next(o for o in order if o.op == T.SEND_FORWARD and o.block_id == op.block_id - 1 and o.mb_id == op.mb_id and o.options.get("dst") == op.block_id)
			assert pos[id(send)] < pos[id(op)]
		if op.op == T.BACKWARD_INPUTS and op.block_id < len(placement) - 1:
			send = next(o for o in order if o.op == T.SEND_BACKWARD and o.block_id == op.block_id + 1 and o.mb_id == op.mb_id and o.options.get("dst") == op.block_id)
			assert pos[id(send)] < pos[id(op)]
	blocks = [FakeBlock(i, placement) for i in range(len(placement))]
	for b in blocks:
		b.local_ids = set(range(len(placement)))
	x = torch.arange(float(2 * nmb)).reshape(nmb, 2)
	result, losses, _, _ = Engine(blocks, all_ranks=True).train_step([x], torch.zeros(nmb, 2), torch.nn.functional.mse_loss, order, [1] * nmb)
	assert torch.equal(torch.cat(result), (2 ** len(placement)) * x)
	assert all(sum(c[0] == k for c in b.calls) == nmb for b in blocks for k in "FBW")
	left = blocks[0].input_variables[0].to_send
	assert torch.equal(torch.cat(left), (2 ** (2 * len(placement))) * x)  # dL/dy = 2y / 2, back through the chain


def test_sequential_order_reports_a_schedule_that_cannot_run():
	from elf_amd.pipeline import sequential_order
	from elf_amd.scheduling import Operation

	sigs = sequential_signatures([0, 1])
	stuck = [Operation(1, 0, T.FORWARD, 1)]  # nobody ever sends block 1 its input
	with pytest.raises(RuntimeError, match="deadlock"):
		sequential_order(stuck, sigs)
	with pytest.raises(AssertionError):
		Engine([FakeBlock(0, [0, 1]), FakeBlock(1, [0, 1])])  # two ranks without all_ranks
