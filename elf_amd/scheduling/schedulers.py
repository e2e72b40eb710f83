"""Static schedule generators: ``(placement, n_micro_batches) -> [Operation]`` for ALL ranks.

Each generator reproduces the op order of its counterpart in the reference's
elf/scheduling/schedulers.py (afab :30-46, 1f1b :49-113, hanayo :116-164, full_remat :167-203,
zbh1 :206-242, zbh2 :245-281, zbv :284-393, inference :396-405, FixedSchedule :408-440).
The last block of the pipeline gets a LOSS_FORWARD after each F and a LOSS_BACKWARD before each B
(:14-23).
"""

import logging

from .scheduling import Operation, OperationType, OpOptions

logger = logging.getLogger("schedulers")

__all__ = [
	"generate_afab_schedule", "generate_1f1b_schedule", "generate_hanayo_schedule",
	"generate_full_remat_schedule", "generate_zbh1_schedule", "generate_zbh2_schedule",
	"generate_zbv_schedule", "generate_inference_schedule", "FixedSchedule",
]

_F, _B, _W = OperationType.FORWARD, OperationType.BACKWARD_INPUTS, OperationType.BACKWARD_PARAMS


class _Builder:
	"""Appends F / B / W ops (plus the loss ops of the last block) to one list."""

	def __init__(self, placement):
		self.placement = placement
		self.last = len(placement) - 1
		self.ops = []

	def f(self, block, mb, rank, **opts):
		self.ops.append(Operation(block, mb, _F, rank, **opts))
		if block == self.last:
			self.ops.append(Operation(block, mb, OperationType.LOSS_FORWARD, rank, **opts))

	def b(self, block, mb, rank, **opts):
		if block == self.last:
			self.ops.append(Operation(block, mb, OperationType.LOSS_BACKWARD, rank, **opts))
		self.ops.append(Operation(block, mb, _B, rank, **opts))

	def w(self, block, mb, rank, **opts):
		self.ops.append(Operation(block, mb, _W, rank, **opts))

	def bw(self, block, mb, rank):
		self.b(block, mb, rank)
		self.w(block, mb, rank)


def _blocks_of(placement, rank):
	return [i for i, r in enumerate(placement) if r == rank]


def generate_afab_schedule(placement, n_micro_batches):
	"""GPipe: every rank runs all forwards, then all backwards (B immediately followed by W)."""
	out = _Builder(placement)
	for rank in range(max(placement) + 1):
		mine = _blocks_of(placement, rank)
		for mb in range(n_micro_batches):
			for blk in mine:
				out.f(blk, mb, rank)
		for mb in range(n_micro_batches):
			for blk in reversed(mine):
				out.bw(blk, mb, rank)
	return out.ops


def generate_1f1b_schedule(placement, n_micro_batches):
	"""One-forward-one-backward (PipeDream / Megatron, interleaved when a rank owns several
	stages).  With one stage per rank, rank r of P runs min(n, P - r) warm-up forwards, then
	(B W F) until the forwards run out, then (B W) to the end."""
	out = _Builder(placement)
	n_stages = len(placement)
	n_dev = int(max(placement)) + 1
	per_dev = n_stages // n_dev
	total = per_dev * n_micro_batches  # forwards (= backwards) a rank has to run

	for rank in range(n_dev):
		done_f = [0] * per_dev  # per local stage: next micro-batch to forward
		done_b = [0] * per_dev
		step = 0
		lf = 0  # local stage that forwards next

		def forward():
			out.f(lf * n_dev + rank, done_f[lf], rank)
			done_f[lf] += 1

		def backward(lb):
			blk = lb * n_dev + rank
			out.bw(blk, done_b[lb], rank)
			done_b[lb] += 1

		# warm-up: a rank may forward until the first micro-batch could have crossed the rest of
		# the pipeline; it moves to its next local stage every n_dev (or n_micro_batches) steps
		while step < total and step < n_stages - rank:
			step += 1
			forward()
			if step % n_dev == 0 or step % n_micro_batches == 0:
				lf = (lf + 1) % per_dev
		warm = step
		lb = per_dev - 1  # backwards start from the deepest local stage

		# steady state: one backward (B, W) then one forward
		while step < total:
			step += 1
			backward(lb)
			if (step - warm) % (n_dev // 2) == 0 or (step - warm) % n_micro_batches == 0:
				lb = (lb - 1) % per_dev
			forward()
			if (step >= n_stages and step % (n_dev // 2) == 0) or step % n_micro_batches == 0:
				lf = (lf + 1) % per_dev

		# cool-down: the `warm` backwards that are still owed
		while step < 2 * total - (total - warm):
			step += 1
			backward(lb)
			k = step - n_micro_batches - warm
			if k % (n_dev // 2) == 0 or k % n_micro_batches == 0:
				lb = (lb - 1) % per_dev
	return out.ops


def generate_hanayo_schedule(placement, n_micro_batches):
	"""Hanayo wave schedule (placement is a V / W shape: each rank owns 2 * n_waves stages)."""
	out = _Builder(placement)
	n_dev = max(placement) + 1
	n_stages = len(placement)
	n_waves = n_stages // (2 * n_dev)
	mine = [_blocks_of(placement, r) for r in range(n_dev)]
	fwd = [0] * n_dev  # forwards issued on the even (downward) stages of each rank
	bwd = [0] * n_dev  # backwards issued on the odd-from-the-end stages of each rank

	for rank in range(n_dev):
		fwd[rank] = min(n_dev - rank, n_micro_batches)
		for mb in range(fwd[rank]):
			out.f(mine[rank][0], mb, rank)

	def late_backward(rank):
		blk = mine[rank][-1 - 2 * (bwd[rank] // n_micro_batches)]
		out.bw(blk, bwd[rank] % n_micro_batches, rank)
		bwd[rank] += 1

	for wave in range(n_waves):
		for mb in range(n_micro_batches):
			for rank in reversed(range(n_dev)):
				out.f(mine[rank][2 * wave + 1], mb, rank)
				if fwd[rank] < n_micro_batches * n_waves:
					out.f(mine[rank][2 * (fwd[rank] // n_micro_batches)], fwd[rank] % n_micro_batches, rank)
					fwd[rank] += 1
				else:
					late_backward(rank)

	for wave in range(n_waves):
		for mb in range(n_micro_batches):
			for rank in reversed(range(n_dev)):
				out.bw(mine[rank][-2 * (wave + 1)], mb, rank)
				if bwd[rank] < n_micro_batches * n_waves:
					late_backward(rank)
	return out.ops


def _recompute_everything(name, _module):
	return name == ""


def generate_full_remat_schedule(placement, n_micro_batches):
	"""All ranks but the last run GPipe with every forward fully checkpointed; the last rank
	alternates F and B/W per micro-batch."""
	out = _Builder(placement)
	n_dev = max(placement) + 1
	for rank in range(n_dev - 1):
		mine = _blocks_of(placement, rank)
		for mb in range(n_micro_batches):
			for blk in mine:
				out.f(blk, mb, rank, **{OpOptions.REMAT_STRATEGY: _recompute_everything})
		for mb in range(n_micro_batches):
			for blk in reversed(mine):
				out.bw(blk, mb, rank)
	rank = n_dev - 1
	mine = _blocks_of(placement, rank)
	for mb in range(n_micro_batches):
		for blk in mine:
			out.f(blk, mb, rank)
		for blk in reversed(mine):
			out.bw(blk, mb, rank)
	return out.ops


def _zb_tail(out, block, rank, n, f, b, w):
	"""Shared tail of ZB-H1 / ZB-H2: repeat (W, F, B), each while there is one left."""
	while f < n or b < n or w < n:
		if w < n:
			out.w(block, w, rank)
			w += 1
		if f < n:
			out.f(block, f, rank)
			f += 1
		if b < n:
			out.b(block, b, rank)
			b += 1


def generate_zbh1_schedule(placement, n_micro_batches):
	"""Zero-Bubble H1: min(D - block, n) warm-up forwards, B0, then `rank` (F, B) pairs, then the
	(W, F, B) tail - W passes are deferred behind the next F and B."""
	out = _Builder(placement)
	n = n_micro_batches
	n_dev = len(set(placement))
	for block, rank in enumerate(placement):
		f = b = 0
		for _ in range(min(n_dev - block, n)):
			out.f(block, f, rank)
			f += 1
		out.b(block, b, rank)
		b += 1
		for _ in range(rank):
			if f < n:
				out.f(block, f, rank)
				f += 1
			if b < n:
				out.b(block, b, rank)
				b += 1
		_zb_tail(out, block, rank, n, f, b, 0)
	return out.ops


def generate_zbh2_schedule(placement, n_micro_batches):
	"""Zero-Bubble H2: a deeper warm-up of min(n, 2 (D - block) - 1) forwards."""
	out = _Builder(placement)
	n = n_micro_batches
	n_dev = len(set(placement))
	for block, rank in enumerate(placement):
		warm = min(n, 2 * (n_dev - block) - 1)
		f = b = 0
		for _ in range(warm):
			out.f(block, f, rank)
			f += 1
		out.b(block, b, rank)
		b += 1
		for _ in range(n - 1 - warm):
			out.f(block, f, rank)
			f += 1
			out.b(block, b, rank)
			b += 1
		_zb_tail(out, block, rank, n, f, b, 0)
	return out.ops


def generate_zbv_schedule(placement, n_micro_batches):
	"""Zero-Bubble V (two stages per rank, V-shaped placement)."""
	out = _Builder(placement)
	n = n_micro_batches
	n_dev = len(set(placement))
	per_dev = len(placement) // n_dev
	if n != 2 * n_dev:
		logger.warning(f"ZBV schedule is only tested for nmb = 2 * n_devices, got {n}. The schedule may be incorrect.")

	for rank in range(n_dev):
		mine = _blocks_of(placement, rank)
		nf, nb, nw = [0] * per_dev, [0] * per_dev, [0] * per_dev

		def f(c):
			out.f(mine[c], nf[c], rank)
			nf[c] += 1

		def b(c):
			out.b(mine[c], nb[c], rank)
			nb[c] += 1

		def w(c):
			out.w(mine[c], nw[c], rank)
			nw[c] += 1

		def fbw(c):
			f(c)
			b(c)
			w(c)

		warm = min(n, 2 * (n_dev - rank) - 1)
		for _ in range(warm):  # first stage only
			f(0)
		c = 1
		for _ in range(2 * n_dev - warm - 1):  # alternate, starting with the second stage
			f(c)
			c = 1 - c
		for _ in range(n_dev - rank):  # steady state on the second stage
			fbw(1)
		for _ in range(rank + 1):  # steady state alternating
			fbw(0)
			fbw(1)
		for _ in range(n_dev - rank - 1):  # the irregular stretch: (B W) on stage 0, (F B W) on stage 1
			b(0)
			w(0)
			fbw(1)
		c = 0
		for _ in range(2 * n_dev - warm):  # cool-down: backwards only, alternating
			b(c)
			c = 1 - c
		for _ in range(n_dev - rank - 1):
			w(0)
			b(0)
		for _ in range(rank + 1):
			w(0)
		for _ in range(rank):
			w(1)
		for i in range(per_dev):
			assert nf[i] == nb[i] == nw[i] == n, f"Rank {rank}, stage {i}: f = {nf[i]}, b = {nb[i]}, w = {nw[i]} (expected {n})"
	return out.ops


def generate_inference_schedule(placement, n_micro_batches):
	"""Forward only, block by block; no loss ops."""
	return [Operation(blk, mb, _F, rank) for blk, rank in enumerate(placement) for mb in range(n_micro_batches)]


class FixedSchedule:
	"""Scheduler from an explicit order: ``{"order": [(optype, block_id, mb_id), ...]}`` with
	optype in "f" / "b" / "w"."""

	def __init__(self, schedule_dict):
		self.schedule_dict = schedule_dict

	def __call__(self, placement, n_micro_batches):
		out = _Builder(placement)
		emit = {"f": out.f, "b": out.b, "w": out.w}
		for kind, block, mb in self.schedule_dict["order"]:
			block, mb = int(block), int(mb)
			if kind in emit:
				emit[kind](block, mb, placement[block])
		return out.ops
