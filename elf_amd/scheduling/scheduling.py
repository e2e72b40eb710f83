"""Data model of a schedule: operation kinds, per-operation options and the Operation record.

Behaviour follows the reference's elf/scheduling/scheduling.py (OperationType :12-37, comm/compute
type sets :40-55, OpOptions :58-86, Operation :89-127, matching/get_peer :130-160,
schedule_to_str :163-229, check_schedule_validity :232-270), including the quirks its callers
rely on: ``Operation.__eq__`` ignores ``block_id`` while ``__hash__`` ignores ``options``, and
option keys are strings equal to their lower-case names.
"""

from enum import Enum

__all__ = [
	"OperationType", "OpOptions", "Operation", "comm_types", "compute_types", "matching",
	"get_peer", "get_peer_rank", "schedule_to_str", "check_schedule_validity",
]


class OperationType(Enum):
	RECV_FORWARD = 0
	FORWARD = 1
	SEND_FORWARD = 2
	RECV_BACKWARD = 3
	BACKWARD_INPUTS = 4
	BACKWARD_PARAMS = 5
	SEND_BACKWARD = 6
	LOSS_FORWARD = 7
	LOSS_BACKWARD = 8
	ALL_REDUCE_PARAM_GRADS = 9
	RECOMPUTE_FORWARD = 10
	RECOMPUTE_BACKWARD_INPUTS = 11
	PREFETCH_ACTIVATIONS = 12

	def __str__(self):
		return self.name.lower()

	__repr__ = __str__


_T = OperationType
comm_types = {_T.RECV_FORWARD, _T.RECV_BACKWARD, _T.SEND_FORWARD, _T.SEND_BACKWARD}
# LOSS_FORWARD / LOSS_BACKWARD are deliberately not "compute": the simulation-based comm
# schedulers drain them between time steps.
compute_types = {_T.FORWARD, _T.BACKWARD_INPUTS, _T.BACKWARD_PARAMS, _T.RECOMPUTE_FORWARD, _T.RECOMPUTE_BACKWARD_INPUTS}


class OpOptions(str, Enum):
	"""Option keys.  Members are strings (usable as ``**kwargs`` names and interchangeable with
	their plain-string spelling in dict lookups), as with enum.StrEnum + auto() on Python 3.11:

	remat_strategy         ``(name, module) -> bool``: which sub-modules are recomputed in backward
	recompute_activations  drop the linear layers' inputs after B, recompute them before W
	recompute_gradients    drop the linear layers' output gradients after B, recompute before W
	activation_offload     keep the forward's saved activations in pinned host memory
	save                   for RECOMPUTE_FORWARD: rebuild the graph for a second backward
	offload_dw             offload the weight-gradient computation
	"""

	REMAT_STRATEGY = "remat_strategy"
	RECOMPUTE_ACTIVATIONS = "recompute_activations"
	RECOMPUTE_GRADIENTS = "recompute_gradients"
	ACTIVATION_OFFLOAD = "activation_offload"
	SAVE = "save"
	OFFLOAD_DW = "offload_dw"

	def __str__(self):
		return self.value

	def __format__(self, spec):
		return format(self.value, spec)

	__hash__ = str.__hash__


class Operation:
	"""One entry of a schedule: which block does what to which micro-batch on which rank."""

	def __init__(self, block_id, mb_id, op, rank, **options):
		self.block_id = block_id
		self.mb_id = mb_id
		self.op = op
		self.rank = rank
		self.options = options

	def __str__(self):
		return f"[Block {self.block_id}, mb {self.mb_id}]:{self.op!r}({self.options})"

	__repr__ = __str__

	def __eq__(self, other):
		return (other.op, other.mb_id, other.rank, other.options) == (self.op, self.mb_id, self.rank, self.options)

	def __hash__(self):
		return hash((self.block_id, self.mb_id, self.rank, self.op))


_MATCH = {
	_T.RECV_FORWARD: _T.SEND_FORWARD, _T.SEND_FORWARD: _T.RECV_FORWARD,
	_T.RECV_BACKWARD: _T.SEND_BACKWARD, _T.SEND_BACKWARD: _T.RECV_BACKWARD,
}


def matching(op_type):
	"""The opposite end of a transfer in the same direction (recv_forward <-> send_forward ...)."""
	return _MATCH[op_type]


def get_peer(op):
	"""Peer block id of a communication op (``dst`` wins over ``src``), None if it has neither."""
	return op.options.get("dst", op.options.get("src", None))


def get_peer_rank(op, placement):
	peer = get_peer(op)
	return None if peer is None else placement[peer]


_LETTERS = {
	_T.RECV_FORWARD: "rf", _T.FORWARD: "f", _T.SEND_FORWARD: "sf", _T.RECV_BACKWARD: "rb",
	_T.BACKWARD_INPUTS: "b", _T.BACKWARD_PARAMS: "w", _T.SEND_BACKWARD: "sb", _T.RECOMPUTE_FORWARD: "R",
	_T.RECOMPUTE_BACKWARD_INPUTS: "R*", _T.ALL_REDUCE_PARAM_GRADS: "(AR)", _T.PREFETCH_ACTIVATIONS: "P",
}


def _letter(op):
	if op.op == _T.FORWARD:
		recomputed = (not op.options.get(OpOptions.SAVE, True)) or bool(op.options.get(OpOptions.REMAT_STRATEGY, False))
		return "F" if recomputed else "f"
	if op.op == _T.BACKWARD_INPUTS:
		return {"full": "b", "gradients": "b*", "none": "B"}.get(op.options.get(OpOptions.SAVE, "full"), "b")
	return _LETTERS[op.op]


def schedule_to_str(schedule, print_comms=False):
	"""One line per rank: ``Rank r: f0-0 f0-1 b0-0 w0-0 ...`` (loss ops are not shown)."""
	lines = []
	for rank in sorted({op.rank for op in schedule}):
		words = []
		for op in schedule:
			if op.rank != rank or op.op not in _LETTERS:
				continue
			if op.op in comm_types and not print_comms:
				continue
			word = f"{_letter(op)}{op.block_id}-{op.mb_id if op.mb_id is not None else ''}"
			if op.op in comm_types:
				word += f"({get_peer(op)})"
			words.append(word)
		lines.append(f"Rank {rank}: " + " ".join(words))
	return "\n".join(lines)


def check_schedule_validity(schedule):
	"""Sanity checks: every rank sees every micro-batch; per (rank, micro-batch) the first F
	precedes the first B, and a B implies a W that does not precede it."""
	n_mb = len({op.mb_id for op in schedule if op.mb_id is not None})

	def first(ops, kind):
		return next((i for i, op in enumerate(ops) if op.op == kind), -1)

	for rank in {op.rank for op in schedule}:
		mine = [op for op in schedule if op.rank == rank]
		mbs = {op.mb_id for op in mine if op.mb_id is not None}
		assert len(mbs) == n_mb, f"[Rank {rank}] has {len(mbs)} microbatches, expected {n_mb}"
		for mb in mbs:
			ops = [op for op in mine if op.mb_id == mb]
			i, j, k = first(ops, _T.FORWARD), first(ops, _T.BACKWARD_INPUTS), first(ops, _T.BACKWARD_PARAMS)
			assert i != -1 or j == -1, f"[Rank {rank}] Forward should be present for microbatch {mb}"
			assert i < j or j == -1, f"[Rank {rank}] Forward should be before backward inputs for microbatch {mb}"
			assert k != -1 or j == -1, f"[Rank {rank}] Backward params should be present for microbatch {mb} since backward inputs is present"
			assert j <= k, f"[Rank {rank}] Backward params should be after backward inputs for microbatch {mb}"
