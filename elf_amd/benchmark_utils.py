"""Scheduler wrappers that define the offload set and the checkpoint set of a run (behaviour of
the reference's benchmarks/benchmark_utils.py:295-407)."""

from .registry import SCHEDULERS, resolve
from .scheduling import Operation, OperationType, OpOptions, compute_types

__all__ = ["get_checkpointed_scheduler", "get_offloaded_scheduler", "SIMPLE_REMAT_CLASSES", "ATTENTION_REMAT_CLASSES"]

# class names selected by the "simple" / "selective" strategies (matched on the class name so
# that both torch.nn modules and this package's own blocks qualify)
SIMPLE_REMAT_CLASSES = ("GELU", "LayerNorm", "Dropout")
ATTENTION_REMAT_CLASSES = ("Attention", "FastAttention")


def _strategy(kind):
	if kind == "full":
		return lambda name, module: name == ""
	if kind == "simple":
		return lambda name, module: type(module).__name__ in SIMPLE_REMAT_CLASSES
	if kind == "selective":
		return lambda name, module: type(module).__name__ in ATTENTION_REMAT_CLASSES
	raise ValueError(f"Invalid checkpointing type: {kind}")


def get_checkpointed_scheduler(scheduler, type):
	"""Every FORWARD gets a ``remat_strategy``: "full" (the stage root), "simple" (GELU /
	LayerNorm / Dropout modules) or "selective" (attention cores)."""
	base = resolve(scheduler, SCHEDULERS)
	strategy = _strategy(type)

	def checkpointed_scheduler(*args, **kwargs):
		schedule = base(*args, **kwargs)
		for op in schedule:
			if op.op == OperationType.FORWARD:
				op.options[OpOptions.REMAT_STRATEGY] = strategy
		return schedule

	return checkpointed_scheduler


def get_offloaded_scheduler(scheduler, ratio, prefetching_time=1):
	"""Marks F(mb) (and its B) with ``activation_offload`` when ``mb % ratio == 0`` and inserts a
	PREFETCH_ACTIVATIONS op before the ``prefetching_time``-th compute op (W passes not counted)
	that precedes that B on its rank.  When that walk back reaches the offloaded F itself there is
	no room to prefetch and the micro-batch is not offloaded."""
	base = resolve(scheduler, SCHEDULERS)
	F, B, W = OperationType.FORWARD, OperationType.BACKWARD_INPUTS, OperationType.BACKWARD_PARAMS
	OFF = OpOptions.ACTIVATION_OFFLOAD

	def offloaded_scheduler(*args, **kwargs):
		schedule = base(*args, **kwargs)
		placement = args[0]
		marked = [[] for _ in range(max(placement) + 1)]
		for op in schedule:
			if op.op == F and op.mb_id % ratio == 0:
				op.options[OFF] = True
				marked[op.rank].append((op.mb_id, op.block_id))

		def is_f_of(op, mb, block):
			return op.op == F and op.mb_id == mb and op.block_id == block

		for rank, pairs in enumerate(marked):
			for mb, block in pairs:
				b_idx = next(i for i, op in enumerate(schedule) if op.block_id == block and op.mb_id == mb and op.op == B)
				b_op = schedule[b_idx]
				b_op.options[OFF] = True
				seen = 0
				for i in range(b_idx - 1, -1, -1):
					op = schedule[i]
					if op.rank != rank or op.op not in compute_types or op.op == W:
						continue
					seen += 1
					if is_f_of(op, mb, block):
						op.options[OFF] = False
						b_op.options[OFF] = False
						break
					if seen == prefetching_time:
						# the compute op just before the insertion point being the offloaded F only
						# clears the F's flag (the B keeps its flag); then the prefetch is inserted
						for j in range(i - 1, -1, -1):
							prev = schedule[j]
							if prev.rank == rank and prev.op in compute_types:
								if is_f_of(prev, mb, block):
									prev.options[OFF] = False
									b_op.options[OFF] = True
								break
						schedule.insert(i, Operation(block, mb, OperationType.PREFETCH_ACTIVATIONS, rank))
						break
		return schedule

	return offloaded_scheduler
