"""``Pipeline`` / ``PipelineConfig``: the orchestration API of the reference (elf/pipeline.py:40-95,
97-207, 209-295, 453-534) over the native stage executor.

What is the same: the configuration fields and their registry resolution, placement defaults,
micro-batch splitting (``_get_mb_sizes``), schedule generation (scheduler -> ``add_comms`` ->
comm scheduler -> validity check -> filter by owned block ids), lazy ILP remat when
``memory_budget`` is set (stages profiled at construction, ILP solved at the first step), the
per-step clearing of the Variable slots, ``stats`` / ``detailed_stats``, the return value of
``step`` and the parameter helpers.

What differs, because this build runs one process on one GPU: the stages this process owns are
``HipStageBlock`` objects (chains of transformer blocks run by the HIP library), the model has to
arrive already partitioned (``partitioner=False``: tracing and graph partitioning are not part of
this path), every stage of the placement must live on this process' rank (stages on the same rank
hand tensors over locally, as in the reference engine), and no process groups are created.
``all_ranks=True`` lets the one process play every rank of a placement such as ``[0, 1]``: it owns
all stages, hands boundary tensors over locally and interprets the ops of all ranks in an order in
which every rank keeps its own op order and no compute op runs before the data it consumes was sent
(``sequential_order``), so that a schedule written for several devices runs on one.
"""

import logging
import os
from dataclasses import asdict, dataclass, field, fields
from typing import Any, List

import torch
import torch.distributed as dist

from .execution import AutogradStageBlock, Engine, HipStageBlock
from .models import EndStage, LlamaBlock, TransformerBlock
from .partitioners.utils import Signature, sequential_signatures
from .registry import COMM_SCHEDULERS, PARTITIONERS, SCHEDULERS, TRACERS, resolve
from .scheduling import OperationType, add_comms, check_schedule_validity, schedule_to_str
from .scheduling.ilp import AutoScheduler, profile_stage, stagerematify
from .utils import Placement

logger = logging.getLogger("pipeline")

__all__ = ["Pipeline", "PipelineConfig", "sequential_order"]


def sequential_order(schedule, signatures):
	"""One order in which a single process can run the ops of every rank of ``schedule``.

	Each rank's ops keep their relative order.  Receives are posts (``irecv`` in the reference,
	block.py:420-446) and never block; a FORWARD waits until every producer of the block's inputs has
	emitted its SEND_FORWARD for that micro-batch, a BACKWARD_INPUTS until every consumer of its
	outputs has emitted its SEND_BACKWARD: what ``Variable.wait_and_pop`` waits for.  Ranks are served
	round-robin, each running until its next op has to wait.  Raises if the schedule deadlocks."""
	T = OperationType
	ranks = sorted({op.rank for op in schedule})
	queues = {r: [op for op in schedule if op.rank == r] for r in ranks}
	heads = {r: 0 for r in ranks}
	sent = set()  # (kind, producing block, consuming block, micro-batch)

	def ready(op):
		sig = signatures[op.block_id]
		if op.op == T.FORWARD:
			return all((T.SEND_FORWARD, src, op.block_id, op.mb_id) in sent for src in sig.get_all_sources() if src is not None)
		if op.op == T.BACKWARD_INPUTS:
			return all((T.SEND_BACKWARD, dst, op.block_id, op.mb_id) in sent for dst in sig.get_all_targets() if dst is not None)
		return True

	out = []
	while any(heads[r] < len(queues[r]) for r in ranks):
		progressed = False
		for r in ranks:
			while heads[r] < len(queues[r]) and ready(queues[r][heads[r]]):
				op = queues[r][heads[r]]
				heads[r] += 1
				if op.op in (T.SEND_FORWARD, T.SEND_BACKWARD):
					sent.add((op.op, op.block_id, op.options.get("dst"), op.mb_id))
				out.append(op)
				progressed = True
		if not progressed:
			stuck = {r: str(queues[r][heads[r]]) for r in ranks if heads[r] < len(queues[r])}
			raise RuntimeError(f"sequential_order: the schedule deadlocks, every rank waits: {stuck}")
	return out


@dataclass
class PipelineConfig:
	"""Same fields and defaults as elf/pipeline.py:40-78.  Registry fields accept a key or an object;
	``partitioner`` may be False (the model is already partitioned), which is the only mode this build
	runs."""

	tracer: Any = field(default="default", metadata={"registry": TRACERS})
	partitioner: Any = field(default="constrained", metadata={"registry": PARTITIONERS})
	scheduler: Any = field(default="auto", metadata={"registry": SCHEDULERS})
	comm_scheduler: Any = field(default="pipelined", metadata={"registry": COMM_SCHEDULERS})
	placement: Any = "auto"
	pp: Any = None
	dp: int = 1
	worker: int = 0
	memory_budget: Any = None
	signatures: Any = None

	def resolve(self):
		resolved = {}
		for f in fields(self):
			val = getattr(self, f.name)
			registry = f.metadata.get("registry")
			resolved[f.name] = resolve(val, registry) if registry is not None and val is not False else val
		return PipelineConfig(**resolved)

	def to_kwargs(self):
		return {k: v for k, v in asdict(self).items() if v is not None}


def _is_transformer_chain(module):
	"""Whether ``module`` is what ``HipStageBlock`` runs inside the library: a chain of ``TransformerBlock``
	or of ``LlamaBlock`` modules, bare or inside an ``EndStage``.  Any other stage module runs through
	``AutogradStageBlock`` (PyTorch autograd with the linear layers on the HIP GEMM)."""
	core = module.blocks if isinstance(module, EndStage) else module
	blocks = [core] if isinstance(core, (TransformerBlock, LlamaBlock)) else list(core.children())
	return bool(blocks) and all(isinstance(b, (TransformerBlock, LlamaBlock)) for b in blocks) and len({type(b) for b in blocks}) == 1 and getattr(core, "seq_len", None) is not None


def _world():
	if dist.is_available() and dist.is_initialized():
		return dist.get_world_size(), dist.get_rank()
	return 1, 0


class Pipeline:
	"""``Pipeline(model, sample, scheduler="afab", partitioner=False, placement=[0, 0], mb_size=2)``.

	``model``: one stage module (a chain of ``TransformerBlock`` / ``LlamaBlock``, e.g. a
	``StageModule``) or the list of stage modules this rank owns, in block-id order.  ``sample`` has
	the shape of one micro-batch ``[mb, seq, d_model]`` (or pass ``mb_size=``)."""

	def __init__(self, model, sample=None, *, config=None, mb_size=None, all_ranks=False, **kwargs):
		ws, rank = _world()
		if ws == 1 and not (dist.is_available() and dist.is_initialized()):
			logger.warning("Trying to create a pipeline but no multi-gpu distributed setup has been found.")
		self.cfg = (config or PipelineConfig(**kwargs)).resolve()
		self.all_ranks = bool(all_ranks)
		if ws != 1:
			raise NotImplementedError("this build runs the stages of one process on one GPU: start it with a world size of 1")
		if self.all_ranks:
			if self.cfg.placement == "auto" and not self.cfg.pp:
				raise ValueError("Pipeline(all_ranks=True) needs an explicit placement or pp")
			self.pp = self.cfg.pp or len(set(self.cfg.placement))
			self.dp = 1
		else:
			self.pp = self.cfg.pp or ws // self.cfg.dp
			self.dp = self.cfg.dp
			assert self.pp * self.dp == ws, f"Requested PP = {self.pp}, DP = {self.dp} need {self.pp * self.dp} processes, but {ws} were spawned"
		self.rank = rank
		if self.cfg.placement == "auto":
			try:
				name = SCHEDULERS.get_key(self.cfg.scheduler)
			except ValueError:
				name = ""
			self.placement = Placement.default(name, self.pp)
		else:
			self.placement = Placement(self.cfg.placement)
		self.dp_rank = rank // self.pp
		self.placement = self.placement.add_offset(self.dp_rank * self.pp)
		self.pp_group, self.dp_groups = None, None

		self.scheduler = self.cfg.scheduler
		self.tracer = self.cfg.tracer
		self.partitioner = self.cfg.partitioner

		parts, signatures = self._partition_model(model, sample, self.cfg.signatures)
		self.signatures = signatures
		if mb_size is None:
			if sample is None:
				raise ValueError("Pipeline: pass a micro-batch-sized sample or mb_size= (the stage buffers are sized for one micro-batch)")
			mb_size = (sample[0] if isinstance(sample, (list, tuple)) else sample).size(0)
		self.mb_size = int(mb_size)
		self.blocks = self._create_pipeline(parts, signatures)
		self.engine = Engine(self.blocks, all_ranks=self.all_ranks)
		self.schedule = []
		self.last_nmb = 0
		self.stats, self.detailed_stats = None, None

		# ILP remat: profile now, solve lazily at the first step() (elf/pipeline.py:186-207)
		self._remat_stats = None
		if self.cfg.memory_budget is not None:
			if any(not isinstance(b, HipStageBlock) for b in self.blocks):
				raise NotImplementedError("Pipeline: memory_budget profiles stages on the native executor; a stage that is not a chain of transformer blocks cannot be profiled")
			# the stages profiled at both lean stash levels: the ILP's makespan decides which one the step runs with (the
			# leaner stash costs two GEMMs per block in B and saves whole recomputed forwards where memory is tight)
			assert len(self.blocks) == len(self.placement), "memory_budget needs the statistics of every stage of the placement"

			def at_level(level):
				def apply():
					for b in self.blocks:
						b.set_lean_stash(level)
				return apply

			self._remat_stats = []
			for level in (1, 2):
				at_level(level)()
				own = {b.id: profile_stage(b)[0] for b in self.blocks}
				self._remat_stats.append((f"lean stash level {level}", [own[i] for i in range(len(self.placement))], at_level(level)))
			if self.scheduler is SCHEDULERS.get("auto"):
				self.scheduler = AutoScheduler(self._remat_stats, self.cfg.memory_budget, self.cfg.worker)
			else:
				self.scheduler = stagerematify(self.scheduler, self._remat_stats, self.cfg.memory_budget, self.cfg.worker)

	# ------------------------------------------------------------------ training step
	def step(self, batch, target, loss_fn, split_size=0, profile=False, scheduler=None):
		"""One pass of the schedule over ``batch`` (elf/pipeline.py:209-295).  Returns
		``(outputs per micro-batch, loss)`` when this process owns the last stage, else ``(None, None)``;
		the loss is the sum of the micro-batch losses divided by the batch size."""
		batch, mb_sizes = self._prepare(batch, split_size, scheduler)

		result, losses, stats, detailed_stats = self.engine.train_step(batch, target, loss_fn, self.schedule, mb_sizes, profile)

		for block in self.blocks:
			block._wait_for_send_ops()
			for var in block.input_variables:
				var.clear()
			for var in block.output_variables:
				for dst in var:
					dst.clear()
			(getattr(block, "end_step", None) or block.clear)()
		self.stats, self.detailed_stats = stats, detailed_stats
		if len(result) != 0:
			with torch.no_grad():
				losses = torch.stack([torch.as_tensor(l, dtype=torch.float32, device="cuda") for l in losses]).sum() / sum(mb_sizes)
			return result, losses
		return None, None

	def __call__(self, *args, **kwargs):
		return self.step(*args, **kwargs)

	def _prepare(self, batch, split_size, scheduler):
		"""Micro-batch sizes of ``batch`` and, when their number changed (or a scheduler is given), a new
		schedule (elf/pipeline.py:237-252)."""
		if batch is not None and isinstance(batch, torch.Tensor):
			batch = [batch]
		mb_sizes = self._get_mb_sizes(split_size, batch)
		if any(not 1 <= m <= self.mb_size for m in mb_sizes):
			raise ValueError(f"Pipeline: the stage buffers are sized for micro-batches of 1..{self.mb_size} samples, got sizes {sorted(set(mb_sizes))}")
		n_micro_batches = len(mb_sizes)
		regenerate = scheduler is not None or n_micro_batches != self.last_nmb
		scheduler = self.scheduler if scheduler is None else resolve(scheduler, SCHEDULERS)
		if regenerate:
			self._generate_schedule(n_micro_batches, scheduler, self.cfg.comm_scheduler, mb_sizes)
			self.last_nmb = n_micro_batches
		return batch, mb_sizes

	def capture_step(self, batch, target, loss_fn, split_size=0, scheduler=None, warmup=1):
		"""``step`` recorded once as a HIP graph (``Engine.capture``).  Returns a callable
		``replay(batch=None, target=None) -> (outputs per micro-batch, loss)`` with the shapes of the
		captured call; outputs and loss are the same tensors at every replay.  No counterpart in the
		reference; for steps whose kernels are short enough that launching them is what takes the time."""
		batch, mb_sizes = self._prepare(batch, split_size, scheduler)
		graphed = self.engine.capture(batch, target, loss_fn, self.schedule, mb_sizes, warmup)
		total = sum(mb_sizes)

		def replay(batch=None, target=None):
			result, losses = graphed.replay(batch, target)
			if len(result) == 0:
				return None, None
			with torch.no_grad():
				return result, torch.stack([torch.as_tensor(l, dtype=torch.float32, device="cuda") for l in losses]).sum() / total

		replay.graphed = graphed
		return replay

	# ------------------------------------------------------------------ parameters
	def parameters(self):
		for block in self.blocks:
			yield from block.model.parameters()

	def named_parameters(self):
		for block in self.blocks:
			yield from block.model.named_parameters()

	def zero_grad(self, set_to_none=True):
		"""Clears the fp32 accumulators the stages add into and the ``param.grad`` views."""
		for block in self.blocks:
			block.zero_grad()

	def clear(self):
		"""The reference synchronises and destroys its process groups here; there are none."""
		torch.cuda.synchronize()
		for block in self.blocks:
			block.clear()

	# ------------------------------------------------------------------ checkpoints (elf/pipeline.py:346-451)
	def checkpoint(self, epoch="init", dir_path="./"):
		"""One file per rank, ``{dir_path}/{epoch}/dp{dp}_pp{pp}.pt`` holding ``rank``, ``pp``, ``dp``,
		``epoch`` and one ``state_dict_{block id}`` per owned block: the reference's format."""
		dp, pp = self.rank // self.pp, self.rank % self.pp
		state = {"rank": self.rank, "pp": pp, "dp": dp, "epoch": epoch}
		for block in self.blocks:
			state[f"state_dict_{block.id}"] = {k: v.data.clone() for k, v in block.model.state_dict().items()}
		dir_path = f"{dir_path}/{epoch}/"
		os.makedirs(dir_path, exist_ok=True)
		torch.save(state, f"{dir_path}/dp{dp}_pp{pp}.pt")

	def load_checkpoint(self, epoch="init", dir_path="./"):
		"""Reads this rank's file back into the owned blocks (the values land in the fused weight
		buffers the library reads, since the modules' parameters are views of them)."""
		dp, pp = self.rank // self.pp, self.rank % self.pp
		state = torch.load(f"{dir_path}/{epoch}/dp{dp}_pp{pp}.pt", map_location="cuda", weights_only=True)
		for block in self.blocks:
			with torch.no_grad():
				for k, v in block.model.state_dict().items():
					v.copy_(state[f"state_dict_{block.id}"][k])

	def gather_parameters(self, dst=0):
		"""{parameter name: tensor} of every block (all of them live on this rank); a name that occurs in
		several blocks keeps its first occurrence, as in the reference."""
		if self.rank != dst:
			return {}
		out = {}
		for block in self.blocks:
			for name, param in block.model.named_parameters():
				if name not in out:
					out[name] = param.data
				else:
					logger.warning(f"Duplicate parameter {name} found in block {block.id}, using first occurrence")
		return out

	def save(self, path, worker=0):
		"""All parameters of the pipeline on the CPU in one file."""
		if self.rank == worker:
			torch.save({name: p.detach().cpu() for name, p in self.named_parameters()}, path)
			logger.info(f"Saved model to {path}")

	def is_first(self):
		return self.all_ranks or self.placement.is_head(self.rank)

	def is_last(self):
		return self.all_ranks or self.placement.is_tail(self.rank)

	def get_profiling_statistics(self):
		if not self._remat_stats:
			raise ValueError("Profiling statistics are not available before the first step() with a memory budget")
		# of the stash level the stages are at (the one the ILP chose, once a step has run)
		return self._remat_stats[max(1, self.blocks[0].lean_stash) - 1][1]

	# ------------------------------------------------------------------ helpers (same arithmetic as the reference)
	def _get_mb_sizes(self, split_size, batch):
		batch_size = batch[0].size(0)
		if isinstance(split_size, int):
			if split_size > batch_size:
				logger.warning(f"Split size {split_size} is greater than batch size {batch_size}")
				split_size = batch_size
			if split_size == 0:
				split_size = batch_size // self.pp if self.pp <= batch_size else 1
			mb_sizes = [split_size] * (batch_size // split_size)
			if batch_size % split_size != 0:
				mb_sizes.append(batch_size % split_size)
		else:
			assert sum(split_size) == batch_size, "Splits do not cover the entire batch"
			mb_sizes = split_size
		return mb_sizes

	def _generate_schedule(self, n_micro_batches, scheduler, comm_scheduler, mb_sizes):
		schedule = scheduler(self.placement, n_micro_batches)
		schedule = add_comms(schedule, self.signatures)
		if comm_scheduler:
			schedule = comm_scheduler(schedule)
		check_schedule_validity(schedule)
		if self.rank == 0:
			logger.debug(f"Schedule:\n{schedule_to_str(schedule)}")
		if self.all_ranks:
			schedule = sequential_order(schedule, self.signatures)
		ids = [b.id for b in self.blocks]
		self.schedule = [op for op in schedule if op.block_id in ids]

	def _partition_model(self, model, sample, signatures):
		if self.partitioner:
			raise NotImplementedError(
				"Pipeline: tracing and graph partitioning are outside this build; pass partitioner=False and the stage modules of this rank"
			)
		parts = [model] if isinstance(model, torch.nn.Module) else list(model)
		if signatures is None:
			if self.rank == 0:
				logger.warning("No signatures provided, assuming sequential partitioning. If this is not what you want, please explicitly provide signatures when creating the pipeline.")
			signatures = sequential_signatures(self.placement)
		return parts, signatures

	def _create_pipeline(self, parts, signatures):
		ids = list(range(len(self.placement))) if self.all_ranks else self.placement.get_ids(self.rank)
		assert len(parts) == len(ids), f"rank {self.rank} owns blocks {ids} of placement {list(self.placement)} but got {len(parts)} stage module(s)"
		# under a memory budget the stages hold the lean stash: the remat ILP then starts from a third less per micro-batch
		lean = self.cfg.memory_budget is not None
		blocks = [(HipStageBlock if _is_transformer_chain(part) else AutogradStageBlock)(part, i, self.placement, signatures[i], mb_size=self.mb_size, lean_stash=lean) for part, i in zip(parts, ids)]
		if self.all_ranks:
			for b in blocks:
				b.local_ids = set(ids)  # peers on other ranks of the placement are in this process too
		return blocks
