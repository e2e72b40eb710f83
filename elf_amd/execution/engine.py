"""Per-rank interpreter of a schedule (the operation stream of the stages this process owns).

Same dispatch, statistics and slot hand-offs as the reference's Engine (elf/execution/engine.py:
96-371, compute_loss :374-410, same-rank transfers :413-445); the differences are that nothing
here needs a process group or a GPU to be importable, and that the offload handles come from the
block when it brings its own (``HipStageBlock`` -> ``StageOffloader``).
"""

import contextlib
import logging
import os
import time
from collections import OrderedDict, deque

import torch
import torch.distributed as dist

from ..scheduling import OperationType, OpOptions
from ..utils import Timer
from .offload import StageOffloader

logger = logging.getLogger("engine")

# read once at import, any non-empty value switches them on (as in the reference)
precise_timings = os.environ.get("ELF_TIMINGS", False)
precise_memory = os.environ.get("ELF_MEMORY", False)

__all__ = ["Engine", "GraphedStep", "compute_loss", "preallocate_pool"]

_GPU = torch.cuda.is_available


def _fake_p2p(data):
	"""A (work, tensor) pair with no pending work: how locally produced data enters a slot."""
	return [None, data.detach()]


def _capturing():
	return _GPU() and torch.cuda.is_current_stream_capturing()


def _sync():
	if _GPU() and not _capturing():
		torch.cuda.synchronize()


def _mem():
	return (torch.cuda.memory_allocated(), torch.cuda.max_memory_allocated()) if _GPU() else (0, 0)


def preallocate_pool(blocks):
	"""``ELF_PREALLOCATE_POOL="bf16:8,f32:1"`` (GiB per dtype, elf/execution/engine.py:71-93) grows the
	pinned-host memory of activation offload before the first step.  The reference has one pool per
	process keyed by dtype; here every stage owns one arena that holds its stash as raw bf16-sized
	elements, so the sizes of all dtypes are added up and shared evenly among the blocks that can offload.
	Returns the bytes reserved per block (0 when the variable is not set)."""
	val = os.environ.get("ELF_PREALLOCATE_POOL")
	if not val:
		return 0
	known = {"f16", "f32", "f64", "bf16", "i8", "i16", "i32", "c64"}
	total = 0
	for part in val.split(","):
		dtype, size = part.split(":")
		if dtype not in known:
			raise KeyError(dtype)
		total += int(size) * 1024**3
	able = [b for b in blocks if hasattr(b, "reserve_pinned")]
	if not able or total <= 0:
		return 0
	share = total // len(able)
	for b in able:
		b.reserve_pinned(share)
	return share


class Engine:
	"""Runs a list of operations on the blocks of one rank; feeds the pipeline input to the first
	block and computes the loss on the last one."""

	def __init__(self, blocks, all_ranks=False):
		"""``all_ranks``: the blocks belong to several ranks of the placement that this one process plays
		(``Pipeline(all_ranks=True)``); the schedule must then come in an order one process can run."""
		self.blocks = blocks
		self.rank = blocks[0].rank if blocks else None
		for b in blocks:
			assert all_ranks or b.rank == self.rank, "All blocks in a stage should be on the same rank"
		self.id_to_block = {b.id: b for b in blocks}
		self.offload_stream = torch.cuda.Stream() if _GPU() else None
		self.pool = None  # the pinned arena lives in the stage library
		preallocate_pool(blocks)

	def _offloader(self, block, mb):
		if hasattr(block, "offload"):
			return StageOffloader(block, mb, self.pool)
		raise NotImplementedError(f"{block}: this block type has no activation offload")

	def train_step(self, batch, target, loss_fn, schedule, mb_sizes, profile=False):
		"""Execute ``schedule`` (ops of other ranks are skipped).

		Returns (result, losses, stats, detailed_stats): ``result`` = per-micro-batch outputs of the
		last block, ``stats`` = {total, idle, start_idle, end_idle, bubble} in seconds (meaningful
		with ELF_TIMINGS), ``detailed_stats`` = {"all_events": {timer name: s}, "memories":
		{str(op): bytes allocated after it}, "peak_memory": {str(op): peak bytes}}; with a
		HipStageBlock the byte counts include the library's own stash."""
		if batch is not None:
			microbatches = iter(zip(*[t.split(mb_sizes, dim=0) for t in batch]))
		if target is not None:
			microtargets = target.split(mb_sizes, dim=0)

		offloaders = {}

		def offloader(block, mb):
			key = (block.id, mb)
			if key not in offloaders:
				offloaders[key] = self._offloader(block, mb)
			return offloaders[key]

		# The step's last W of a block that can fold the gradient scale into it (HipStageBlock): that W is told the scale
		# the ALL_REDUCE_PARAM_GRADS op behind it will apply (block.scale_grads then skips what the W has already done).
		final_w = {}
		for i, op in enumerate(schedule):
			blk = self.id_to_block.get(op.block_id)
			if blk is None or not getattr(blk, "folds_grad_scale", False):
				continue
			if op.op == OperationType.BACKWARD_PARAMS:
				final_w[op.block_id] = [i, False]
			elif op.op == OperationType.ALL_REDUCE_PARAM_GRADS and op.block_id in final_w:
				final_w[op.block_id][1] = True
			elif op.op == OperationType.ALL_REDUCE_PARAM_GRADS:
				final_w[op.block_id] = [-1, False]
		final_w = {i for i, scaled in final_w.values() if scaled and i >= 0}
		final_scale = 1.0 / float(sum(mb_sizes))

		result, losses, grad_fns = [], [], deque()
		if precise_timings:
			if dist.is_available() and dist.is_initialized():
				dist.barrier()
			_sync()
			t_sync = time.time()
		pipe_start = time.time()
		warmup_time = None
		memories, peak_memories = OrderedDict(), OrderedDict()
		T = OperationType

		for op_index, op in enumerate(schedule):
			block = self.id_to_block.get(op.block_id)
			if block is None:
				continue
			if profile and _GPU():
				torch.cuda.nvtx.range_push(f"{block}:{op}")
			if precise_memory and _GPU():
				torch.cuda.reset_peak_memory_stats()
				if hasattr(block, "reset_peak"):
					block.reset_peak()
			if warmup_time is None and op.op != T.RECV_FORWARD:
				warmup_time = 0
				if precise_timings:
					_sync()
					warmup_time = time.time() - t_sync

			kind = op.op
			if kind == T.FORWARD:
				ctx = offloader(block, op.mb_id) if op.options.get(OpOptions.ACTIVATION_OFFLOAD) else contextlib.nullcontext()
				with ctx:
					y = block.forward(op.mb_id, **op.options)
				if y is not None:
					for out in y:
						result.append(out.detach() if isinstance(out, torch.Tensor) else out)
			elif kind == T.BACKWARD_INPUTS:
				block.backward_inputs(op.mb_id, **op.options)
				if op.options.get(OpOptions.ACTIVATION_OFFLOAD):
					offloader(block, op.mb_id).release()
			elif kind == T.BACKWARD_PARAMS:
				if op_index in final_w:
					block.backward_params(op.mb_id, final_scale=final_scale, **op.options)
				else:
					block.backward_params(op.mb_id, **op.options)
			elif kind == T.SEND_FORWARD:
				dst = self.id_to_block.get(op.options.get("dst"))
				if dst is not None:
					_transfer_forward(block, dst, op.mb_id)
				block.send_forward(op.mb_id, **op.options)
			elif kind == T.SEND_BACKWARD:
				dst = self.id_to_block.get(op.options.get("dst"))
				if dst is not None:
					_transfer_backward(block, dst, op.mb_id)
				block.send_backward(op.mb_id, **op.options)
			elif kind == T.RECV_FORWARD:
				if block.is_first:
					for mb, var in zip(next(microbatches), block.input_variables):
						var.set(var.to_process, op.mb_id, _fake_p2p(mb))
				block.recv_forward(op.mb_id, mb_sizes[op.mb_id], **op.options)
			elif kind == T.RECV_BACKWARD:
				block.recv_backward(op.mb_id, mb_sizes[op.mb_id], **op.options)
			elif kind == T.LOSS_FORWARD:
				if not block.is_last:
					logger.warning(f"Tried to compute loss on a non-last block {block}")
					continue
				assert op.mb_id < len(result), f"Loss forward for mb {op.mb_id} but only {len(result)} results computed"
				loss, grad_fn = compute_loss(block, result[op.mb_id], microtargets[op.mb_id], loss_fn)
				losses.append(loss)
				grad_fns.append(grad_fn)
			elif kind == T.LOSS_BACKWARD:
				if not block.is_last:
					logger.warning(f"Tried to compute loss backward on a non-last block {block}")
					continue
				assert op.mb_id < len(losses), f"Loss backward for mb {op.mb_id} but only {len(losses)} losses computed"
				with Timer(name=f"backward({block.id}:{op.mb_id})") as timer:
					grads = grad_fns.popleft()()
				block.compute_time.append(timer)
				if self.offload_stream is not None and not _capturing():  # a captured step keeps its outputs on the GPU
					self.offload_stream.wait_stream(torch.cuda.current_stream())
					with torch.cuda.stream(self.offload_stream), torch.no_grad():
						result[op.mb_id] = result[op.mb_id].to("cpu", non_blocking=True)
				for grad, var in zip(grads, block.output_variables):
					for dst in var:
						dst.set(dst.to_process, op.mb_id, _fake_p2p(grad))
			elif kind == T.RECOMPUTE_FORWARD:
				block.recompute_forward(op.mb_id, **op.options)
			elif kind == T.RECOMPUTE_BACKWARD_INPUTS:
				block.recompute_backward_inputs(op.mb_id, **op.options)
			elif kind == T.PREFETCH_ACTIVATIONS:
				offloader(block, op.mb_id).prefetch()
			elif kind == T.ALL_REDUCE_PARAM_GRADS:
				block.scale_grads(sum(mb_sizes))
				block.all_reduce_param_grads(**op.options)
			else:
				raise Exception(f"Unknown operation : {op}")

			if precise_memory:
				_sync()
			alloc, peak = _mem()
			if hasattr(block, "mem_stats"):
				st = block.mem_stats()
				alloc, peak = alloc + st["live_bytes"], peak + st["peak_bytes"]
			memories[str(op)] = alloc
			peak_memories[str(op)] = peak
			if profile and _GPU():
				torch.cuda.nvtx.range_pop()

		if precise_timings:
			_sync()
		cooldown_start = time.time()
		if precise_timings:
			_sync()
		pipe_end = time.time()

		compute_time, all_events = 0, {}
		if precise_timings:
			for block in self.blocks:
				compute_time += sum(t.time() for t in block.compute_time)
				all_events.update({t.name: t.time() for t in block.compute_time})
		stats = {
			"total": pipe_end - pipe_start,
			"idle": pipe_end - pipe_start - compute_time,
			"start_idle": warmup_time,
			"end_idle": pipe_end - cooldown_start,
		}
		stats["bubble"] = stats["idle"] - (stats["start_idle"] or 0) - stats["end_idle"]
		detailed_stats = {"all_events": all_events, "memories": memories, "peak_memory": peak_memories}
		for block in self.blocks:
			block.compute_time.clear()
		if self.offload_stream is not None and not _capturing():
			torch.cuda.current_stream().wait_stream(self.offload_stream)
		for off in offloaders.values():
			off.release()
		return result, losses, stats, detailed_stats

	def capture(self, batch, target, loss_fn, schedule, mb_sizes, warmup=1):
		"""Record one ``train_step`` as a HIP graph and return a ``GraphedStep`` that replays it.

		A stage step is a fixed sequence of kernel launches (hundreds to thousands per step: one op is
		40-50 launches); replaying it as a graph takes the Python interpreter, the slot bookkeeping
		and the per-launch driver work out of the step.  The reference has no counterpart (its ops
		build autograd graphs on the fly).  Conditions: the schedule must not offload activations
		(copies to pinned memory on side streams stay eager), and between replays nothing else may
		run stage ops of these blocks.  ``warmup`` eager steps run first so that every pool and
		workspace has its final size (nothing may allocate device memory while capturing); the
		gradient accumulators are put back as they were, so the capture itself adds no gradient.
		"""
		for op in schedule:
			if op.op == OperationType.PREFETCH_ACTIVATIONS or op.options.get(OpOptions.ACTIVATION_OFFLOAD):
				raise NotImplementedError("Engine.capture: schedules with activation offload are not captured")
		static_batch = None if batch is None else [t.clone() for t in batch]
		static_target = None if target is None else target.clone()
		kept = [[g.clone() for g in getattr(b, "_fused_g", [])] for b in self.blocks]
		side = torch.cuda.Stream()
		side.wait_stream(torch.cuda.current_stream())
		with torch.cuda.stream(side):
			for _ in range(max(1, warmup)):
				self.train_step(static_batch, static_target, loss_fn, schedule, mb_sizes)
				self._reset_slots()
		torch.cuda.current_stream().wait_stream(side)
		torch.cuda.synchronize()
		for b, gs in zip(self.blocks, kept):
			for g, keep in zip(getattr(b, "_fused_g", []), gs):
				g.copy_(keep)
		graph = torch.cuda.CUDAGraph()
		with torch.cuda.graph(graph):
			result, losses, _, _ = self.train_step(static_batch, static_target, loss_fn, schedule, mb_sizes)
		self._reset_slots()
		return GraphedStep(graph, static_batch, static_target, result, losses)

	def _reset_slots(self):
		"""Empty the per-micro-batch slot lists of every block (what Pipeline.step does after a step)."""
		for block in self.blocks:
			block._wait_for_send_ops()
			for var in block.input_variables:
				var.clear()
			for var in block.output_variables:
				for dst in var:
					dst.clear()


class GraphedStep:
	"""A captured ``Engine.train_step``.  ``replay(batch, target)`` copies the new data into the
	buffers the graph reads, launches the graph and returns ``(result, losses)``: the same GPU tensors
	every time (an eager step moves its outputs to the host), overwritten by each replay.  Weight gradients accumulate into the blocks' ``main_grad``
	buffers exactly as in an eager step (zero them between steps as usual)."""

	def __init__(self, graph, batch, target, result, losses):
		self.graph, self.batch, self.target, self.result, self.losses = graph, batch, target, result, losses

	def replay(self, batch=None, target=None):
		if batch is not None:
			for dst, src in zip(self.batch, [batch] if isinstance(batch, torch.Tensor) else batch):
				dst.copy_(src)
		if target is not None:
			self.target.copy_(target)
		self.graph.replay()
		return self.result, self.losses


def compute_loss(block, output, target, loss_fn):
	"""Loss of one micro-batch, summed over its samples and divided by the elements per sample
	(the division by the batch size happens with the gradient scale at the end of the step), and
	the closure that back-propagates it to the block output."""
	if not isinstance(output, torch.Tensor) or not isinstance(target, torch.Tensor):
		logger.warning("Loss computation with non-tensor output or target")
	elems = target.numel() // target.size(0)
	fused = getattr(loss_fn, "loss_and_grad", None)
	if fused is not None:
		# loss and gradient from one kernel (elf_amd.losses): nothing for autograd to record
		with Timer(name="loss_forward") as timer:
			loss, grad = fused(output.detach(), target, reduction="sum", scale=1.0 / elems)
		block.compute_time.append(timer)
		return (loss / elems).detach(), lambda: (grad,)
	output = output.detach().requires_grad_()
	with Timer(name="loss_forward") as timer:
		try:
			loss = loss_fn(output, target, reduction="sum")
		except TypeError:
			loss = loss_fn(output, target)
	block.compute_time.append(timer)
	loss = loss / elems

	def grad_fn():
		loss.backward()
		return (output.grad.data,)

	return loss.detach().requires_grad_(False), grad_fn


def _transfer_forward(block, dst_block, mb_id):
	"""Same-rank hand-off of activations: outputs of ``block`` bound for ``dst_block`` become its
	pending inputs (matched by position)."""
	outgoing = [d for var in block.output_variables for d in var if d.peer == dst_block.id]
	incoming = [v for v in dst_block.input_variables if v.peer == block.id]
	for src, dst in zip(outgoing, incoming):
		dst.set(dst.to_process, mb_id, _fake_p2p(src.get(src.to_send, mb_id)))


def _transfer_backward(block, dst_block, mb_id):
	"""Same-rank hand-off of input gradients to the block that produced those inputs."""
	outgoing = [v for v in block.input_variables if v.peer == dst_block.id]
	incoming = [s for var in dst_block.output_variables for s in var if s.peer == block.id]
	for src, dst in zip(outgoing, incoming):
		dst.set(dst.to_process, mb_id, _fake_p2p(src.get(src.to_send, mb_id)))
