"""Placement and timers (behaviour of the reference's elf/utils.py:50-147, 249-324)."""

import logging
import time

import torch
import torch.distributed as dist

logger = logging.getLogger("utils")

__all__ = ["Placement", "Timer", "TimerCPU", "TimerGPU"]


class Placement(list):
	"""placement[block] = rank hosting that pipeline stage, e.g. linear [0,1,2,3], interleaved
	[0,1,2,3,0,1,2,3], V-shaped [0,1,2,3,3,2,1,0]."""

	def __init__(self, placement):
		super().__init__(placement)
		assert not dist.is_initialized() or max(self) < dist.get_world_size(), "Placement is out of bounds"

	def get_ids(self, rank):
		return [i for i, r in enumerate(self) if r == rank]

	@staticmethod
	def default(scheduler, pp):
		"""hanayo / zbv -> V shape, megatron -> two interleaved rounds, anything else -> linear.
		A scheduler object (instead of its name) gets the linear placement."""
		if callable(scheduler):
			logger.warning("Placement.default() expects a scheduler name, not the scheduler object itself. Using the default placement.")
			scheduler = ""
		ranks = list(range(pp))
		if scheduler in ("hanayo", "zbv"):
			return Placement(ranks + ranks[::-1])
		if scheduler == "megatron":
			return Placement(ranks * 2)
		return Placement(ranks)

	def head(self):
		return self[0]

	def tail(self):
		return self[-1]

	def add_offset(self, offset):
		return Placement([r + offset for r in self])

	def is_head(self, rank):
		return rank == self[0]

	def is_tail(self, rank):
		return rank == self[-1]


class TimerCPU:
	def __init__(self, name="unknown"):
		self.name = name

	def __enter__(self):
		self.start = time.perf_counter()
		return self

	def __exit__(self, *_):
		self.end = time.perf_counter()

	def time(self):
		"""Elapsed seconds."""
		return self.end - self.start


class TimerGPU:
	"""Event pair on the current stream; ``time()`` waits for the closing event."""

	def __init__(self, name="unknown"):
		self.name = name
		self.start_event = torch.cuda.Event(enable_timing=True)
		self.end_event = torch.cuda.Event(enable_timing=True)

	def __enter__(self):
		# timing events cannot be recorded into a stream capture: a step being captured as a graph is
		# not timed (time() gives 0)
		self.recorded = not torch.cuda.is_current_stream_capturing()
		if self.recorded:
			self.start_event.record()
		return self

	def __exit__(self, *_):
		if self.recorded:
			self.end_event.record()

	def time(self):
		if not self.recorded:
			return 0.0
		self.end_event.synchronize()
		return self.start_event.elapsed_time(self.end_event) / 1000


class Timer:
	"""``with Timer(name=...) as t: ...; t.time()`` - GPU events when a GPU is present (or
	type="gpu"/"cuda"), wall clock otherwise (or type="cpu")."""

	def __new__(cls, type=None, name=None, *, type_=None, name_=None):
		kind, label = type or type_, name or name_
		if kind:
			if kind.lower() in ("gpu", "cuda"):
				return TimerGPU(label)
			if kind.lower() == "cpu":
				return TimerCPU(label)
		return TimerGPU(label) if torch.cuda.is_available() else TimerCPU(label)
