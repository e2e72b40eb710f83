"""Placement and timers (behaviour of the reference's elf/utils.py:50-147, 249-324)."""

import logging
import time

import torch
import torch.distributed as dist

logger = logging.getLogger("utils")

__all__ = ["Placement", "TensorMetadata", "Timer", "TimerCPU", "TimerGPU", "WIRE_DTYPES"]

# Position in this table = the dtype code on the wire (order of the reference's elf/utils.py:19-31).
WIRE_DTYPES = (
	torch.float16, torch.bfloat16, torch.float32, torch.float64, torch.int16, torch.int32, torch.int64,
	torch.complex32, torch.complex64, torch.complex128, torch.bool,
)


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


class TensorMetadata:
	"""What a stage tells its neighbour about a boundary tensor before the first payload: a header of
	MAX_SIZE fp32 values [dtype code, dim 0, dim 1, ..., 0 padding], the wire format of the reference's
	elf/utils.py:150-220 (sent by block.py:552-568, received by :536-548).  The shape is that of one
	sample (the sender describes ``value[0]``, block.py:577-584); ``get_buffer`` puts the batch
	dimension back.  As in the reference a zero ends the shape when the header is decoded, so a
	dimension of extent 0 (and everything after it) does not survive the round trip, and extents are
	carried as fp32 (exact up to 2**24).  On one GPU no header travels: the boundary buffers are local;
	the class is here so that a stage pair on two devices can speak the reference's format."""

	MAX_SIZE = 16

	def __init__(self, t):
		self.shape = list(t.shape)
		self.dtype = t.dtype
		self.device = torch.cuda.current_device() if torch.cuda.is_available() else "cpu"

	@staticmethod
	def from_tensor(t):
		"""Decode a received header."""
		assert t.dim() == 1, "Metadata should only have one dimension"
		fields = [int(v) for v in t.tolist()]
		meta = TensorMetadata(torch.empty(0, dtype=WIRE_DTYPES[fields[0]]))
		extents = fields[1:]
		meta.shape = extents[: extents.index(0)] if 0 in extents else extents
		return meta

	def to_tensor(self):
		"""Encode for sending.  More than MAX_SIZE - 1 dimensions do not fit (IndexError, as in the reference)."""
		if len(self.shape) > self.MAX_SIZE - 1:
			raise IndexError(f"TensorMetadata: {len(self.shape)} dimensions do not fit a header of {self.MAX_SIZE} values")
		header = [float(WIRE_DTYPES.index(self.dtype))] + [float(e) for e in self.shape]
		header += [0.0] * (self.MAX_SIZE - len(header))
		return torch.tensor(header, dtype=torch.float32, device=self.device)

	def get_buffer(self, batch_size):
		"""An uninitialised tensor for ``batch_size`` samples of this description."""
		return torch.empty((batch_size, *self.shape), dtype=self.dtype, device=self.device)

	def __repr__(self):
		return f"TensorMetadata({self.shape})"


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
