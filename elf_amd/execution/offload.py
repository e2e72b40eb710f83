"""Activation offload handles and the pinned-host pool, as the engine sees them.

``StageOffloader`` has the life cycle of the reference's OffloadToCPU (elf/execution/offload.py:
166-411): used as a context manager around F (what F saved goes to pinned host memory on a side
stream when the context closes), ``prefetch()`` starts the copy back on another side stream,
``release()`` returns the pinned blocks.  The copies, streams, events and the arena live in
libelf_stage.so; this class only forwards to the stage that owns the micro-batch.

``PinnedHostTensorPool`` exposes the library's pinned arena, which follows the placement rules
of the reference pool (offload.py:14-158), for pre-reservation and for inspection.
"""

import ctypes

from .. import _lib

__all__ = ["StageOffloader", "PinnedHostTensorPool"]

_P, _I, _L = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
for _name, _ret, _args in [
	("elf_pinned_pool_create", _I, [_I, ctypes.POINTER(_P)]),
	("elf_pinned_pool_destroy", None, [_P]),
	("elf_pinned_pool_allocate", _I, [_P, _L, _I, _I, ctypes.POINTER(_P), ctypes.POINTER(_I), ctypes.POINTER(_L)]),
	("elf_pinned_pool_free", _I, [_P, _P]),
	("elf_pinned_pool_reserve", _I, [_P, _L, _I, _I]),
	("elf_pinned_pool_size", _L, [_P]),
	("elf_pinned_pool_n_parents", _I, [_P]),
	("elf_pinned_pool_n_free", _I, [_P, _I]),
	("elf_pinned_pool_free_segment", _I, [_P, _I, _I, ctypes.POINTER(_L), ctypes.POINTER(_L)]),
]:
	_lib.register(_name, _ret, _args)


class StageOffloader:
	"""Offload handle of one (stage, micro-batch)."""

	def __init__(self, block, mb_id, pool=None):
		self.block, self.mb_id, self.pool = block, mb_id, pool
		self.active = False

	def exclude(self, storages):
		"""Parameters are never part of the activation stash; nothing to record."""

	def __enter__(self):
		return self

	def __exit__(self, exc_type, exc, tb):
		if exc_type is None:
			self.block.offload(self.mb_id)
			self.active = True
		return False

	def prefetch(self):
		if self.active:
			self.block.prefetch(self.mb_id)

	def release(self):
		if self.active:
			self.block.release(self.mb_id)
			self.active = False


class PinnedHostTensorPool:
	"""First-fit pinned arena: per dtype, parent chunks of power-of-two length, allocation from
	the start of the first free segment that fits, coalescing on free.  ``host_backing=True``
	backs it with ordinary host memory (placement-rule tests on machines without a GPU)."""

	DTYPE_KEYS = {"f16": (0, 2), "bf16": (1, 2), "f32": (2, 4), "f64": (3, 8), "i8": (4, 1), "i16": (5, 2), "i32": (6, 4), "c64": (7, 8)}

	def __init__(self, host_backing=False):
		self.lib = _lib.load()
		h = _P()
		_lib.check(self.lib.elf_pinned_pool_create(int(host_backing), ctypes.byref(h)), "elf_pinned_pool_create")
		self._h = h

	def __del__(self):
		try:
			if self._h:
				self.lib.elf_pinned_pool_destroy(self._h)
				self._h = None
		except Exception:
			pass

	def allocate(self, required_elems, dtype="bf16"):
		"""Returns (address, parent index, offset in elements)."""
		key, size = self.DTYPE_KEYS[dtype]
		ptr, parent, off = _P(), _I(), _L()
		_lib.check(self.lib.elf_pinned_pool_allocate(self._h, int(required_elems), size, key, ctypes.byref(ptr), ctypes.byref(parent), ctypes.byref(off)), "elf_pinned_pool_allocate")
		return ptr.value, parent.value, off.value

	def free(self, address):
		"""Blocks that do not belong to the pool are ignored, as in the reference."""
		return self.lib.elf_pinned_pool_free(self._h, address) == 0

	def reserve(self, required_bytes, dtype="f32"):
		key, size = self.DTYPE_KEYS[dtype]
		_lib.check(self.lib.elf_pinned_pool_reserve(self._h, int(required_bytes), size, key), "elf_pinned_pool_reserve")

	def size(self):
		return self.lib.elf_pinned_pool_size(self._h)

	def free_segments(self):
		"""[[(offset, length), ...] per parent]"""
		out = []
		for p in range(self.lib.elf_pinned_pool_n_parents(self._h)):
			segs = []
			for i in range(self.lib.elf_pinned_pool_n_free(self._h, p)):
				off, ln = _L(), _L()
				_lib.check(self.lib.elf_pinned_pool_free_segment(self._h, p, i, ctypes.byref(off), ctypes.byref(ln)), "elf_pinned_pool_free_segment")
				segs.append((off.value, ln.value))
			out.append(segs)
		return out
