"""TEST INFRASTRUCTURE - CPU restatement of the placement policy of the reference's
PinnedHostTensorPool (elf/execution/offload.py:14-158), on plain integers (no memory behind it).

Only tests/ may import this file.  Pins (tests/test_abi_cpu.py): hand-worked sequences from the
rules quoted below, the invariants "live blocks never overlap" and "freeing everything coalesces
each parent back to one (0, size) segment", and power-of-two parent sizes (offload.py:45-52).

Rules restated:
  _bucket_size (:45-52)      parent length = smallest power of two >= requested elements
  _first_fit   (:54-76)      parents of the dtype in creation order; inside a parent the free list
                             in offset order; first segment with length >= request; carve from
                             its start
  allocate     (:130-141)    request = max(1, elems); no fit -> new parent, carve from its start
  _insert_free (:102-128)    insert by offset, then merge every pair of adjacent segments
  free         (:143-153)    unknown blocks are ignored
  reserve      (:155-159)    new parent for ceil(bytes / itemsize) elements (rounded up to a power
                             of two like any other parent)
"""


class PoolModel:
	def __init__(self):
		self.parents = []  # {"dtype", "elems", "free": [(off, len), ...]}
		self.live = {}     # (parent, off) -> len

	@staticmethod
	def bucket(n):
		b = 1
		while b < n:
			b <<= 1
		return b

	def _new_parent(self, dtype, elems):
		self.parents.append({"dtype": dtype, "elems": self.bucket(elems), "free": [(0, self.bucket(elems))]})
		return len(self.parents) - 1

	def allocate(self, elems, dtype):
		req = max(1, int(elems))
		for pi, p in enumerate(self.parents):
			if p["dtype"] != dtype:
				continue
			for si, (off, ln) in enumerate(p["free"]):
				if ln >= req:
					return self._carve(pi, si, req)
		return self._carve(self._new_parent(dtype, req), 0, req)

	def _carve(self, pi, si, req):
		off, ln = self.parents[pi]["free"][si]
		if ln == req:
			del self.parents[pi]["free"][si]
		else:
			self.parents[pi]["free"][si] = (off + req, ln - req)
		self.live[(pi, off)] = req
		return pi, off

	def free(self, pi, off):
		ln = self.live.pop((pi, off), None)
		if ln is None:
			return False
		segs = self.parents[pi]["free"]
		at = next((i for i, (o, _) in enumerate(segs) if off < o), len(segs))
		segs.insert(at, (off, ln))
		merged = []
		for o, l in segs:
			if merged and merged[-1][0] + merged[-1][1] == o:
				merged[-1] = (merged[-1][0], merged[-1][1] + l)
			else:
				merged.append((o, l))
		self.parents[pi]["free"] = merged
		return True

	def reserve(self, nbytes, itemsize, dtype):
		self._new_parent(dtype, (int(nbytes) + itemsize - 1) // itemsize)

	def size_bytes(self, itemsizes):
		return sum(p["elems"] * itemsizes[p["dtype"]] for p in self.parents)
