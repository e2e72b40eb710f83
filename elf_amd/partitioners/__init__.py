"""Partitioning plug points.  Only what the stage execution path needs is provided:
``Signature`` / ``sequential_signatures`` for pre-partitioned models (``partitioner=False``).
The graph-partitioning algorithms of the reference (elf/partitioners/*.py) are a one-off set-up
step outside this path; their registry keys exist and raise when called."""

from ..registry import PARTITIONERS, TRACERS
from .utils import Signature, sequential_signatures, signatures_from_sources_targets, get_sources_targets_sequential


def _not_built(kind, name):
	def stub(*_args, **_kwargs):
		raise NotImplementedError(
			f"{kind} '{name}' is not part of this build: pass pre-partitioned stage modules with partitioner=False"
		)

	stub.__name__ = f"{kind}_{name}"
	return stub


for _name in ("naive", "constrained", "metis", "dagP"):
	PARTITIONERS.register(_name, _not_built("partitioner", _name), "not built: use partitioner=False")
for _name in ("default", "fx", "fx_safe", "export"):
	TRACERS.register(_name, _not_built("tracer", _name), "not built: use partitioner=False")

__all__ = ["Signature", "sequential_signatures", "signatures_from_sources_targets", "get_sources_targets_sequential"]
