"""Plug-in registries (same keys and lookup behaviour as the reference's elf/registry.py:32-144):
``SCHEDULERS``, ``COMM_SCHEDULERS``, ``PARTITIONERS`` and ``TRACERS`` map names to callables.

  scheduler       (placement: list[int], n_micro_batches: int) -> list[Operation]  (for ALL ranks)
  comm scheduler  (list[Operation]) -> list[Operation]  (must keep each rank's compute order)
  partitioner     (fx.GraphModule, times, memories, n_parts) -> list[list[fx.Node]]
  tracer          (model, sample) -> fx.GraphModule
"""

__all__ = ["Registry", "SCHEDULERS", "PARTITIONERS", "TRACERS", "COMM_SCHEDULERS", "resolve"]


class Registry:
	"""Name -> object table; several names may point to one object."""

	def __init__(self, name):
		self._name = name
		self._values = {}
		self._descriptions = {}

	def register(self, key, obj, description=""):
		"""Register ``obj`` under one key or a list of keys; re-registering a key with another
		object is an error."""
		for k in ([key] if isinstance(key, str) else key):
			old = self._values.get(k)
			if old is not None and old is not obj:
				raise KeyError(f"{self._name!s} '{k}' already registered with a different object")
			self._values[k] = obj
			self._descriptions[k] = description
		return obj

	def _unknown(self, key):
		names = ", ".join(sorted(self._values)) or "<empty>"
		return KeyError(f"Unknown {self._name} '{key}'. Available {self._name}s: [{names}]")

	def get(self, key):
		if key not in self._values:
			raise self._unknown(key)
		return self._values[key]

	__getitem__ = get

	def get_key(self, obj):
		"""First key (registration order) bound to exactly this object."""
		for k, v in self._values.items():
			if v is obj:
				return k
		raise ValueError(f"Object {obj} not found in {self._name}")

	def get_description(self, key):
		if key not in self._descriptions:
			raise self._unknown(key)
		return self._descriptions[key]

	def available(self):
		"""Sorted keys, one per distinct object (aliases collapse onto their first sorted name)."""
		seen, keys = set(), []
		for k in sorted(self._values):
			if id(self._values[k]) not in seen:
				seen.add(id(self._values[k]))
				keys.append(k)
		return keys

	def __contains__(self, key):
		return key in self._values

	def __iter__(self):
		return iter(self._values)

	def __len__(self):
		return len(self._values)

	def __repr__(self):
		return f"<Registry[{self._name}] ({len(self)} items): {', '.join(sorted(self._values))}>"


SCHEDULERS = Registry("scheduler")
PARTITIONERS = Registry("partitioner")
TRACERS = Registry("tracer")
COMM_SCHEDULERS = Registry("comm_scheduler")


def resolve(var, registry):
	"""A callable is returned as is; a name is looked up; anything else is a ValueError that lists
	what is available."""
	if callable(var):
		return var
	if var in registry:
		return registry[var]
	lines = [f"Unknown {registry._name} '{var}'. Available ones:"]
	lines += [f"\t{name}: {registry.get_description(name)}" for name in registry.available()]
	raise ValueError("\n".join(lines) + "\n")
