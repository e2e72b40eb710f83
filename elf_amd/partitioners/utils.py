"""Stage signatures (who feeds a block, who consumes its outputs); behaviour of the reference's
elf/partitioners/utils.py:17-146."""

__all__ = ["Signature", "sequential_signatures", "signatures_from_sources_targets", "get_sources_targets_sequential"]


def _unique(seq):
	seen = set()
	return [x for x in seq if not (x in seen or seen.add(x))]


class Signature:
	"""inputs / outputs are variable names; sources[i] is the block producing inputs[i] (None =
	pipeline input); targets[i] is the list of blocks consuming outputs[i] (None = pipeline output)."""

	def __init__(self, inputs, outputs, sources, targets):
		assert len(sources) == len(inputs)
		assert len(targets) == len(outputs)
		self.inputs, self.outputs = inputs, outputs
		self.ninputs, self.noutputs = len(inputs), len(outputs)
		self.sources, self.targets = sources, targets

	def get_all_sources(self):
		return _unique(self.sources)

	def get_all_targets(self):
		return _unique(t for tgt in self.targets for t in tgt)

	def __str__(self):
		ins = ", ".join(f"{i} ({s})" for i, s in zip(self.inputs, self.sources))
		outs = ", ".join(f"{o} ({t})" for o, t in zip(self.outputs, self.targets))
		return f"Signature({ins}) -> ({outs})"

	__repr__ = __str__


def signatures_from_sources_targets(sources, targets):
	assert len(sources) == len(targets), "Sources and targets must have the same length"
	sigs = []
	for i in range(len(sources)):
		ins, outs = sorted(sources[i]), sorted(targets[i])
		sigs.append(Signature(ins, outs, [sources[i][k] for k in ins], [targets[i][k] for k in outs]))
	return sigs


def get_sources_targets_sequential(placement):
	"""One input ("input", from the previous block) and one output ("output", to the next block)
	per stage; the ends of the chain use None."""
	n = len(placement)
	sources = {i: {"input": i - 1 if i else None} for i in range(n)}
	targets = {i: {"output": [i + 1 if i != n - 1 else None]} for i in range(n)}
	return sources, targets


def sequential_signatures(placement):
	return signatures_from_sources_targets(*get_sources_targets_sequential(placement))
