"""Writes tests/golden/schedule_vectors.json: op lists produced by the REFERENCE's pure-host
scheduling functions that none of the reference's own tests pins bit-exactly
(pipelined / simulation / topo comm schedulers, ZB-H1/H2, Hanayo, ZB-V, interleaved 1F1B op
lists, RematScheduler and get_offloaded_scheduler / get_checkpointed_scheduler rewrites).

Run once in the build container (the reference lives at /root/reference there and never travels):
    python tests/golden/make_schedule_vectors.py
The reference needs enum.StrEnum (Python >= 3.11); on 3.10 a three-line backport is put into the
``enum`` module before the import - nothing in the reference tree is modified.
"""

import enum
import json
import os
import sys

REF = "/root/reference"

if not hasattr(enum, "StrEnum"):

	class StrEnum(str, enum.Enum):
		def _generate_next_value_(name, start, count, last_values):
			return name.lower()

		__str__ = str.__str__
		__format__ = str.__format__

	enum.StrEnum = StrEnum

sys.path.insert(0, REF)
sys.path.insert(0, os.path.join(REF, "benchmarks"))

from elf.registry import SCHEDULERS, COMM_SCHEDULERS  # noqa: E402
from elf.scheduling import add_comms  # noqa: E402
from elf.scheduling.ilp import RematScheduler  # noqa: E402
from elf.partitioners.utils import sequential_signatures  # noqa: E402


def probes():
	"""(label, module name, module) triples a remat strategy is evaluated on: the stage root, a
	sub-module name without a module, and one instance of each module class the benchmark's
	strategies look at (plus a Linear, which none of them selects)."""
	import torch.nn as nn
	from models.simple import Attention, FastAttention

	return [
		("root", "", None), ("x", "x", None), ("gelu", "mlp.activation", nn.GELU()), ("layernorm", "norm1", nn.LayerNorm(4)),
		("dropout", "dropout", nn.Dropout()), ("linear", "proj", nn.Linear(2, 2)), ("attention", "attn.attn", Attention(8)),
		("fastattention", "attn.attn", FastAttention(8)),
	]


PROBES = None


def enc(op):
	"""[OperationType value, block, mb, rank(, {option: value})]; a callable option value (a remat
	strategy) is replaced by "fn:" + the labels of the probes it selects, e.g. "fn:root"."""
	global PROBES
	opts = {}
	for k, v in op.options.items():
		k = str(k.value) if hasattr(k, "value") else str(k)
		if callable(v):
			PROBES = PROBES or probes()
			v = "fn:" + ",".join(label for label, name, module in PROBES if v(name, module))
		opts[k] = v
	rec = [op.op.value, op.block_id, op.mb_id, op.rank]
	return rec + [opts] if opts else rec


cases = []


def add(name, ops, **meta):
	cases.append({"name": name, **meta, "ops": [enc(o) for o in ops]})


# raw generators
for sched, placement, nmb in [
	("1f1b", [0, 1, 2, 3], 8), ("1f1b", [0, 1, 2, 3, 0, 1, 2, 3], 8), ("1f1b", [0, 1, 2, 3], 3), ("zbh1", [0, 1, 2, 3], 16),
	("zbh1", [0, 1], 4), ("zbh2", [0, 1, 2, 3], 8), ("zbh2", [0, 1], 2), ("hanayo", [0, 1, 2, 3, 3, 2, 1, 0], 4),
	("zbv", [0, 1, 2, 3, 3, 2, 1, 0], 8), ("full_remat", [0, 1, 2], 2), ("inference", [0, 1, 2], 2), ("afab", [0, 1, 0, 1], 2),
]:
	add(f"gen:{sched}", SCHEDULERS[sched](placement, nmb), scheduler=sched, placement=placement, nmb=nmb)

# add_comms + comm schedulers
for sched, placement, nmb, comm in [
	("1f1b", [0, 1], 8, "pipelined"), ("1f1b", [0, 1, 2, 3], 8, "pipelined"), ("zbh1", [0, 1, 2, 3], 16, "pipelined"),
	("1f1b", [0, 1, 2, 3], 4, "simulation"), ("1f1b", [0, 1, 2, 3], 4, "topo"), ("zbh1", [0, 1], 4, "simulation"),
	("zbh2", [0, 1, 2, 3], 4, "pipelined"), ("afab", [0, 1, 2], 2, "topo"), ("1f1b", [0, 1, 0, 1], 4, "pipelined"),
]:
	s = add_comms(SCHEDULERS[sched](placement, nmb), sequential_signatures(placement))
	add(f"comm:{sched}:{comm}", COMM_SCHEDULERS[comm](s), scheduler=sched, placement=placement, nmb=nmb, comm=comm)

# RematScheduler rewrites
nmb, placement = 4, [0, 1]
solution = {
	"full_fwd": [[1.0, 0.0, 0.0, 1.0], [0.0, 0.0, 0.0, 0.0]],
	"activations_bwd": [[0.0, 1.0, 0.0, 0.0], [0.0, 0.0, 1.0, 0.0]],
	"full_bwd": [[0.0, 0.0, 1.0, 0.0], [1.0, 0.0, 0.0, 0.0]],
}
for sched in ("1f1b", "zbh1"):
	add(f"remat:{sched}", RematScheduler(SCHEDULERS[sched], solution)(placement, nmb), scheduler=sched, placement=placement, nmb=nmb, solution=solution)
	s = add_comms(RematScheduler(SCHEDULERS[sched], solution)(placement, nmb), sequential_signatures(placement))
	add(f"remat+comm:{sched}", COMM_SCHEDULERS["pipelined"](s), scheduler=sched, placement=placement, nmb=nmb, solution=solution, comm="pipelined")

# benchmark-side wrappers that define the offload / checkpoint sets
from benchmark_utils import get_offloaded_scheduler, get_checkpointed_scheduler  # noqa: E402

for sched, placement, nmb, ratio, pt in [("1f1b", [0, 1, 2, 3], 8, 1, 1), ("1f1b", [0, 1, 2, 3], 8, 2, 2), ("afab", [0, 1], 3, 1, 1), ("1f1b", [0, 1], 4, 1, 3), ("zbh1", [0, 1, 2, 3], 8, 3, 1)]:
	add(f"offload:{sched}", get_offloaded_scheduler(sched, ratio, pt)(placement, nmb), scheduler=sched, placement=placement, nmb=nmb, ratio=ratio, prefetching_time=pt)
s = add_comms(get_offloaded_scheduler("1f1b", 1, 1)([0, 1, 2, 3], 8), sequential_signatures([0, 1, 2, 3]))
add("offload+comm:1f1b", COMM_SCHEDULERS["pipelined"](s), scheduler="1f1b", placement=[0, 1, 2, 3], nmb=8, ratio=1, prefetching_time=1, comm="pipelined")
for kind in ("full", "simple", "selective"):
	add(f"ckpt:{kind}", get_checkpointed_scheduler("1f1b", kind)([0, 1], 2), scheduler="1f1b", placement=[0, 1], nmb=2, type=kind)

out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "schedule_vectors.json")
with open(out, "w") as f:
	json.dump(cases, f, separators=(",", ":"))
print(f"wrote {len(cases)} cases, {sum(len(c['ops']) for c in cases)} ops -> {out} ({os.path.getsize(out)} bytes)")
