"""Rematerialisation under a memory budget: the ILP over per-(stage, micro-batch) remat choices,
the schedule rewrite that applies a solution, and the profiling record that feeds the ILP.

The model is the one the reference builds in elf/scheduling/ilp.py:440-747 (parameters
:440-485, variables and helpers :540-610, constraints :643-679, solution dict :709-742), and
``RematScheduler`` performs the op-list rewrite of :753-825.  The reference states the model with
PuLP and hands it to CBC / CPLEX (neither ships with it); here the same rows are assembled as
sparse matrices and solved with scipy.optimize.milp (HiGHS) under the same limits (60 s, 3 %
relative gap).  Solutions of an ILP solved to a gap are not unique, so parity of decisions is
defined on the model: same feasible set, objective within the gap (tests brute-force small cases).

Units: times in ms, memory in MiB (``memory_budget`` is what the reference calls MB).
"""

import logging
import time

import numpy as np

from ..registry import SCHEDULERS, resolve
from .scheduling import Operation, OperationType, OpOptions

logger = logging.getLogger("ilp")

__all__ = ["build_ilp_params", "solve_remat", "solve_remat_best", "evaluate_remat", "RematScheduler", "stagerematify", "AutoScheduler", "RematOption", "profile_stage"]

_OPS = ("f", "b", "w")
_KIND = {OperationType.FORWARD: "f", OperationType.BACKWARD_INPUTS: "b", OperationType.BACKWARD_PARAMS: "w"}


class RematOption:
	def __init__(self, name, type, mem_freed, time_overhead):
		self.name, self.type, self.mem_freed, self.time_overhead = name, type, mem_freed, time_overhead

	def __repr__(self):
		return f"RematOption({self.name!r}, {self.type!r}, mem_freed={self.mem_freed}, time_overhead={self.time_overhead})"


def profile_stage(stage, sample_metadata=None, n_iter=10):
	"""Profiling record of one stage for the ILP, measured on the native executor
	(elf/scheduling/ilp.py:50-126 ``_measure_full_pass``, :224-254 ``profile_stage``).

	``stage`` is a ``HipStageBlock``.  One warm-up pass, then ``n_iter`` passes of F, B, W on a
	reserved micro-batch slot with N(0,1) boundary tensors; medians are reported:

	T[f|b|w]      ms, event pairs on the launch stream
	M[f|b|w]      MiB still held after the op, relative to before F (after F: output + stash;
	              after B: the W stash; after W: 0)
	Mpeak[f|b|w]  MiB high-water mark during the op (relative to before F for f, to before the op
	              for b and w, as in the reference)
	Mpeak_ckpt    the same for a forward that keeps nothing (whole-stage checkpoint)
	Mba / Mbg     the two halves of the W stash after B: layer inputs / output gradients
	Minput, Moutput  boundary tensor sizes;  Tcomm 0 (no transfers on one GPU)
	Mparams       MiB of the bf16 weights x 1.5, plus half of Mworkspace: the ILP charges 2 x Mparams per
	              stage for weights + gradients, this executor keeps bf16 weights plus fp32 accumulators
	              (6 B/param), and the stage's fixed scratch is resident like they are
	Mworkspace    MiB of fixed device scratch the stage allocated at creation (attention backward
	              partials, norm backward partials, rope table)

	Memory = bytes held by the stage library (stash + temporaries) + torch's allocator (boundary
	tensors).  Returns ``(stats, next_stage_input)`` like the reference (warm-up output on the CPU).
	"""
	import ctypes

	import torch

	from .. import _lib
	from ..execution.block import BWD_RECOMPUTE_GRADIENTS, FWD_REMAT_ROOT

	block, lib = stage, stage.lib
	h = block._handle
	mb = 1 << 20  # a slot no schedule uses
	stream = torch.cuda.current_stream().cuda_stream
	MiB = 1024.0 * 1024.0
	# a first stage reads token ids and sends no input gradient; a last stage writes logits (rows padded
	# to vld columns) and reads their gradient in the same layout
	vin, vout = getattr(block, "vocab_in", 0), getattr(block, "vocab_out", 0)
	if vin:
		x = torch.randint(0, vin, (block.T,), device="cuda")
	else:
		x = torch.randn(block.T, block.d, device="cuda").to(torch.bfloat16)
	out_cols = block.vld if vout else block.d
	dy = torch.randn(block.T, out_cols, device="cuda").to(torch.bfloat16)
	if vout:
		dy[:, vout:] = 0
	new_y = lambda: torch.empty(block.T, out_cols, dtype=torch.bfloat16, device="cuda")
	new_dx = lambda: None if vin else torch.empty_like(x)

	def held():
		return torch.cuda.memory_allocated() + block.mem_stats()["live_bytes"]

	def peak():
		return torch.cuda.max_memory_allocated() + block.mem_stats()["peak_bytes"]

	def reset():
		torch.cuda.reset_peak_memory_stats()
		block.reset_peak()

	def timed(fn):
		e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
		e0.record()
		fn()
		e1.record()
		e1.synchronize()
		return e0.elapsed_time(e1)

	def fwd(y, flags=0):
		_lib.check(lib.elf_stage_forward(h, mb, x.data_ptr(), y.data_ptr(), flags, stream), "elf_stage_forward")

	def bwd(dx, flags=0):
		_lib.check(lib.elf_stage_backward_inputs(h, mb, x.data_ptr(), dy.data_ptr(), dx.data_ptr() if dx is not None else None, flags, stream), "elf_stage_backward_inputs")

	def wgrad():
		_lib.check(lib.elf_stage_backward_params(h, mb, stream), "elf_stage_backward_params")

	saved_grads = [g.clone() for g in block._fused_g]  # the passes below accumulate into main_grad
	y = new_y()
	fwd(y)
	warmup_output = (y[:, :vout] if vout else y).detach().cpu()
	dx = new_dx()
	bwd(dx)
	wgrad()
	del y, dx
	torch.cuda.synchronize()

	times, mems, peaks = ({k: [] for k in _OPS} for _ in range(3))
	for _ in range(n_iter):
		reset()
		start = held()
		y = new_y()
		times["f"].append(timed(lambda: fwd(y)))
		mems["f"].append((held() - start) / MiB)
		peaks["f"].append((peak() - start) / MiB)
		reset()
		before = held()
		dx = new_dx()
		times["b"].append(timed(lambda: bwd(dx)))
		del y, dx
		mems["b"].append((held() - start) / MiB)
		peaks["b"].append((peak() - before) / MiB)
		reset()
		before = held()
		times["w"].append(timed(wgrad))
		mems["w"].append((held() - start) / MiB)
		peaks["w"].append((peak() - before) / MiB)
	med = lambda d: {k: float(np.median(v)) for k, v in d.items()}
	T, M, Mpeak = med(times), med(mems), med(peaks)

	# whole-stage checkpoint forward
	reset()
	start = held()
	y = new_y()
	fwd(y, FWD_REMAT_ROOT)
	torch.cuda.synchronize()
	peak_ckpt = (peak() - start) / MiB
	# B re-runs the forward of a checkpointed micro-batch; with recompute_gradients it leaves only the
	# layer-input half of the W stash behind: that is Mba
	start = held() - y.numel() * 2
	dx = new_dx()
	bwd(dx, BWD_RECOMPUTE_GRADIENTS)
	torch.cuda.synchronize()
	del dx, y
	mba = (held() - start) / MiB
	_lib.check(lib.elf_stage_clear(h), "elf_stage_clear")
	for g, keep in zip(block._fused_g, saved_grads):
		g.copy_(keep)
	torch.cuda.synchronize()

	stats = {
		"T": T, "M": M, "Mpeak": Mpeak, "Mpeak_ckpt": peak_ckpt,
		"Mparams": 1.5 * sum(w.numel() * 2 for w in block._fused_w) / MiB + 0.5 * block.mem_stats()["workspace_bytes"] / MiB,
		"Mworkspace": block.mem_stats()["workspace_bytes"] / MiB,
		"Mba": mba, "Mbg": M["b"] - mba, "Minput": x.numel() * x.element_size() / MiB, "Moutput": dy.numel() * 2 / MiB, "Tcomm": 0.0,
		"forward_remat_options": [], "backward_remat_options": [],
	}
	return stats, warmup_output


def _simplified_schedule(placement, n_micro_batches, scheduler):
	"""Per rank, the base scheduler's compute ops as ("f"|"b"|"w", block, mb) in rank order."""
	per_rank = [[] for _ in range(len(set(placement)))]
	for op in scheduler(placement, n_micro_batches):
		if op.op in _KIND:
			per_rank[op.rank].append((_KIND[op.op], op.block_id, op.mb_id))
	return per_rank


def build_ilp_params(statistics, placement, scheduler, n_micro_batches, memory_budget):
	"""Profiling records -> the parameter dict of the ILP.  Per stage: ``full_fwd`` frees
	M_f - Minput - Moutput and costs T_f inside B; ``activations_bwd`` frees Mba and costs T_f
	inside W; ``full_bwd`` frees M_b - Moutput - Minput and costs T_f + T_b inside W."""
	assert len(statistics) == len(placement)
	stages = []
	for st in statistics:
		T, M = st["T"], st["M"]
		peaks = dict(st["Mpeak"])
		peaks["f_no_grad"] = st["Mpeak_ckpt"]
		stages.append({
			"T": T, "M": M, "Mpeak": peaks, "Tcomm": st["Tcomm"], "Mparams": st["Mparams"],
			"fwd_remat_options": [RematOption("full_fwd", "forward", M["f"] - st["Minput"] - st["Moutput"], T["f"])],
			"bwd_remat_options": [
				RematOption("activations_bwd", "backward", st["Mba"], T["f"]),
				RematOption("full_bwd", "backward", M["b"] - st["Moutput"] - st["Minput"], T["f"] + T["b"]),
			],
		})
	return {
		"p": len(set(placement)), "m": n_micro_batches, "nstages": len(placement), "MGpu": memory_budget,
		"sched": _simplified_schedule(placement, n_micro_batches, scheduler), "placement": list(placement), "stages": stages,
	}


class _Lin:
	"""Linear expression: {column: coefficient} + constant."""

	__slots__ = ("c", "k")

	def __init__(self, coeffs=None, const=0.0):
		self.c = dict(coeffs or {})
		self.k = float(const)

	def add(self, other, scale=1.0):
		if isinstance(other, _Lin):
			for col, v in other.c.items():
				self.c[col] = self.c.get(col, 0.0) + scale * v
			self.k += scale * other.k
		else:
			self.k += scale * float(other)
		return self

	def copy(self):
		return _Lin(self.c, self.k)

	def value(self, x):
		return self.k + sum(v * x[col] for col, v in self.c.items())


class _Model:
	"""Column layout and the linear helpers of the ILP (time_op / mem_kept / delta_mem / peak_mem)."""

	def __init__(self, params):
		self.P = params
		self.m, self.ns = params["m"], params["nstages"]
		self.stages = params["stages"]
		n = self.ns * self.m
		self.off_xF, self.off_xA, self.off_xG, self.off_E = 0, n, 2 * n, 3 * n
		self.col_T = 3 * n + 3 * n
		self.ncols = self.col_T + 1
		self.by_rank = {r: [i for i, k in enumerate(params["placement"]) if k == r] for r in range(params["p"])}

	def x(self, name, i, j):
		return {"full_fwd": self.off_xF, "activations_bwd": self.off_xA, "full_bwd": self.off_xG}[name] + i * self.m + j

	def E(self, s, j, op):
		return self.off_E + (s * self.m + j) * 3 + _OPS.index(op)

	def time_op(self, op, i, j):
		st = self.stages[i]
		e = _Lin(const=st["T"][op])
		if op == "b":
			for o in st["fwd_remat_options"]:
				e.add(_Lin({self.x(o.name, i, j): o.time_overhead}))
		elif op == "w":
			for o in st["bwd_remat_options"]:
				e.add(_Lin({self.x(o.name, i, j): o.time_overhead}))
		return e

	def mem_kept(self, op, i, j):
		st = self.stages[i]
		e = _Lin(const=st["M"][op])
		if op == "f":
			for o in st["fwd_remat_options"]:
				e.add(_Lin({self.x(o.name, i, j): -o.mem_freed}))
		elif op == "b":
			for o in st["bwd_remat_options"]:
				e.add(_Lin({self.x(o.name, i, j): -o.mem_freed}))
		return e

	def delta_mem(self, op, i, j):
		e = self.mem_kept(op, i, j)
		if op != "f":
			e.add(self.mem_kept(_OPS[_OPS.index(op) - 1], i, j), -1.0)
		return e

	def peak_mem(self, op, i, j):
		st = self.stages[i]
		pk = st["Mpeak"]
		pF, pB, pW, pNG = pk["f"], pk["b"], pk["w"], pk["f_no_grad"]
		mf, mb = st["M"]["f"], st["M"]["b"]
		if op == "f":
			return _Lin({self.x("full_fwd", i, j): pNG - pF}, pF)
		if op == "b":
			return _Lin({self.x("full_fwd", i, j): max(pF, mf + pB) - pB}, pB)
		return _Lin({self.x("full_bwd", i, j): max(pF, mf + pB, mb + pW) - pW, self.x("activations_bwd", i, j): pNG - pW}, pW)

	def mparams(self, rank):
		return 2 * sum(self.stages[s]["Mparams"] for s in self.by_rank[rank])

	def rank_time(self, rank):
		sched = self.P["sched"][rank]
		(fo, fs, fj), (lo, ls, lj) = sched[0], sched[-1]
		e = _Lin({self.E(ls, lj, lo): 1.0})
		e.add(_Lin({self.E(fs, fj, fo): 1.0}), -1.0)
		return e.add(self.time_op(fo, fs, fj))

	def rows(self):
		"""Yield (expr, sense, rhs) with sense in "<=", ">=", "==": expr sense rhs."""
		P, m, ns = self.P, self.m, self.ns
		plc = P["placement"]
		T = _Lin({self.col_T: 1.0})
		for rank in range(P["p"]):
			yield T.copy().add(self.rank_time(rank), -1.0), ">=", 0.0
		yield _Lin({self.E(0, 0, "f"): 1.0}).add(self.time_op("f", 0, 0), -1.0), "==", 0.0
		for rank in range(P["p"]):
			sched = P["sched"][rank]
			n_ops = 3 * m * len(self.by_rank[rank])
			kept = _Lin(const=self.mparams(rank))
			for k in range(n_ops):
				op, s, j = sched[k]
				cur = _Lin({self.E(s, j, op): 1.0})
				if op == "f" and s != 0:
					tcomm = self.stages[s - 1]["Tcomm"] if plc[s - 1] != rank else 0
					yield cur.copy().add(_Lin({self.E(s - 1, j, "f"): 1.0}), -1.0).add(self.time_op(op, s, j), -1.0).add(tcomm, -1.0), ">=", 0.0
				elif op == "b" and s != ns - 1:
					tcomm = self.stages[s]["Tcomm"] if plc[s + 1] != rank else 0
					yield cur.copy().add(_Lin({self.E(s + 1, j, "b"): 1.0}), -1.0).add(self.time_op(op, s, j), -1.0).add(tcomm, -1.0), ">=", 0.0
				if k != 0:
					po, ps, pj = sched[k - 1]
					yield cur.copy().add(_Lin({self.E(ps, pj, po): 1.0}), -1.0).add(self.time_op(op, s, j), -1.0), ">=", 0.0
				yield kept.copy().add(self.peak_mem(op, s, j)), "<=", float(P["MGpu"])
				kept.add(self.delta_mem(op, s, j))
		for s in range(ns):
			for j in range(m):
				yield _Lin({self.x("full_fwd", s, j): 1.0}), "<=", 1.0
				yield _Lin({self.x("activations_bwd", s, j): 1.0, self.x("full_bwd", s, j): 1.0}), "<=", 1.0

	def lower_bound_T(self):
		return max(sum(sum(self.stages[s]["T"][op] for op in _OPS) * self.m for s in self.by_rank[r]) for r in range(self.P["p"]))


def evaluate_remat(params, decisions):
	"""Makespan and per-rank peak memory of given 0/1 decisions {"full_fwd": [[..m]..stages], ...}
	under the model: end times are the longest-path solution of the precedence rows.  Returns
	(objective, peak_mems, feasible)."""
	mdl = _Model(params)
	x = np.zeros(mdl.ncols)
	for name in ("full_fwd", "activations_bwd", "full_bwd"):
		for i in range(mdl.ns):
			for j in range(mdl.m):
				x[mdl.x(name, i, j)] = float(decisions.get(name, [[0] * mdl.m] * mdl.ns)[i][j])
	# longest path: relax the ">=" rows between E columns until stable
	prec = []
	for e, sense, rhs in mdl.rows():
		ecols = [c for c in e.c if mdl.off_E <= c < mdl.col_T]
		if sense == "<=" or mdl.col_T in e.c or not ecols:
			continue
		prec.append((e, sense))
	for _ in range(mdl.ncols + 2):
		changed = False
		for e, sense in prec:
			tgt = [c for c in e.c if mdl.off_E <= c < mdl.col_T and e.c[c] > 0][0]
			need = x[tgt] - e.value(x)  # value that makes the row tight
			if need > x[tgt] + 1e-9 or (sense == "==" and abs(need - x[tgt]) > 1e-9):
				x[tgt] = need
				changed = True
		if not changed:
			break
	obj = max(mdl.lower_bound_T(), max(mdl.rank_time(r).value(x) for r in range(params["p"])))
	peaks, feasible = [], True
	for rank in range(params["p"]):
		acc, pk = mdl.mparams(rank), 0.0
		for op, s, j in params["sched"][rank]:
			pk = max(pk, acc + mdl.peak_mem(op, s, j).value(x))
			acc += mdl.delta_mem(op, s, j).value(x)
		peaks.append(pk)
		feasible &= pk <= params["MGpu"] + 1e-6
	return obj, peaks, feasible


def solve_remat(statistics, placement, scheduler, n_micro_batches, memory_budget, time_limit=60, gap_rel_limit=0.03):
	"""Solve the remat ILP; returns {"placement", "objective", "peak_mems", "order", "full_fwd",
	"activations_bwd", "full_bwd"} with the decisions as [stage][mb] lists of 0.0 / 1.0.
	Raises RuntimeError when the schedule cannot fit in ``memory_budget``."""
	from scipy.optimize import milp, LinearConstraint, Bounds
	from scipy.sparse import csr_matrix

	params = build_ilp_params(statistics, placement, scheduler, n_micro_batches, memory_budget)
	mdl = _Model(params)
	data, ri, ci, lo, hi = [], [], [], [], []
	for r, (e, sense, rhs) in enumerate(mdl.rows()):
		for col, v in e.c.items():
			if v != 0.0:
				data.append(v)
				ri.append(r)
				ci.append(col)
		bound = rhs - e.k
		lo.append(bound if sense in (">=", "==") else -np.inf)
		hi.append(bound if sense in ("<=", "==") else np.inf)
	A = csr_matrix((data, (ri, ci)), shape=(len(lo), mdl.ncols))
	c = np.zeros(mdl.ncols)
	c[mdl.col_T] = 1.0
	lb = np.zeros(mdl.ncols)
	ub = np.full(mdl.ncols, np.inf)
	ub[: mdl.off_E] = 1.0
	lb[mdl.col_T] = mdl.lower_bound_T()
	integrality = np.zeros(mdl.ncols)
	integrality[: mdl.off_E] = 1
	try:
		name = SCHEDULERS.get_key(scheduler)
	except ValueError:
		name = getattr(scheduler, "__name__", "custom")
	logger.info(f"Solving ILP with HiGHS, {name} scheduler, {time_limit} seconds time limit and {memory_budget} MB memory budget")
	t0 = time.time()
	res = milp(c, constraints=LinearConstraint(A, lo, hi), integrality=integrality, bounds=Bounds(lb, ub),
	           options={"time_limit": float(time_limit), "mip_rel_gap": float(gap_rel_limit), "disp": False})
	solve_time = time.time() - t0
	if res.status == 2 or res.x is None:
		raise RuntimeError(
			f"ILP is infeasible: cannot fit the schedule within {memory_budget} MB. "
			"Try increasing memory_budget, reducing n_micro_batches or using a different scheduler."
		)
	x = res.x
	solution = {"placement": list(params["placement"]), "objective": float(res.fun)}
	peaks = []
	for rank in range(params["p"]):
		acc, pk = mdl.mparams(rank), 0
		for op, s, j in params["sched"][rank]:
			pk = max(pk, acc + mdl.peak_mem(op, s, j).value(x))
			acc += mdl.delta_mem(op, s, j).value(x)
		peaks.append(pk)
	solution["peak_mems"] = peaks
	solution["order"] = [op for rank_sched in params["sched"] for op in rank_sched]
	for nm in ("full_fwd", "activations_bwd", "full_bwd"):
		solution[nm] = [[float(round(x[mdl.x(nm, i, j)])) for j in range(mdl.m)] for i in range(mdl.ns)]
	logger.info(f"ILP solved in {solve_time:.2f} seconds: objective={solution['objective']:.1f}ms, peak_mems={[f'{p:.0f}MB' for p in peaks]}")
	return solution


class RematScheduler:
	"""Base scheduler + a solution dict -> op list with the remat decisions applied:

	full_fwd[b][mb]         F gets ``remat_strategy`` = "the stage root" (whole-stage checkpoint);
	activations_bwd[b][mb]  B gets ``recompute_activations``; a RECOMPUTE_FORWARD is inserted
	                        right before W(b, mb);
	full_bwd[b][mb]         additionally B gets ``recompute_gradients``, that RECOMPUTE_FORWARD gets
	                        ``save`` and a RECOMPUTE_BACKWARD_INPUTS is inserted between it and W."""

	def __init__(self, base_scheduler, solution):
		self.base_scheduler = base_scheduler
		self.solution = solution

	@property
	def makespan(self):
		return self.solution["objective"]

	@staticmethod
	def _root_only(name, module):
		return name == ""

	def _flag(self, key, op):
		table = self.solution.get(key, [])
		return bool(table and table[op.block_id][op.mb_id])

	def __call__(self, placement, nmb):
		schedule = self.base_scheduler(placement, nmb)

		def index_of_w(op):
			for i, o in enumerate(schedule):
				if o.op == OperationType.BACKWARD_PARAMS and o.block_id == op.block_id and o.mb_id == op.mb_id:
					return i
			return None

		for op in list(schedule):
			if op.op == OperationType.FORWARD:
				if self._flag("full_fwd", op):
					op.options[OpOptions.REMAT_STRATEGY] = self._root_only
			elif op.op == OperationType.BACKWARD_INPUTS:
				acts, everything = self._flag("activations_bwd", op), self._flag("full_bwd", op)
				if not (acts or everything):
					continue
				op.options[OpOptions.RECOMPUTE_ACTIVATIONS] = True
				rf = Operation(op.block_id, op.mb_id, OperationType.RECOMPUTE_FORWARD, op.rank)
				at = index_of_w(op)
				if at is not None:
					schedule.insert(at, rf)
				if everything:
					rf.options[OpOptions.SAVE] = True
					op.options[OpOptions.RECOMPUTE_GRADIENTS] = True
					at = index_of_w(op)
					if at is not None:
						schedule.insert(at, Operation(op.block_id, op.mb_id, OperationType.RECOMPUTE_BACKWARD_INPUTS, op.rank))
		return schedule


def _broadcast(obj, src):
	import torch.distributed as dist

	if dist.is_available() and dist.is_initialized() and dist.get_world_size() > 1:
		box = [obj]
		dist.broadcast_object_list(box, src=src)
		return box[0]
	return obj


def _my_rank():
	import torch.distributed as dist

	return dist.get_rank() if dist.is_available() and dist.is_initialized() else 0


def _alternatives(stats):
	"""``stats`` as the callers give it -> [(label, statistics per stage, callable that puts the stages into that
	state or None)].  Plain per-stage statistics are one alternative; a list of ``(label, statistics, apply)``
	triples (e.g. the stages profiled at two stash levels) is taken as it is."""
	if stats and isinstance(stats[0], tuple):
		return list(stats)
	return [(None, stats, None)]


def solve_remat_best(stats, placement, scheduler, n_micro_batches, memory_budget, **kw):
	"""``solve_remat`` over every alternative of ``stats`` (see ``_alternatives``) -> (index of the alternative
	with the smallest makespan, its solution).  An alternative the budget cannot hold is skipped; when none
	fits, the last error is raised."""
	best, err = (None, None), None
	for k, (label, st, _) in enumerate(_alternatives(stats)):
		try:
			sol = solve_remat(st, placement, scheduler, n_micro_batches, memory_budget, **kw)
		except RuntimeError as e:
			err = e
			continue
		if label is not None:
			logger.info(f"remat ILP, {label}: makespan {sol['objective']:.2f} ms")
		if best[1] is None or sol["objective"] < best[1]["objective"]:
			best = (k, sol)
	if best[1] is None:
		raise err
	return best


def stagerematify(scheduler, stats, budget, worker=0):
	"""scheduler -> scheduler that solves the ILP on rank ``worker`` (lazily, per call), shares the
	solution with the other ranks and applies it.  ``stats``: the statistics of every stage, or alternatives
	of them (``_alternatives``): the one with the best makespan is applied, stages included."""

	def StageRemat(placement, nmb):
		choice = solve_remat_best(stats, placement, scheduler, nmb, budget) if _my_rank() == worker else None
		k, solution = _broadcast(choice, worker)
		apply = _alternatives(stats)[k][2]
		if apply is not None:
			apply()
		return RematScheduler(scheduler, solution)(placement, nmb)

	return StageRemat


class AutoScheduler:
	"""Solves the ILP for every base scheduler and applies the one with the best makespan."""

	def __init__(self, stats, budget, worker=0):
		self.stats, self.budget, self.worker = stats, budget, worker
		self.schedulers = [k for k in SCHEDULERS.available() if k not in ("auto", "fixed", "full_remat")]

	def __call__(self, placement, nmb):
		best = (float("inf"), None, None, 0)
		if _my_rank() == self.worker:
			for name in self.schedulers:
				try:
					k, sol = solve_remat_best(self.stats, placement, resolve(name, SCHEDULERS), nmb, self.budget)
					if sol["objective"] < best[0]:
						best = (sol["objective"], name, sol, k)
				except Exception as e:  # e.g. a multi-wave scheduler on a single-wave placement
					logger.info(f"Error solving ILP for {name} scheduler: {e}. Skipping.")
			logger.info(f"Best scheduler: {best[1]} with {best[0]:.2f}ms makespan")
		best = _broadcast(best, self.worker)
		if best[1] is None:
			raise RuntimeError("AutoScheduler: no base scheduler admits a feasible remat plan for this budget and placement")
		apply = _alternatives(self.stats)[best[3]][2]
		if apply is not None:
			apply()
		return RematScheduler(resolve(best[1], SCHEDULERS), best[2])(placement, nmb)
