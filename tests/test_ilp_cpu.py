"""The remat ILP (elf_amd/scheduling/ilp.py).  The reference states the same model with PuLP and
solves it with CBC / CPLEX to a 3 % gap (elf/scheduling/ilp.py:491-747); neither PuLP nor a
solver ships with it and its tests do not touch it, so decisions are pinned through the model:
closed forms on single-rank instances, brute force over the binaries on small pipelines,
feasibility replay, monotonicity in the budget, and the infeasible / no-remat limits."""

import itertools

import pytest

from elf_amd.registry import SCHEDULERS
from elf_amd.scheduling.ilp import build_ilp_params, evaluate_remat, solve_remat


def _stats(Tf=10.0, Tb=12.0, Tw=8.0, Mf=100.0, Mb=60.0, Mw=0.0, Pf=120.0, Pb=110.0, Pw=70.0, Pck=30.0, Mp=50.0, Mba=25.0, Min=5.0, Mout=5.0, Tcomm=1.0):
	return {"T": {"f": Tf, "b": Tb, "w": Tw}, "M": {"f": Mf, "b": Mb, "w": Mw}, "Mpeak": {"f": Pf, "b": Pb, "w": Pw}, "Mpeak_ckpt": Pck,
	        "Mparams": Mp, "Mba": Mba, "Minput": Min, "Moutput": Mout, "Tcomm": Tcomm}


def test_no_remat_when_the_budget_is_loose():
	st = [_stats(), _stats()]
	sol = solve_remat(st, [0, 1], SCHEDULERS["1f1b"], 4, 10_000)
	assert all(v == 0.0 for key in ("full_fwd", "activations_bwd", "full_bwd") for row in sol[key] for v in row)
	assert sol["placement"] == [0, 1] and len(sol["order"]) == 2 * 3 * 4
	assert set(sol) == {"placement", "objective", "peak_mems", "order", "full_fwd", "activations_bwd", "full_bwd"}
	# rank 0 under 1F1B holds 2 forwards when its first B runs: 2*Mparams + Mf + (Mf + Pb)
	assert sol["peak_mems"][0] == pytest.approx(2 * 50 + 100 + max(120, 100 + 110))


def test_single_rank_closed_form():
	"""One rank, AFAB: the makespan is the sum of op times; with m = 2 the memory rows are
	2 Mp + P_f, + kept_f + P_f, + 2 kept_f + P_b, ...  A budget that only admits one un-rematted
	forward forces exactly one full_fwd (cheapest: +T_f) and the objective is sum + T_f."""
	st = [_stats()]
	base = 2 * (10 + 12 + 8)
	loose = solve_remat(st, [0], SCHEDULERS["afab"], 2, 1000)
	assert loose["objective"] == pytest.approx(base)
	# no remat: after F0, F1 kept = 200, B0 peak: 100 + 200 + 110 = 410
	assert loose["peak_mems"][0] == pytest.approx(410)
	tight = solve_remat(st, [0], SCHEDULERS["afab"], 2, 409)
	n_ff = sum(tight["full_fwd"][0])
	assert n_ff >= 1 and tight["objective"] == pytest.approx(base + 10 * n_ff + 10 * sum(tight["activations_bwd"][0]) + 22 * sum(tight["full_bwd"][0]))
	assert tight["objective"] <= (base + 10) * 1.03 + 1e-6
	assert tight["peak_mems"][0] <= 409 + 1e-6


def test_infeasible_budget_raises():
	with pytest.raises(RuntimeError, match="infeasible"):
		solve_remat([_stats(), _stats()], [0, 1], SCHEDULERS["1f1b"], 4, 150)


@pytest.mark.parametrize("sched,placement,nmb", [("1f1b", [0, 1], 2), ("zbh1", [0, 1], 2), ("afab", [0, 1], 2)])
def test_objective_within_gap_of_bruteforce(sched, placement, nmb):
	st = [_stats(), _stats(Tf=9.0, Tb=11.0, Mf=90.0, Mba=20.0)]
	loose = build_ilp_params(st, placement, SCHEDULERS[sched], nmb, 1e9)
	zeros = lambda v: [[v] * nmb for _ in placement]
	_, p_none, _ = evaluate_remat(loose, {})
	_, p_all, _ = evaluate_remat(loose, {"full_fwd": zeros(1), "full_bwd": zeros(1), "activations_bwd": zeros(0)})
	budget = 0.5 * (max(p_none) + max(p_all))  # binding, but reachable
	assert max(p_all) < budget < max(p_none)
	sol = solve_remat(st, placement, SCHEDULERS[sched], nmb, budget)
	assert any(v for key in ("full_fwd", "activations_bwd", "full_bwd") for row in sol[key] for v in row), "the budget must force some remat"
	params = build_ilp_params(st, placement, SCHEDULERS[sched], nmb, budget)
	obj, peaks, feasible = evaluate_remat(params, sol)
	assert feasible and all(p <= budget + 1e-6 for p in peaks), "replayed decisions must respect the budget"
	assert peaks == pytest.approx(sol["peak_mems"])
	# brute force over the binaries ({f} x {none, activations_bwd, full_bwd} per (stage, mb)); the
	# earliest-start replay is an upper bound of each LP, so the best replay >= the true optimum
	best = float("inf")
	choices = list(itertools.product([0, 1], [(0, 0), (1, 0), (0, 1)]))
	n = len(placement) * nmb
	for combo in itertools.product(choices, repeat=n):
		dec = {"full_fwd": zeros(0), "activations_bwd": zeros(0), "full_bwd": zeros(0)}
		for idx, (ff, (ab, fb)) in enumerate(combo):
			s, j = divmod(idx, nmb)
			dec["full_fwd"][s][j], dec["activations_bwd"][s][j], dec["full_bwd"][s][j] = ff, ab, fb
		o, _, ok = evaluate_remat(params, dec)
		if ok:
			best = min(best, o)
	assert sol["objective"] <= best * 1.03 + 1e-6


def test_monotone_in_budget():
	st = [_stats(), _stats()]
	objs = [solve_remat(st, [0, 1], SCHEDULERS["1f1b"], 4, b)["objective"] for b in (330, 345, 360, 450, 1000)]
	assert all(a >= b - 1e-6 - 0.03 * b for a, b in zip(objs, objs[1:]))
	assert objs[-1] == pytest.approx(min(objs), rel=0.03)


def test_auto_scheduler_picks_the_best_base_scheduler_and_stagerematify_applies_its_plan():
	"""``AutoScheduler`` (elf/scheduling/ilp.py:828-853 of the reference: solve the ILP for every registered
	base scheduler, keep the smallest makespan) and ``stagerematify`` (the lazy per-call wrapper
	``Pipeline(memory_budget=)`` builds): the chosen plan is the best of the per-scheduler solutions, the op
	list is that scheduler's list rewritten by ``RematScheduler``, and a tight budget shows up as remat ops."""
	from elf_amd.scheduling import OperationType as T, OpOptions, check_schedule_validity
	from elf_amd.scheduling.ilp import AutoScheduler, RematScheduler, stagerematify

	st, placement, nmb = [_stats(), _stats()], [0, 1], 4
	loose, tight = 10_000, 400  # the no-remat peak of rank 0 under 1F1B is 410 (see the first test); nothing fits below 330
	auto = AutoScheduler(st, loose)
	assert "auto" not in auto.schedulers and "fixed" not in auto.schedulers and "1f1b" in auto.schedulers and "zbh1" in auto.schedulers
	objectives = {}
	for name in auto.schedulers:
		try:
			objectives[name] = solve_remat(st, placement, SCHEDULERS[name], nmb, loose)["objective"]
		except Exception:
			pass
	best = min(objectives, key=objectives.get)
	got = auto(placement, nmb)
	check_schedule_validity(got)
	want = RematScheduler(SCHEDULERS[best], solve_remat(st, placement, SCHEDULERS[best], nmb, loose))(placement, nmb)
	assert [(o.op, o.block_id, o.mb_id, o.rank) for o in got] == [(o.op, o.block_id, o.mb_id, o.rank) for o in want]
	assert not any(o.op in (T.RECOMPUTE_FORWARD, T.RECOMPUTE_BACKWARD_INPUTS) or o.options.get(OpOptions.REMAT_STRATEGY) for o in got)

	def remat_ops(schedule):
		return [o for o in schedule if o.op in (T.RECOMPUTE_FORWARD, T.RECOMPUTE_BACKWARD_INPUTS) or o.options.get(OpOptions.REMAT_STRATEGY) is not None]

	constrained = AutoScheduler(st, tight)(placement, nmb)
	check_schedule_validity(constrained)
	assert remat_ops(constrained), "a budget below the no-remat peak must force rematerialisation"
	wrapped = stagerematify(SCHEDULERS["1f1b"], st, tight)
	s1 = wrapped(placement, nmb)
	s2 = RematScheduler(SCHEDULERS["1f1b"], solve_remat(st, placement, SCHEDULERS["1f1b"], nmb, tight))(placement, nmb)
	assert [(o.op, o.block_id, o.mb_id, o.rank) for o in s1] == [(o.op, o.block_id, o.mb_id, o.rank) for o in s2] and remat_ops(s1)
	with pytest.raises(RuntimeError):
		AutoScheduler(st, 1.0)(placement, nmb)  # no scheduler fits 1 MiB


def test_alternatives_of_the_stage_statistics_compete_on_the_makespan():
	"""``Pipeline(memory_budget=)`` profiles its stages at two lean stash levels and hands both to the ILP wrappers
	(no counterpart in the reference, whose stages have one stash): a leaner stash costs backward time and frees
	memory.  With a loose budget the faster alternative wins, with a tight one the leaner one (it needs fewer
	recomputed forwards), an alternative the budget cannot hold at all is skipped, and the winner's ``apply`` is
	the one that runs."""
	from elf_amd.scheduling.ilp import AutoScheduler, RematScheduler, solve_remat_best, stagerematify

	placement, nmb = [0, 1], 4
	fast = [_stats(), _stats()]                                        # stash 100 per micro-batch
	lean = [_stats(Tb=13.0, Mf=60.0, Pf=110.0), _stats(Tb=13.0, Mf=60.0, Pf=110.0)]  # 40 less, backward 1 ms slower
	applied = []
	alts = [("fast", fast, lambda: applied.append("fast")), ("lean", lean, lambda: applied.append("lean"))]

	k, sol = solve_remat_best(alts, placement, SCHEDULERS["1f1b"], nmb, 10_000)
	assert k == 0 and sol["objective"] == pytest.approx(solve_remat(fast, placement, SCHEDULERS["1f1b"], nmb, 10_000)["objective"])
	# plain statistics are one alternative
	k1, sol1 = solve_remat_best(fast, placement, SCHEDULERS["1f1b"], nmb, 10_000)
	assert k1 == 0 and sol1["objective"] == pytest.approx(sol["objective"])

	tight = 400  # below the fast stash's no-remat peak of 410; the lean stash fits without recomputing
	o_fast = solve_remat(fast, placement, SCHEDULERS["1f1b"], nmb, tight)["objective"]
	o_lean = solve_remat(lean, placement, SCHEDULERS["1f1b"], nmb, tight)["objective"]
	assert o_lean < o_fast
	k, sol = solve_remat_best(alts, placement, SCHEDULERS["1f1b"], nmb, tight)
	assert k == 1 and sol["objective"] == pytest.approx(o_lean)

	got = stagerematify(SCHEDULERS["1f1b"], alts, tight)(placement, nmb)
	assert applied == ["lean"]
	want = RematScheduler(SCHEDULERS["1f1b"], solve_remat(lean, placement, SCHEDULERS["1f1b"], nmb, tight))(placement, nmb)
	assert [(o.op, o.block_id, o.mb_id, o.rank) for o in got] == [(o.op, o.block_id, o.mb_id, o.rank) for o in want]
	stagerematify(SCHEDULERS["1f1b"], alts, 10_000)(placement, nmb)
	assert applied == ["lean", "fast"]
	AutoScheduler(alts, tight)(placement, nmb)
	assert applied[-1] == "lean"

	# the fast stash cannot fit 300 at all (its infeasibility is not an error while another alternative fits)
	with pytest.raises(RuntimeError):
		solve_remat(fast, placement, SCHEDULERS["1f1b"], nmb, 300)
	k, _ = solve_remat_best(alts, placement, SCHEDULERS["1f1b"], nmb, 300)
	assert k == 1
	with pytest.raises(RuntimeError, match="infeasible"):
		solve_remat_best(alts, placement, SCHEDULERS["1f1b"], nmb, 100)
