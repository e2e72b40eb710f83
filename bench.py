#!/usr/bin/env python3
"""Stage throughput benchmark: one pass ("step") of a pipeline stage's operation stream
(F, split B, deferred W, grad scale) over one batch of synthetic micro-batches on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

Prints ONE JSON line.  ``value`` = tokens/s of the whole stream with weights, boundary
activations and boundary gradients already resident in HBM.  ``roofline`` is for the dominant
kernel family (the bf16 MFMA GEMM): algorithmic FLOPs (2MNK per launch) divided by the launch
durations measured live with HIP events on the launch stream, against the published dense bf16
peak.  ``cpu_baseline`` times the plain-PyTorch CPU restatement of the reference stage (oracle/)
on a bounded sample (one micro-batch of F, B and W through ONE block, fp32; one warm-up pass, median of
three) on the host cores.
"""

import argparse
import contextlib
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0


def gemm_traffic_bytes(workload):
	"""HBM bytes per GEMM launch (mean over the launches of one step) of ``workload``: read from the line the counter
	summary under profiles/ ends with (rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs of this script, scaled by
	the same counters' reading for a copy kernel of known size, --calibration-copy), so that the figure has one
	source; None where no counter run was summarised."""
	import re

	try:
		text = open(os.path.join(ROOT, "profiles", f"stage_kernels_{workload}.md")).read()
	except OSError:
		return None
	m = re.search(r"\(([0-9.e+]+) bytes: bench\.py's `roofline\.traffic`\)", text)
	return float(m.group(1)) if m else None


WORKLOADS = {
	# headline configuration: Llama-3-8B-shaped stage, ZB-H1 stream of block 1 in a 4-stage pipeline
	"llama3_8b_zbh1": dict(arch="llama", n_blocks=4, d=4096, heads=32, kv_heads=8, head_dim=128, ffn=14336, seq=4096, mb=2, n_mb=16,
	                       scheduler="zbh1", causal=True, rope_theta=5e5),
	# same stage under 1F1B
	"llama3_8b_1f1b": dict(arch="llama", n_blocks=4, d=4096, heads=32, kv_heads=8, head_dim=128, ffn=14336, seq=4096, mb=2, n_mb=16,
	                       scheduler="1f1b", causal=True, rope_theta=5e5),
	# small configuration: GPT-2-small-shaped stage, 1F1B
	"gpt2s_1f1b": dict(arch="gpt", n_blocks=3, d=768, heads=12, kv_heads=12, head_dim=64, ffn=3072, seq=1024, mb=8, n_mb=8,
	                   scheduler="1f1b", causal=False, time_one_in=16),
	# offload configuration: Llama-3-70B-shaped stage, 1F1B with activation offload
	"llama3_70b_offload": dict(arch="llama", n_blocks=2, d=8192, heads=64, kv_heads=8, head_dim=128, ffn=28672, seq=8192, mb=1, n_mb=8,
	                           scheduler="1f1b", causal=True, rope_theta=5e5, offload=True),
	# remat configuration: the Llama-3-8B-shaped stage with 8 blocks at seq 8192 under a 48 GB budget: the stage is
	# profiled on the native executor, the remat ILP is solved for a pipeline of 8 such stages (the other stages are
	# copies of the measured one) and block 1's rewritten 1F1B stream runs
	"llama3_8b_remat": dict(arch="llama", n_blocks=8, d=4096, heads=32, kv_heads=8, head_dim=128, ffn=14336, seq=8192, mb=1, n_mb=16,
	                        scheduler="1f1b", causal=True, rope_theta=5e5, placement=list(range(8)), memory_budget_mib=48e9 / 2**20),
	# small shape for smoke runs
	"tiny": dict(arch="llama", n_blocks=2, d=512, heads=4, kv_heads=2, head_dim=128, ffn=768, seq=256, mb=2, n_mb=4,
	             scheduler="zbh1", causal=True, rope_theta=5e5),
}
PLACEMENT = [0, 1, 2, 3]
BLOCK_ID = 1  # a middle stage: no embedding, no loss


def stream_flops(w):
	"""Algorithmic FLOPs of one step (F + B + W over all blocks and micro-batches); attention
	backward counted as 4 matmuls, causal attention at half the square."""
	T, d, F = w["mb"] * w["seq"], w["d"], w["ffn"]
	nq, nkv = w["heads"] * w["head_dim"], w["kv_heads"] * w["head_dim"]
	lin = 2.0 * T * (d * (nq + 2 * nkv) + nq * d + d * F * (3 if w["arch"] == "llama" else 2))
	att = (2.0 if w["causal"] else 4.0) * w["mb"] * w["heads"] * w["seq"] ** 2 * w["head_dim"]
	return (3 * lin + 3 * att) * w["n_blocks"] * w["n_mb"]


def build_stage(w):
	from elf_amd import models

	if w["arch"] == "llama":
		return models.llama_stage(w["n_blocks"], w["d"], w["heads"], w["kv_heads"], w["ffn"], w["seq"], head_dim=w["head_dim"], rope_theta=w["rope_theta"], seed=0)
	return models.gpt_stage(w["n_blocks"], w["d"], w["heads"], w["ffn"], w["seq"], causal=w["causal"], seed=0)


def op_stream(w, sched=None):
	from elf_amd.benchmark_utils import get_offloaded_scheduler
	from elf_amd.partitioners.utils import sequential_signatures
	from elf_amd.registry import COMM_SCHEDULERS, SCHEDULERS
	from elf_amd.scheduling import add_comms, check_schedule_validity

	placement = w.get("placement", PLACEMENT)
	if sched is None:
		sched = get_offloaded_scheduler(w["scheduler"], 1, w.get("prefetching_time", 1)) if w.get("offload") else SCHEDULERS[w["scheduler"]]
	schedule = COMM_SCHEDULERS["pipelined"](add_comms(sched(placement, w["n_mb"]), sequential_signatures(placement)))
	check_schedule_validity(schedule)
	return [op for op in schedule if op.block_id == BLOCK_ID]


def make_block(w, stage):
	"""The stage executor of block ``BLOCK_ID`` as Pipeline builds it: a stage that runs under a memory budget holds the lean stash."""
	from elf_amd.execution import HipStageBlock
	from elf_amd.partitioners.utils import sequential_signatures

	placement = w.get("placement", PLACEMENT)
	return HipStageBlock(stage, BLOCK_ID, placement, sequential_signatures(placement)[BLOCK_ID], mb_size=w["mb"], lean_stash=bool(w.get("memory_budget_mib")))


def plan_stream(w, block):
	"""(op stream of the workload, remat record or None).  Under a memory budget the stage is profiled on the native
	executor, the remat ILP is solved for a pipeline of such stages and the block's rewritten stream is returned."""
	import torch

	if not w.get("memory_budget_mib"):
		return op_stream(w), None
	from elf_amd.registry import SCHEDULERS
	from elf_amd.scheduling.ilp import RematScheduler, profile_stage, solve_remat_best

	placement = w.get("placement", PLACEMENT)
	# as Pipeline does: the stage profiled at both lean stash levels, the ILP's makespan picks one
	by_level = {}
	for level in (1, 2):
		block.set_lean_stash(level)
		by_level[level] = profile_stage(block, n_iter=3)[0]
	stats = by_level[1]
	# The budget is for everything this process holds on the device.  The ILP's memory model covers weights,
	# fp32 gradient accumulators, the stage's fixed scratch (2 x Mparams) and the activations; what is resident
	# beyond that comes off the budget it is given: the boundary tensors of all micro-batches (inputs and
	# output gradients now, outputs and input gradients as the step produces them; a pipeline would pass them
	# on one at a time) and the bf16 copies of the gradients that scale_grads leaves behind.
	unmodelled_mib = max(0.0, torch.cuda.memory_allocated() / 2**20 + stats["Mworkspace"] - 2 * stats["Mparams"])
	unmodelled_mib += w["n_mb"] * (stats["Minput"] + stats["Moutput"]) + sum(p.numel() * 2 for p in block._fused_w) / 2**20
	t_ilp = time.perf_counter()
	alternatives = [(f"lean stash level {level}", [by_level[level]] * len(placement), None) for level in (1, 2)]
	k, solution = solve_remat_best(alternatives, placement, SCHEDULERS[w["scheduler"]], w["n_mb"], w["memory_budget_mib"] - unmodelled_mib)
	t_ilp = time.perf_counter() - t_ilp
	block.set_lean_stash(k + 1)
	stats = by_level[k + 1]
	remat = {
		"lean_stash_level": k + 1,
		"memory_budget_mib": w["memory_budget_mib"], "unmodelled_resident_mib": unmodelled_mib, "ilp_seconds": t_ilp, "ilp_makespan_ms": solution["objective"],
		"ilp_peak_mib_rank": solution["peak_mems"][placement[BLOCK_ID]],
		"decisions_block": {k: int(sum(solution[k][BLOCK_ID])) for k in ("full_fwd", "activations_bwd", "full_bwd")},
		"profile": {k: stats[k] for k in ("T", "M", "Mpeak", "Mpeak_ckpt", "Mparams", "Mba", "Mbg", "Minput")},
	}
	return op_stream(w, RematScheduler(SCHEDULERS[w["scheduler"]], solution)), remat


def plain_stream(w):
	"""(name, op stream) of the stream the workload's own stream must reproduce bit for bit on the same stage: the
	scheduler without the remat rewrite, without the offload wrapper, or - for the split-backward ZB-H1 stream -
	plain 1F1B, which runs the same F, B and W per micro-batch with every accumulation in the same order; a plain
	1F1B workload is compared with a second run of itself."""
	from elf_amd.registry import SCHEDULERS

	if w.get("memory_budget_mib"):
		return f"{w['scheduler']} without the remat rewrite", op_stream(w, SCHEDULERS[w["scheduler"]])
	if w.get("offload"):
		return f"{w['scheduler']} without activation offload", op_stream(w, SCHEDULERS[w["scheduler"]])
	if w["scheduler"] != "1f1b":
		return "1f1b", op_stream(w, SCHEDULERS["1f1b"])
	return "a second run of the same stream", op_stream(w)


def run_and_keep(block, engine, stream, mb_sizes, xs, dys):
	"""One step of ``stream`` from zeroed accumulators with everything the stage produces kept: what SEND_FORWARD and
	SEND_BACKWARD would ship per micro-batch, a copy of every fused fp32 gradient accumulator, the library's counters."""
	import torch

	block.set_boundary(inputs=xs, grads=dys, keep_sent=True)
	block.zero_grad()
	block.reset_peak()
	torch.cuda.reset_peak_memory_stats()
	before = block.mem_stats()
	engine.train_step(None, None, None, stream, mb_sizes)
	torch.cuda.synchronize()
	mem = block.mem_stats()
	peak = mem["peak_bytes"] + mem["workspace_bytes"] + torch.cuda.max_memory_allocated()  # before the copies below are made
	kept = {"y": dict(block.sent_forward), "dx": dict(block.sent_backward), "grads": [g.clone() for g in block._fused_g], "mem": mem,
	        "d2h": mem["d2h_bytes"] - before["d2h_bytes"], "h2d": mem["h2d_bytes"] - before["h2d_bytes"], "peak_bytes": peak}
	block.set_boundary(inputs=xs, grads=dys)
	return kept


def compare_kept(a, b):
	"""Bit equality of two ``run_and_keep`` records, and the largest difference relative to the tensor's largest
	magnitude where they differ."""
	import torch

	out = {"micro_batches": len(a["y"]), "outputs_equal": True, "input_grads_equal": True, "weight_grads_equal": True, "max_rel_diff": 0.0}

	def cmp(x, y, key):
		if x.shape != y.shape or not torch.equal(x, y):
			out[key] = False
			d = (x.float() - y.float()).abs().max().item() / (y.float().abs().max().item() + 1e-30) if x.shape == y.shape else float("inf")
			out["max_rel_diff"] = max(out["max_rel_diff"], d)

	if set(a["y"]) != set(b["y"]) or set(a["dx"]) != set(b["dx"]) or len(a["grads"]) != len(b["grads"]):
		return dict(out, outputs_equal=False, input_grads_equal=False, weight_grads_equal=False, max_rel_diff=float("inf"))
	for m in a["y"]:
		cmp(a["y"][m], b["y"][m], "outputs_equal")
	for m in a["dx"]:
		cmp(a["dx"][m], b["dx"][m], "input_grads_equal")
	for x, y in zip(a["grads"], b["grads"]):
		cmp(x, y, "weight_grads_equal")
	return out


def check_stream(w, block, engine, stream, mb_sizes, xs, dys):
	"""The reference's own criterion, "the pipeline gives what the plain model gives" (benchmarks/benchmark_utils.py:
	215-292), at the workload's full size: the workload's stream and its plain counterpart (``plain_stream``) run on
	the same stage from the same boundary tensors and must agree bit for bit in every stage output, every input
	gradient and every accumulated weight gradient."""
	name, plain = plain_stream(w)
	got = run_and_keep(block, engine, stream, mb_sizes, xs, dys)
	want = run_and_keep(block, engine, plain, mb_sizes, xs, dys)
	out = compare_kept(got, want)
	out.update({"against": name, "peak_bytes": got["peak_bytes"], "plain_peak_bytes": want["peak_bytes"], "d2h_bytes": got["d2h"], "h2d_bytes": got["h2d"]})
	out["ok"] = bool(out["outputs_equal"] and out["input_grads_equal"] and out["weight_grads_equal"] and got["d2h"] == got["h2d"])
	return out


def cpu_baseline(w, stage_module, repeats=3):
	"""Oracle stage on the host cores: F, B, W of ONE micro-batch through ONE block, fp32; one untimed
	warm-up pass, then the median of ``repeats`` timed passes."""
	import statistics

	import torch
	from oracle import stage_ref as R
	from tests.helpers import cfg_from_stage, oracle_params_from_stage

	cores = os.cpu_count() or 1
	torch.set_num_threads(cores)
	cfg = cfg_from_stage(stage_module, w["mb"])
	cfg["n_blocks"] = 1
	params = [{k: v.cpu() for k, v in oracle_params_from_stage(stage_module)[0].items()}]
	ref = R.RefStage(cfg, params, compute_dtype=torch.float32, device="cpu", use_sdpa=True)
	xs, dys = R.make_boundary(cfg, 1, seed=1)

	def one_pass():
		t0 = time.perf_counter()
		ref.forward(0, xs[0])
		t1 = time.perf_counter()
		ref.backward_inputs(0, dys[0])
		t2 = time.perf_counter()
		ref.backward_params(0)
		t3 = time.perf_counter()
		ref.zero_grad()
		return t1 - t0, t2 - t1, t3 - t2

	one_pass()  # warm-up: thread pool, allocator, first-touch of the weights
	runs = [one_pass() for _ in range(repeats)]
	f, b, wt = (statistics.median(r[i] for r in runs) for i in range(3))
	T = w["mb"] * w["seq"]
	per_block = statistics.median(sum(r) for r in runs)
	return {
		"value": T / (per_block * w["n_blocks"]), "unit": "tokens/s", "cores": cores, "kind": "port",
		"sample": f"oracle/stage_ref.py RefStage on CPU, fp32, SDPA attention: 1 micro-batch ({T} tokens) of F+B+W through 1 of {w['n_blocks']} blocks, "
		          f"1 warm-up pass then the median of {repeats} (F {f:.2f}s, B {b:.2f}s, W {wt:.2f}s), extrapolated to the {w['n_blocks']}-block stage",
	}


class Telemetry:
	"""Socket power and shader clock sampled on a host thread while the timed steps run (``--telemetry``):
	amdsmi's gpu_metrics (per-XCD ``current_gfxclks``, ``average_socket_power`` / ``current_socket_power``)
	where the module is importable, else the hwmon ``power1_input`` file alone."""

	def __init__(self, period=0.05):
		import threading

		self.period, self.samples, self._stop = period, [], threading.Event()
		self._thread = threading.Thread(target=self._run, daemon=True)
		self._smi = None
		try:
			import amdsmi

			amdsmi.amdsmi_init()
			self._smi, self._dev = amdsmi, amdsmi.amdsmi_get_processor_handles()[0]
		except Exception:
			self._smi = None

	def _sample(self):
		rec = {}
		if self._smi is not None:
			try:
				m = self._smi.amdsmi_get_gpu_metrics_info(self._dev)
				clks = [c for c in (m.get("current_gfxclks") or []) if isinstance(c, (int, float)) and 0 < c < 60000]
				if clks:
					rec["sclk_mhz"] = sum(clks) / len(clks)
				for key in ("current_socket_power", "average_socket_power"):
					v = m.get(key)
					if isinstance(v, (int, float)) and 0 < v < 60000:
						rec["power_w"] = float(v)
						break
			except Exception:
				pass
		if "power_w" not in rec:
			import glob

			for f in glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"):
				try:
					rec["power_w"] = int(open(f).read()) / 1e6
					break
				except Exception:
					pass
		return rec

	def _run(self):
		while not self._stop.is_set():
			rec = self._sample()
			if rec:
				rec["t"] = time.perf_counter()
				self.samples.append(rec)
			self._stop.wait(self.period)

	def __enter__(self):
		self._thread.start()
		return self

	def __exit__(self, *_):
		self._stop.set()
		self._thread.join()

	def summary(self, t0, t1):
		"""Over the samples taken in [t0 + 20 % , t1] (the first fifth is left to the governor to settle)."""
		lo = t0 + 0.2 * (t1 - t0)
		out = {"samples": 0, "period_s": self.period, "power_cap_w": None}
		try:
			import glob

			out["power_cap_w"] = int(open(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap")[0]).read()) / 1e6
		except Exception:
			pass
		for key in ("sclk_mhz", "power_w"):
			vals = [r[key] for r in self.samples if key in r and lo <= r["t"] <= t1]
			if vals:
				out["samples"] = max(out["samples"], len(vals))
				out[key] = {"mean": sum(vals) / len(vals), "min": min(vals), "max": max(vals)}
		return out


def hbm_ceiling():
	"""What the memory system sustains for a plain read, copy and write of 1 GiB (elf_hbm_probe; 20 launches each after
	3 warm-ups, timed with one event pair): the practical ceiling the bandwidth-bound kernels are compared with."""
	import torch
	from elf_amd import _lib

	lib = _lib.load()
	n = 1 << 30
	src = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda")
	dst = torch.empty(n, dtype=torch.uint8, device="cuda")
	st = torch.cuda.current_stream().cuda_stream
	out = {"bytes": n, "peak_gbs": PEAK_HBM_GBS}
	# "read3_write1": three input streams of n / 4 bytes each and one output stream (a norm backward's pattern)
	for mode, name, size, moved in ((0, "read", n, n), (1, "copy", n, 2 * n), (2, "write", n, n), (3, "read3_write1", n // 4, n)):
		for _ in range(3):
			_lib.check(lib.elf_hbm_probe(mode, src.data_ptr(), dst.data_ptr(), size, st), "elf_hbm_probe")
		e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
		e0.record()
		for _ in range(20):
			_lib.check(lib.elf_hbm_probe(mode, src.data_ptr(), dst.data_ptr(), size, st), "elf_hbm_probe")
		e1.record()
		torch.cuda.synchronize()
		ms = e0.elapsed_time(e1) / 20
		out[name] = {"ms": ms, "gbs": moved / ms / 1e6, "frac_of_peak": moved / ms / 1e6 / PEAK_HBM_GBS}
	return out


def vendor_gemm(w, seconds=1.5):
	"""The twelve dense contractions of one block of the workload (forward y = x W^T, input gradient dX = dY W, weight
	gradient dW = dY^T X for each of the four projections), each run back to back for ``seconds`` through this library
	and through torch.matmul (the vendor's GEMM library), on the same operands and the same GPU, with socket power and
	shader clock sampled meanwhile.  A yardstick only: what another bf16 GEMM sustains on this part under its power cap."""
	import torch
	from elf_amd import kernels as K

	T, d, F = w["mb"] * w["seq"], w["d"], w["ffn"]
	nq, nkv = w["heads"] * w["head_dim"], w["kv_heads"] * w["head_dim"]
	shapes = [("qkv", nq + 2 * nkv, d), ("proj", d, nq), ("up", F * (2 if w["arch"] == "llama" else 1), d), ("down", d, F)]

	def sustained(fn, flops):
		t0 = time.perf_counter()
		while time.perf_counter() - t0 < 0.3 * seconds:  # untimed: lets the governor and the smoothed power reading settle
			for _ in range(25):
				fn()
			torch.cuda.synchronize()
		n, t0 = 0, time.perf_counter()
		with Telemetry(period=0.02) as tel:
			while time.perf_counter() - t0 < seconds:
				for _ in range(25):
					fn()
				torch.cuda.synchronize()
				n += 25
			t1 = time.perf_counter()
		summ = tel.summary(t0, t1)
		return {"tflops": flops * n / (t1 - t0) / 1e12, "us": (t1 - t0) / n * 1e6, "power_w": summ.get("power_w", {}).get("mean"), "sclk_mhz": summ.get("sclk_mhz", {}).get("mean")}

	rows, total = [], {"elf": 0.0, "vendor": 0.0}
	for name, N, Kd in shapes:
		x = torch.randn(T, Kd, device="cuda").bfloat16()
		wt = (torch.randn(N, Kd, device="cuda") * 0.02).bfloat16()
		dy = torch.randn(T, N, device="cuda").bfloat16()
		y, dx = torch.empty(T, N, device="cuda", dtype=torch.bfloat16), torch.empty(T, Kd, device="cuda", dtype=torch.bfloat16)
		dw32, dw16 = torch.zeros(N, Kd, device="cuda", dtype=torch.float32), torch.empty(N, Kd, device="cuda", dtype=torch.bfloat16)
		legs = (
			("forward", lambda: K.gemm(x, wt, out=y), lambda: torch.matmul(x, wt.t(), out=y)),
			("dX", lambda: K.gemm(dy, wt, b_t=True, out=dx), lambda: torch.matmul(dy, wt, out=dx)),
			# this library adds into the fp32 gradient; the vendor leg writes a bf16 product, which is less work
			("dW", lambda: K.gemm(dy, x, a_t=True, b_t=True, out=dw32, epilogue=K.EPI_F32_ACC), lambda: torch.matmul(dy.t(), x, out=dw16)),
		)
		for leg, ours, theirs in legs:
			r = {"gemm": f"{name}/{leg}", "M": T if leg != "dW" else N, "N": N if leg == "forward" else Kd, "K": Kd if leg == "forward" else (N if leg == "dX" else T)}
			r["elf"], r["vendor"] = sustained(ours, 2.0 * T * N * Kd), sustained(theirs, 2.0 * T * N * Kd)
			total["elf"] += r["elf"]["us"]
			total["vendor"] += r["vendor"]["us"]
			rows.append(r)
		del x, wt, dy, y, dx, dw32, dw16
	return {"seconds_per_leg": seconds, "gemms": rows, "sum_us": total}


def vendor_attention(w, repeats=20):
	"""The attention of one block at the workload's shape, forward and backward, through this library and through
	torch's scaled_dot_product_attention (the vendor's flash attention), same values, back to back.  A yardstick only."""
	import torch
	import torch.nn.functional as F
	from elf_amd import kernels as K

	B, S, Hq, Hkv, D, causal = w["mb"], w["seq"], w["heads"], w["kv_heads"], w["head_dim"], w["causal"]
	g = torch.Generator(device="cuda").manual_seed(3)
	qkv = torch.randn(B * S, (Hq + 2 * Hkv) * D, device="cuda", generator=g).bfloat16()
	do = torch.randn(B * S, Hq * D, device="cuda", generator=g).bfloat16()
	flops_f = (2.0 if causal else 4.0) * B * Hq * S * S * D

	def timed(fn):
		for _ in range(3):
			fn()
		torch.cuda.synchronize()
		t0 = time.perf_counter()
		for _ in range(repeats):
			fn()
		torch.cuda.synchronize()
		return (time.perf_counter() - t0) / repeats

	o, lse = K.attn_fwd(qkv, B, S, Hq, Hkv, D, causal)
	t_f = timed(lambda: K.attn_fwd(qkv, B, S, Hq, Hkv, D, causal))
	t_b = timed(lambda: K.attn_bwd(qkv, o, do, lse, B, S, Hq, Hkv, D, causal))
	out = {"shape": {"B": B, "S": S, "Hq": Hq, "Hkv": Hkv, "D": D, "causal": causal},
	       "elf": {"fwd_us": t_f * 1e6, "fwd_tflops": flops_f / t_f / 1e12, "bwd_us": t_b * 1e6, "bwd_tflops": 2 * flops_f / t_b / 1e12}}
	# [B, H, S, D] views of the same values for torch
	q, k, v = (t.view(B, S, -1, D).transpose(1, 2).contiguous().requires_grad_(True)
	           for t in (qkv[:, : Hq * D], qkv[:, Hq * D : (Hq + Hkv) * D], qkv[:, (Hq + Hkv) * D :]))
	do4 = do.view(B, S, Hq, D).transpose(1, 2).contiguous()
	try:
		fwd = lambda: F.scaled_dot_product_attention(q, k, v, is_causal=causal, enable_gqa=Hq != Hkv)
		t_vf = timed(fwd)

		def both():
			fwd().backward(do4)

		t_vfb = timed(both)
		out["vendor"] = {"fwd_us": t_vf * 1e6, "fwd_tflops": flops_f / t_vf / 1e12, "bwd_us": (t_vfb - t_vf) * 1e6, "bwd_tflops": 2 * flops_f / (t_vfb - t_vf) / 1e12}
	except Exception as e:  # no fused kernel for this shape in this torch build
		out["vendor"] = {"error": f"{type(e).__name__}: {e}"[:200]}
	return out


def main():
	ap = argparse.ArgumentParser()
	ap.add_argument("--gpus", type=int, default=1)
	ap.add_argument("--steps", type=int, default=3)
	ap.add_argument("--warmup", type=int, default=1)
	ap.add_argument("--workload", default="llama3_8b_zbh1", choices=sorted(WORKLOADS))
	ap.add_argument("--no-cpu-baseline", action="store_true")
	ap.add_argument("--prefetching-time", type=int, default=None,
	                help="offload workloads: how many compute ops before its B a micro-batch's PREFETCH_ACTIVATIONS is placed (reference default 1)")
	ap.add_argument("--time-one-in", type=int, default=None, metavar="N",
	                help="per-kernel figures (the roofline's among them) from HIP events carried by one launch in N of the timed steps, "
	                     "picked pseudo-randomly, the same picks every run (default 4, 16 for the GPT-2-small stream of 25 us kernels; "
	                     "1 = every launch: an event pair costs the stream about 2 us per launch, 0.5 %% of a Llama step and 8 %% of a "
	                     "GPT-2-small step)")
	ap.add_argument("--graph", action="store_true",
	                help="time replays of the step captured as one HIP graph (Engine.capture) instead of eager steps; the per-kernel figures "
	                     "then come from one extra eager step after the timed region (a replay runs no host code that could bracket launches)")
	ap.add_argument("--telemetry", action="store_true",
	                help="sample socket power and shader clock on a host thread during the timed steps and report them under \"telemetry\"")
	ap.add_argument("--hbm-ceiling", action="store_true",
	                help="also time a plain read / copy / write of 1 GiB (elf_hbm_probe) and report the rates under \"hbm_ceiling\"")
	ap.add_argument("--vendor-gemm", action="store_true",
	                help="also run the twelve GEMMs of one block back to back through this library and through torch.matmul (the vendor's "
	                     "library), with power and clock, and report both under \"vendor_gemm\"")
	ap.add_argument("--vendor-attention", action="store_true",
	                help="also time the block's attention, forward and backward, through this library and through torch's scaled_dot_product_attention, "
	                     "and report both under \"vendor_attention\"")
	ap.add_argument("--check", action="store_true",
	                help="after the timed region run the workload's stream and its plain counterpart (no remat rewrite / no offload / 1F1B for ZB-H1) once "
	                     "each on the same stage and report under \"check\" whether every output, input gradient and weight gradient agrees bit for bit")
	ap.add_argument("--calibration-copy", action="store_true",
	                help="also launch one elf::add_kernel over 2 x 128 MiB in, 128 MiB out: a kernel of known HBM traffic to scale profiler byte counters with")
	args = ap.parse_args()
	if args.gpus != 1:
		print("bench.py: this build runs one stage on ONE GPU; --gpus must be 1 (multi-GPU sharding is design-only).", file=sys.stderr)
		sys.exit(2)

	import torch
	from elf_amd import _lib
	from elf_amd.execution import Engine
	from elf_amd.synthetic import make_boundary

	if not torch.cuda.is_available():
		print("bench.py: no GPU visible; the stage kernels have no CPU path.", file=sys.stderr)
		sys.exit(1)
	lib = _lib.load()
	w = dict(WORKLOADS[args.workload])
	if args.time_one_in is None:
		args.time_one_in = w.get("time_one_in", 4)
	if args.prefetching_time is not None:
		w["prefetching_time"] = args.prefetching_time
	stage = build_stage(w)
	cpu_stats = None
	if not args.no_cpu_baseline:
		cpu_stats = cpu_baseline(w, stage)
	placement = w.get("placement", PLACEMENT)
	block = make_block(w, stage)
	xs, dys = make_boundary(w["mb"], w["seq"], w["d"], w["n_mb"], seed=1, device="cuda")
	block.set_boundary(inputs=xs, grads=dys)
	stream, remat = plan_stream(w, block)
	engine = Engine([block])
	mb_sizes = [w["mb"]] * w["n_mb"]

	def step():
		block.zero_grad()
		engine.train_step(None, None, None, stream, mb_sizes)

	if args.calibration_copy:
		from elf_amd import kernels
		n = 64 * 1024 * 1024
		ca = torch.ones(n, dtype=torch.bfloat16, device="cuda")
		cb = torch.ones(n, dtype=torch.bfloat16, device="cuda")
		kernels.add(ca, cb)
		torch.cuda.synchronize()
		del ca, cb
	for _ in range(args.warmup):
		step()
	torch.cuda.synchronize()
	eager_step = step
	if args.graph:
		graphed = engine.capture(None, None, None, stream, mb_sizes)

		def step():
			block.zero_grad()
			graphed.replay()

		step()
		torch.cuda.synchronize()
	else:
		lib.elf_prof_enable(args.time_one_in)
	mem_before = block.mem_stats()
	telemetry = Telemetry() if args.telemetry else contextlib.nullcontext()
	with telemetry:
		t0 = time.perf_counter()
		for _ in range(args.steps):
			step()
		torch.cuda.synchronize()
		elapsed = time.perf_counter() - t0
	if args.graph:
		lib.elf_prof_enable(1)  # one eager step outside the timed region, every launch timed
		eager_step()
		torch.cuda.synchronize()
	kinds = ["gemm", "attn_fwd", "attn_bwd", "norm_fwd", "norm_bwd", "act_fwd", "act_bwd", "rope", "grad_scale", "add", "embed", "loss"]
	per_kernel = {}
	for i, name in enumerate(kinds):
		ms, work = ctypes.c_double(), ctypes.c_double()
		n = lib.elf_prof_collect(i, ctypes.byref(ms), ctypes.byref(work))
		if n > 0:
			# the family's rate = work over duration of the launches that carried events; "launches" counts all launches and
			# "avg_ms" is their mean duration at that rate (all launches' work / rate / launches: with every launch timed,
			# the plain mean of the event durations)
			rate = work.value / (ms.value * 1e-3)
			all_work = ctypes.c_double()
			launches = lib.elf_prof_launches(i, ctypes.byref(all_work))
			per_kernel[name] = {"launches": launches, "timed_launches": n, "avg_ms": all_work.value / rate / launches * 1e3,
			                    "timed_ms": ms.value, ("tflops" if i < 3 else "gbs"): rate / (1e12 if i < 3 else 1e9)}
	lib.elf_prof_enable(0)
	mem = block.mem_stats()
	tokens = w["mb"] * w["seq"] * w["n_mb"]
	ms_per_step = elapsed / args.steps * 1e3
	g = per_kernel.get("gemm", {"tflops": 0.0, "launches": 0, "avg_ms": 0.0})
	out = {
		"metric": "stage tokens/sec (F+B+W) on 1 MI355X", "value": tokens / (elapsed / args.steps), "unit": "tokens/s", "n_gpus": 1,
		"steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
		"vs_baseline": None, "dtype": "bf16", "data": "synthetic",
		"config": {
			"workload": args.workload, "blocks": w["n_blocks"], "d_model": w["d"], "heads": w["heads"], "kv_heads": w["kv_heads"], "ffn": w["ffn"],
			"seq_len": w["seq"], "micro_batch": w["mb"], "n_micro_batches": w["n_mb"], "op_stream": f"{w['scheduler']} block {BLOCK_ID} of placement {placement}",
			"tokens_per_step": tokens, "ops_per_step": len(stream), "offload": bool(w.get("offload")), "hip_graph": bool(args.graph),
		},
		"roofline": {"bound": "mfma", "achieved": g["tflops"], "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": g["tflops"] / PEAK_BF16_TFLOPS, "traffic": gemm_traffic_bytes(args.workload),
		             "kernel": "elf::dma::gemm_pers_kernel / elf::dma::gemm_dma_kernel / elf::dma::gemm_dw_group_kernel / elf::gemm_kernel (bf16 MFMA GEMM, all layouts)", "launches": g["launches"], "avg_launch_ms": g["avg_ms"]},
		"stream_mfu": stream_flops(w) / (elapsed / args.steps) / (PEAK_BF16_TFLOPS * 1e12),
		"kernels": per_kernel,
		"peak_stage_memory_bytes": mem["peak_bytes"] + mem["workspace_bytes"] + torch.cuda.max_memory_allocated(),
		"workspace_bytes": mem["workspace_bytes"],
		"stash_peak_bytes": mem["peak_bytes"], "offload_d2h_bytes": mem["d2h_bytes"], "offload_h2d_bytes": mem["h2d_bytes"],
	}
	if remat is not None:
		out["remat"] = remat
	if w.get("offload"):
		# bytes moved by the side-stream copies of the timed steps over the steps' wall time: the
		# rate the host link sustained while overlapped with the kernels (both directions at once)
		d2h = mem["d2h_bytes"] - mem_before["d2h_bytes"]
		h2d = mem["h2d_bytes"] - mem_before["h2d_bytes"]
		out["host_link"] = {"d2h_gbs": d2h / elapsed / 1e9, "h2d_gbs": h2d / elapsed / 1e9, "d2h_bytes_per_step": d2h / args.steps,
		                    "h2d_bytes_per_step": h2d / args.steps, "prefetching_time": w.get("prefetching_time", 1)}
	if args.telemetry:
		out["telemetry"] = telemetry.summary(t0, t0 + elapsed)
	if args.hbm_ceiling:
		out["hbm_ceiling"] = hbm_ceiling()
	if args.vendor_gemm:
		out["vendor_gemm"] = vendor_gemm(w)
	if args.vendor_attention:
		out["vendor_attention"] = vendor_attention(w)
	if cpu_stats is not None:
		out["cpu_baseline"] = cpu_stats
	if args.check:
		out["check"] = check_stream(w, block, engine, stream, mb_sizes, xs, dys)
	print(json.dumps(out))
	if args.check and not out["check"]["ok"]:
		sys.exit(3)


if __name__ == "__main__":
	main()
