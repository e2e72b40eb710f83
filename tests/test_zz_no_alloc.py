"""The norm backward entry point that allocates nothing (its partial sums go to an array of the library's
device image) against the entry point with a caller-supplied workspace, through the C ABI: two calls in a
row on the shared array, the second on a smaller input, for both norm kinds and both row layouts
(d <= 2048: one wave per row; above: one workgroup per row).  Everything is bit-identical: the same kernels
on the same operands, and the gamma / beta gradients are folded in a fixed order by one writer per column."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(K, kind, T, d, seed, with_dres):
	g = torch.Generator(device="cuda").manual_seed(seed)
	rnd = lambda *shape: torch.randn(*shape, generator=g, device="cuda")
	x = (rnd(T, d) * 2 + 0.5).to(torch.bfloat16)
	dy = rnd(T, d).to(torch.bfloat16)
	dres = rnd(T, d).to(torch.bfloat16) if with_dres else None
	gamma = (1 + 0.1 * rnd(d)).to(torch.bfloat16)
	beta = (0.1 * rnd(d)).to(torch.bfloat16) if kind == K.NORM_LAYER else None
	_, stats = K.norm_fwd(kind, x, gamma, beta)
	want_dg = torch.full((d,), 0.25, dtype=torch.float32, device="cuda")  # the accumulators are added to
	want_db = torch.full((d,), -0.5, dtype=torch.float32, device="cuda") if kind == K.NORM_LAYER else None
	got_dg, got_db = want_dg.clone(), (want_db.clone() if want_db is not None else None)
	want_dx = K.norm_bwd(kind, dy, x, gamma, stats, want_dg, want_db, dres)
	got_dx = torch.empty_like(x)
	K.norm_bwd_noalloc(kind, dy, x, gamma, stats, got_dg, got_dx, got_db, dres)
	torch.cuda.synchronize()
	assert torch.equal(got_dx, want_dx), f"dx differs (kind {kind}, T {T}, d {d})"
	for got, want, what in ((got_dg, want_dg, "dgamma"), (got_db, want_db, "dbeta")):
		if want is not None:
			assert torch.equal(got, want), f"{what} (kind {kind}, T {T}, d {d})"
	# and against fp32 torch, so that both entry points being wrong together would show
	xf = x.float().requires_grad_(True)
	gf = gamma.float().requires_grad_(True)
	if kind == K.NORM_LAYER:
		bf = beta.float().requires_grad_(True)
		y = torch.nn.functional.layer_norm(xf, (d,), gf, bf, 1e-5)
	else:
		y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5) * gf
	y.backward(dy.float())
	ref_dx = xf.grad + (dres.float() if dres is not None else 0)
	assert (got_dx.float() - ref_dx).abs().max().item() <= 2e-2 * ref_dx.abs().max().item()
	assert ((got_dg - 0.25) - gf.grad).abs().max().item() <= 2e-2 * gf.grad.abs().max().item()


def test_norm_bwd_noalloc_matches_norm_bwd_on_two_calls_in_a_row():
	from elf_amd import kernels as K

	for kind in (K.NORM_RMS, K.NORM_LAYER):
		# large first, then smaller: the second call finds the first call's partial sums in the shared array
		for T, d, with_dres in ((8192, 4096, True), (1000, 768, False), (4096, 8192, True), (64, 256, True)):
			print(f"[case] norm_bwd_noalloc kind={kind} T={T} d={d} dres={with_dres}", flush=True)
			_case(K, kind, T, d, seed=T + d, with_dres=with_dres)


def test_norm_bwd_noalloc_refuses_what_the_array_cannot_hold():
	from elf_amd import _lib, kernels as K

	x = torch.zeros(4, 16384, dtype=torch.bfloat16, device="cuda")
	st = torch.zeros(4, 2, dtype=torch.float32, device="cuda")
	g = torch.ones(16384, dtype=torch.bfloat16, device="cuda")
	dg = torch.zeros(16384, dtype=torch.float32, device="cuda")
	with pytest.raises(_lib.ElfStageError):
		K.norm_bwd_noalloc(K.NORM_RMS, x, x, g, st, dg, torch.empty_like(x))


def _inputs(K, kind, T, d, seed):
	g = torch.Generator(device="cuda").manual_seed(seed)
	rnd = lambda *shape: torch.randn(*shape, generator=g, device="cuda")
	x = (rnd(T, d) * 2 + 0.5).to(torch.bfloat16)
	dy = rnd(T, d).to(torch.bfloat16)
	gamma = (1 + 0.1 * rnd(d)).to(torch.bfloat16)
	_, stats = K.norm_fwd(kind, x, gamma, None)
	return x, dy, gamma, stats


def test_norm_bwd_noalloc_takes_no_device_memory():
	"""What the entry point exists for: across a call neither torch's allocator nor the driver's free-memory
	figure moves (after one earlier call on the device, which looks the array's address up)."""
	from elf_amd import kernels as K

	T, d = 4096, 4096
	x, dy, gamma, stats = _inputs(K, K.NORM_RMS, T, d, 5)
	dg, dx = torch.zeros(d, dtype=torch.float32, device="cuda"), torch.empty_like(x)
	K.norm_bwd_noalloc(K.NORM_RMS, dy, x, gamma, stats, dg, dx)
	torch.cuda.synchronize()
	allocated, reserved, free = torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]
	for _ in range(3):
		K.norm_bwd_noalloc(K.NORM_RMS, dy, x, gamma, stats, dg, dx)
	torch.cuda.synchronize()
	assert torch.cuda.memory_allocated() == allocated and torch.cuda.memory_reserved() == reserved
	assert torch.cuda.mem_get_info()[0] == free, "the driver's free memory moved across elf_norm_bwd_noalloc"


def test_norm_bwd_noalloc_under_graph_capture():
	"""Captured into a HIP graph (where hipMalloc is not allowed) and replayed three times with eager work and
	synchronisations in between; every replay equals the eager call bit for bit."""
	from elf_amd import kernels as K

	T, d = 2048, 4096
	x, dy, gamma, stats = _inputs(K, K.NORM_RMS, T, d, 6)
	want_dg = torch.zeros(d, dtype=torch.float32, device="cuda")
	want_dx = torch.empty_like(x)
	K.norm_bwd_noalloc(K.NORM_RMS, dy, x, gamma, stats, want_dg, want_dx)  # eager; also the first call on the device
	torch.cuda.synchronize()
	dg, dx = torch.zeros(d, dtype=torch.float32, device="cuda"), torch.empty_like(x)
	graph = torch.cuda.CUDAGraph()
	with torch.cuda.graph(graph):
		K.norm_bwd_noalloc(K.NORM_RMS, dy, x, gamma, stats, dg, dx)
	for replay in range(3):
		dg.zero_()
		dx.fill_(7.0)
		# eager work on the shared array between the replays: another shape leaves other partial sums in it
		x2, dy2, g2, st2 = _inputs(K, K.NORM_RMS, 512, 1024, 70 + replay)
		K.norm_bwd_noalloc(K.NORM_RMS, dy2, x2, g2, st2, torch.zeros(1024, dtype=torch.float32, device="cuda"), torch.empty_like(x2))
		torch.cuda.synchronize()
		graph.replay()
		torch.cuda.synchronize()
		assert torch.equal(dx, want_dx) and torch.equal(dg, want_dg), f"replay {replay} differs from the eager call"
