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
