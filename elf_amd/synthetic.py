"""Seeded synthetic stage-boundary data: what a stage would receive from its pipeline peers."""

import torch

__all__ = ["make_boundary"]


def make_boundary(mb, seq, d_model, n_mb, seed=1, dtype=torch.bfloat16, device=None):
	"""N(0,1) incoming activations X[m] and incoming gradients dY[m], each [mb, seq, d_model], one
	independent draw per micro-batch from a CPU generator (so that a CPU run and a GPU run see
	identical bits), first all X then all dY."""
	g = torch.Generator(device="cpu").manual_seed(seed)
	shape = (mb, seq, d_model)
	xs = [torch.randn(shape, generator=g).to(dtype) for _ in range(n_mb)]
	dys = [torch.randn(shape, generator=g).to(dtype) for _ in range(n_mb)]
	if device is not None:
		xs, dys = [x.to(device) for x in xs], [d.to(device) for d in dys]
	return xs, dys
