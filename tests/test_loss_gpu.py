"""The one-kernel cross-entropy of a last stage (elf_cross_entropy) against the CPU oracle
(oracle/loss_ref.py: fp32 torch.nn.functional.cross_entropy on the upcast logits, as
benchmarks/models/simple.py:520-524).  Tolerances: per-row loss rel 1e-5 / abs 2e-5 (fp32 arithmetic
on identical bf16 inputs; only the summation order differs); gradient within one bf16 rounding of
the fp32 gradient (rel 2^-7 of the element, abs 1e-6 of the scale)."""

import pytest
import torch

from oracle import loss_ref as L

pytestmark = pytest.mark.gpu


def _case(rows, V, seed, ld=None, spread=4.0):
	g = torch.Generator().manual_seed(seed)
	x = (torch.randn(rows, V, generator=g) * spread).to(torch.bfloat16)
	t = torch.randint(0, V, (rows,), generator=g)
	t[::7] = -100
	t[1] = V - 1
	t[2] = 0
	if ld is None:
		return x, t, x.cuda()
	buf = torch.full((rows, ld), float("nan"), dtype=torch.bfloat16).cuda()  # what lies between rows must not matter
	buf[:, :V] = x.cuda()
	return x, t, buf[:, :V]


def _check_grad(got, want_f32, scale):
	got, want = got.float().cpu(), want_f32
	err = (got - want).abs()
	assert bool((err <= want.abs() * 2.0**-7 + 1e-6 * scale).all()), f"max err {err.max().item():.3e}"


# (rows, V, row stride): wave per row (two register depths), 4 / 16 waves per row, 16 chunks per lane,
# the two-read kernel for rows beyond the register budget, V not a multiple of 8 (padded copy), tiny rows
@pytest.mark.parametrize("rows,V,ld", [(37, 1000, 1024), (64, 1000, None), (16, 50257, None), (33, 4096, 4096), (9, 16384, 16400), (5, 65536, None), (6, 128256, None), (3, 150001, None), (3, 200000, None), (3, 8, None), (5, 3, None)])
def test_cross_entropy_loss_and_gradient(rows, V, ld):
	from elf_amd import losses

	x, t, xg = _case(rows, V, seed=rows + V, ld=ld)
	tg = t.cuda()
	want_rows = L.cross_entropy_ref(x, t, "none")
	for reduction in ("none", "sum", "mean"):
		got = losses.cross_entropy(xg, tg, reduction=reduction)
		want = L.cross_entropy_ref(x, t, reduction)
		assert torch.allclose(got.cpu(), want, rtol=1e-5, atol=2e-5 * (1 if reduction != "sum" else rows)), reduction
	# gradient, scaled in the kernel
	xf = x.float().requires_grad_()
	L.cross_entropy_ref(xf, t, "sum").backward()
	scale = 1.0 / 128
	loss, grad = losses.cross_entropy.loss_and_grad(xg, tg, reduction="sum", scale=scale)
	assert float(loss) == pytest.approx(float(want_rows.sum()), rel=1e-5)
	assert tuple(grad.shape) == (rows, V) and grad.stride(0) % 64 == 0
	_check_grad(grad, xf.grad * scale, scale)
	assert grad[t == -100].abs().max().item() == 0
	base = torch.as_strided(grad, (rows, grad.stride(0)), (grad.stride(0), 1))
	assert base[:, V:].abs().sum().item() == 0  # padding columns are zeros
	# mean: divides by the live rows, through autograd with an upstream factor
	xa = xg.detach().clone().requires_grad_()
	(losses.cross_entropy(xa, tg) * 3.0).backward()
	live = int((t != -100).sum())
	_check_grad(xa.grad, xf.grad * (3.0 / live), 3.0 / live)


def test_cross_entropy_rejects_what_it_cannot_run_and_flags_bad_targets():
	from elf_amd import _lib, losses

	x = torch.randn(4, 16).to(torch.bfloat16).cuda()
	t = torch.tensor([1, 2, 99, -100]).cuda()
	got = losses.cross_entropy(x, t, reduction="none")
	assert torch.isnan(got[2]) and not torch.isnan(got[[0, 1, 3]]).any() and got[3].item() == 0
	with pytest.raises(_lib.ElfStageError):
		losses.cross_entropy(x.float(), t)
	with pytest.raises(_lib.ElfStageError):
		losses.cross_entropy(x, t.int())
	with pytest.raises(_lib.ElfStageError):
		losses.cross_entropy(x.cpu(), t.cpu())
	with pytest.raises(ValueError):
		losses.cross_entropy(x, t, reduction="max")


def test_engine_compute_loss_takes_the_one_kernel_path():
	"""Engine.compute_loss with the library loss equals the oracle's restatement of the reference's
	compute_loss (sum over the micro-batch / elements per sample, gradient in bf16)."""
	from elf_amd import losses
	from elf_amd.execution.engine import compute_loss

	class _Block:
		compute_time = []

	mb, S, V = 4, 128, 1000
	g = torch.Generator().manual_seed(5)
	buf = (torch.randn(mb, S, 1024, generator=g) * 3).to(torch.bfloat16).cuda()
	out = buf[..., :V]  # the view a last stage hands out
	tgt = torch.randint(0, V, (mb, S), generator=g)
	want_loss, want_grad = L.compute_loss_ref(out.cpu(), tgt)
	loss, grad_fn = compute_loss(_Block, out, tgt.cuda(), losses.cross_entropy)
	(grad,) = grad_fn()
	assert float(loss) == pytest.approx(float(want_loss), rel=1e-5)
	assert not loss.requires_grad and grad.shape == out.shape
	xf = out.cpu().float().requires_grad_()
	(L.cross_entropy_ref(xf, tgt, "sum") / S).backward()
	_check_grad(grad, xf.grad, 1.0 / S)
	assert torch.equal(grad.cpu(), want_grad) or (grad.cpu().float() - want_grad.float()).abs().max().item() <= 2.0**-7 / S
