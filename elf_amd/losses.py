"""Loss functions of a pipeline's last stage that run as one HIP kernel.

``cross_entropy`` has the call shape ``Engine.compute_loss`` uses for ``loss_fn`` —
``loss_fn(output, target, reduction="sum")`` (elf/execution/engine.py:374-410) — and the semantics of
the reference transformer's loss (benchmarks/models/simple.py:520-524): logits flattened to
``[rows, V]``, arithmetic in fp32, ``torch.nn.functional.cross_entropy`` reductions and
``ignore_index``.  Loss and gradient come out of a single pass over the logits; there is no CPU path.
"""

import torch

from . import _lib

_PAD = 64  # gradient rows are padded to this many columns, the layout the stage's head GEMM reads


def _stream():
	return torch.cuda.current_stream().cuda_stream


def _rows_view(pred, V):
	"""``pred`` as (tensor whose memory the kernel reads, row stride) without copying when its rows are
	evenly strided and 16-byte aligned; otherwise a padded contiguous copy."""
	if pred.dtype != torch.bfloat16 or not pred.is_cuda:
		raise _lib.ElfStageError(f"cross_entropy: logits must be a bf16 GPU tensor, got {pred.dtype} on {pred.device}")
	if pred.shape[-1] != V:
		raise _lib.ElfStageError("cross_entropy: the last dimension of the logits must be the class dimension")
	p = pred if pred.dim() >= 2 else pred.unsqueeze(0)
	ld = p.stride(-2)
	ok = p.stride(-1) == 1 and ld % 8 == 0 and ld >= V and p.data_ptr() % 16 == 0
	expect = ld
	for size, stride in zip(reversed(p.shape[:-1]), reversed(p.stride()[:-1])):
		ok = ok and (size == 1 or stride == expect)
		expect *= size
	if ok:
		return p, ld
	ld = -(-V // 8) * 8
	buf = torch.zeros(p.numel() // V, ld, dtype=torch.bfloat16, device=pred.device)
	buf[:, :V] = p.reshape(-1, V)
	return buf, ld


def _check_target(target, rows):
	if target.dtype != torch.int64 or not target.is_cuda or target.numel() != rows:
		raise _lib.ElfStageError(f"cross_entropy: target must be an int64 GPU tensor of {rows} class indices (probabilities are not supported), got {tuple(target.shape)} {target.dtype} on {target.device}")
	return target.contiguous().view(-1)


def _run(pred, target, *, ignore_index, scale, mean, want_grad):
	"""(row_loss fp32 [rows], out2 = [sum, count] fp32, grad [rows, ld_out] bf16 or None)."""
	V = pred.shape[-1]
	src, ld = _rows_view(pred, V)
	rows = pred.numel() // V
	target = _check_target(target, rows)
	lib = _lib.load()
	dev = pred.device
	row_loss = torch.empty(rows, dtype=torch.float32, device=dev)
	out2 = torch.empty(2, dtype=torch.float32, device=dev)
	grad, ld_out, div = None, 0, None
	if mean:  # the gradient divides by the number of live rows, which only depends on the target
		_lib.check(lib.elf_cross_entropy_reduce(None, target.data_ptr(), rows, ignore_index, out2.data_ptr(), _stream()), "elf_cross_entropy_reduce")
		div = out2[1:]
	if want_grad:
		ld_out = -(-V // _PAD) * _PAD
		grad = torch.empty(rows, ld_out, dtype=torch.bfloat16, device=dev)
	_lib.check(
		lib.elf_cross_entropy(src.data_ptr(), ld, target.data_ptr(), rows, V, ignore_index, scale, div.data_ptr() if div is not None else None,
			row_loss.data_ptr(), grad.data_ptr() if grad is not None else None, ld_out, _stream()),
		"elf_cross_entropy",
	)
	_lib.check(lib.elf_cross_entropy_reduce(row_loss.data_ptr(), target.data_ptr(), rows, ignore_index, out2.data_ptr(), _stream()), "elf_cross_entropy_reduce")
	return row_loss, out2, grad


def _reduced(row_loss, out2, reduction, shape):
	if reduction == "sum":
		return out2[0].clone()
	if reduction == "mean":
		return out2[0] / out2[1]
	if reduction == "none":
		return row_loss.view(shape)
	raise ValueError(f"{reduction} is not a valid value for reduction")


class _CrossEntropy(torch.autograd.Function):
	@staticmethod
	def forward(ctx, pred, target, reduction, ignore_index):
		row_loss, out2, grad = _run(pred, target, ignore_index=ignore_index, scale=1.0, mean=reduction == "mean", want_grad=ctx.needs_input_grad[0])
		ctx.grad, ctx.shape, ctx.per_row = grad, pred.shape, reduction == "none"
		return _reduced(row_loss, out2, reduction, pred.shape[:-1])

	@staticmethod
	def backward(ctx, g):
		V = ctx.shape[-1]
		grad = ctx.grad[:, :V]
		grad = grad * (g.reshape(-1, 1) if ctx.per_row else g).to(grad.dtype)
		return grad.view(ctx.shape), None, None, None


def cross_entropy(pred, target, reduction="mean", ignore_index=-100):
	"""Drop-in for ``torch.nn.functional.cross_entropy(pred.float().view(-1, V), target.view(-1))`` on
	bf16 GPU logits ``[..., V]`` and int64 class indices ``[...]``; differentiable w.r.t. ``pred``."""
	if pred.requires_grad and torch.is_grad_enabled():
		return _CrossEntropy.apply(pred, target, reduction, ignore_index)
	row_loss, out2, _ = _run(pred, target, ignore_index=ignore_index, scale=1.0, mean=reduction == "mean", want_grad=False)
	return _reduced(row_loss, out2, reduction, pred.shape[:-1])


def _loss_and_grad(pred, target, reduction="sum", ignore_index=-100, scale=1.0):
	"""The loss and ``scale`` times its gradient w.r.t. ``pred`` from one kernel, without autograd.
	``Engine.compute_loss`` calls this when the loss function offers it.  The gradient is a view of a
	``[rows, V rounded up to 64]`` buffer whose extra columns are zero: the layout a last stage reads
	in place."""
	if reduction not in ("sum", "mean"):
		raise ValueError("loss_and_grad needs a scalar loss: reduction must be 'sum' or 'mean'")
	row_loss, out2, grad = _run(pred, target, ignore_index=ignore_index, scale=scale, mean=reduction == "mean", want_grad=True)
	V = pred.shape[-1]
	return _reduced(row_loss, out2, reduction, None), grad.view(*pred.shape[:-1], -1)[..., :V]


cross_entropy.loss_and_grad = _loss_and_grad
