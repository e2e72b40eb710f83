"""TEST INFRASTRUCTURE ONLY — CPU restatement of the last stage's loss; never imported by the product.

``cross_entropy_ref`` follows the reference transformer's loss function
(benchmarks/models/simple.py:520-524): upcast the logits to fp32, flatten all leading dimensions,
``torch.nn.functional.cross_entropy``.  ``compute_loss_ref`` follows ``Engine.compute_loss``
(elf/execution/engine.py:374-410): the sum-reduced loss divided by the elements per sample, and its
gradient with respect to the (bf16) stage output through autograd.

Pinned by tests/test_oracle_cpu.py against the closed form -log softmax(x)[target] evaluated with
fp64 Python loops on small inputs (sum / mean / none reductions, ignored rows).
"""

import torch
import torch.nn.functional as F


def cross_entropy_ref(pred, target, reduction="mean", ignore_index=-100):
	V = pred.shape[-1]
	return F.cross_entropy(pred.to(torch.float32).reshape(-1, V), target.reshape(-1), reduction=reduction, ignore_index=ignore_index)


def compute_loss_ref(output, target, ignore_index=-100):
	"""(loss, gradient w.r.t. ``output`` in its dtype) of one micro-batch as the engine computes them."""
	out = output.detach().clone().requires_grad_()
	loss = cross_entropy_ref(out, target, reduction="sum", ignore_index=ignore_index) / (target.numel() // target.size(0))
	loss.backward()
	return loss.detach(), out.grad
