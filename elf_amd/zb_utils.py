"""The split-backward operator plug-in of the reference (elf/zb_utils.py) on the HIP GEMM.

``LinearDX`` / ``LayerDW`` / ``LinearDW`` / ``MappingDW`` / ``replace_layer_with_layer_dw`` keep the
reference's names, queues and call order (elf/zb_utils.py:9-40, 43-194, 198-256, 487-513):

* forward   ``LinearDX.forward``  : Y = X W^T (+ b) and the input is stashed  -> ``elf_gemm_bf16`` (A, B k-contiguous)
* B         ``LinearDX.backward`` : the incoming gradient is stashed (summed when the module is used
                                    several times) and dX = dY W is returned    -> ``elf_gemm_bf16`` (B reduction-major)
* W         ``LinearDW.backward`` : dW += dY^T X, db += sum_t dY                -> ``elf_gemm_bf16`` (both reduction-major,
                                    fp32 ``C +=``) and ``elf_colsum_bf16``

Differences from the reference, both on purpose: gradients accumulate in fp32 buffers
(``weight.main_grad`` / ``bias.main_grad``; ``weight.grad`` is only written by a block's ``scale_grads``)
instead of in the parameter dtype, and there is no other execution path: the layer must be bf16 on
the GPU with ``in_features`` and ``out_features`` multiples of 64, and the tokens of a call a
multiple of 64 (the GEMM's tile constraints) - anything else raises.
"""

import torch
import torch.nn as nn

from . import _lib, kernels

__all__ = ["LinearDX", "LayerDW", "LinearDW", "MappingDW", "replace_layer_with_layer_dw", "replace_linear_with_linear_dw"]


def _as_rows(t):
	"""[..., C] -> contiguous [rows, C] view (a copy only if the layout forces one)."""
	t2 = t.reshape(-1, t.shape[-1])
	return t2 if t2.is_contiguous() else t2.contiguous()


class LinearDX(torch.autograd.Function):
	"""y = linear(x) whose backward only computes the input gradient (elf/zb_utils.py:9-40)."""

	@staticmethod
	def forward(ctx, input, weight, bias, linear):
		ctx.linear = linear
		linear._store_input(input)
		ctx.save_for_backward(input.detach())  # marks the input as needed by the backward, so that torch.utils.checkpoint recomputes it
		x = _as_rows(input)
		if bias is not None:
			y = kernels.gemm(x, weight, epilogue=kernels.EPI_BF16_RESID, residual=bias.reshape(1, -1).expand(1, weight.shape[0]), residual_ld=0)
		else:
			y = kernels.gemm(x, weight)
		return y.view(*input.shape[:-1], weight.shape[0])

	@staticmethod
	def backward(ctx, grad_output):
		linear = ctx.linear
		linear._accumulate_grad_output(grad_output)
		go = _as_rows(grad_output)
		grad_input = kernels.gemm(go, linear.weight.detach(), b_t=True)  # dY [T, out] x W [out, in] with W read as it lies
		return grad_input.view(*grad_output.shape[:-1], linear.weight.shape[1]), None, None, None


class LayerDW:
	"""Mixin for modules whose backward is split: an autograd function that only produces the input
	gradient and stashes what the parameter gradient needs, and ``backward(mb_id)`` that consumes the
	stash (elf/zb_utils.py:43-194).  ``ctx["input"]`` / ``ctx["grad_output"]`` are per-micro-batch lists."""

	_dx_function_registry = {}

	def __init__(self, *args, **kwargs):
		with torch.device("meta"):  # the tensors are replaced by the wrapped layer's right away
			super().__init__(*args, **kwargs)
		self.ctx = {"input": [], "grad_output": []}
		self.last_input = None
		self.last_grad_output = None

	@classmethod
	def register_dx_function(cls, dx_class):
		cls._dx_function_registry[cls] = dx_class
		return dx_class

	def backward(self, mb_id):
		raise NotImplementedError("Subclasses must implement backward()")

	def clear(self):
		self.ctx["input"].clear()
		self.ctx["grad_output"].clear()
		self.last_input = None
		self.last_grad_output = None

	def is_empty(self, queue):
		return all(x is None for x in self.ctx[queue])

	def _state(self):
		return f"({sum(x is not None for x in self.ctx['input'])},{sum(x is not None for x in self.ctx['grad_output'])})"

	def _store_input(self, input):
		self.last_input = input.detach()
		# an input without a grad_fn is the stage's own input: checkpointing will not recompute it, so the
		# remat logic must not drop it
		setattr(self.last_input, "is_model_input", input.grad_fn is None)

	def _accumulate_grad_output(self, grad_output):
		if getattr(self, "last_grad_output", None) is None:
			self.last_grad_output = grad_output
		else:
			self.last_grad_output = self.last_grad_output + grad_output

	def set(self, queue, idx, value):
		values = self.ctx[queue]
		if len(values) <= idx:
			values.extend([None] * (idx - len(values) + 1))
		if values[idx] is not None:
			raise ValueError(f"{queue} at index {idx} already set")
		values[idx] = value

	def delete(self, queue, idx):
		values = self.ctx[queue]
		if idx >= len(values) or values[idx] is None:
			raise ValueError(f"{queue} at index {idx} not set")
		values[idx] = None

	def move_last_computed(self, queue, idx):
		last_value = getattr(self, f"last_{queue}", None)
		if last_value is None:
			return  # a sub-module the forward did not use
		self.set(queue, idx, last_value)
		setattr(self, f"last_{queue}", None)

	def offload_last(self, idx, to="cpu"):
		with torch.no_grad():
			self.ctx["grad_output"][idx] = self.ctx["grad_output"][idx].to(to, non_blocking=True)
			self.ctx["input"][idx] = self.ctx["input"][idx].to(to, non_blocking=True)


class LinearDW(LayerDW, nn.Linear):
	"""``nn.Linear`` with the split backward (elf/zb_utils.py:198-256), sharing the wrapped layer's
	parameters.  Call order: LinearDW.forward -> LinearDX.forward -> LinearDX.backward -> LinearDW.backward."""

	def __init__(self, linear, *args, **kwargs):
		if linear.in_features % 64 or linear.out_features % 64:
			raise _lib.ElfStageError(f"LinearDW: in_features and out_features must be multiples of 64 for the HIP GEMM, got {linear.in_features} -> {linear.out_features}")
		super().__init__(linear.in_features, linear.out_features, linear.bias is not None, *args, **kwargs)
		self.weight = linear.weight
		if linear.bias is not None:
			self.bias = linear.bias

	def _check(self, x):
		if x.dtype != torch.bfloat16 or not x.is_cuda or self.weight.dtype != torch.bfloat16 or not self.weight.is_cuda:
			raise _lib.ElfStageError(f"LinearDW: bf16 tensors on the GPU only (input {x.dtype} on {x.device}, weight {self.weight.dtype} on {self.weight.device})")
		if (x.numel() // x.shape[-1]) % 64:
			raise _lib.ElfStageError(f"LinearDW: the number of tokens of a call must be a multiple of 64, got input {tuple(x.shape)}")

	def forward(self, x, *args, **kwargs):
		self._check(x)
		return LinearDX.apply(x, self.weight, self.bias, self, *args, **kwargs)

	def _main_grad(self, param):
		g = getattr(param, "main_grad", None)
		if g is None:
			g = torch.zeros(param.shape, dtype=torch.float32, device=param.device)
			param.main_grad = g
		return g

	def backward(self, mb_id):
		"""W: main_grad += dY^T X (fp32), bias main_grad += sum over tokens of dY; drops the stash."""
		grad_output = self.ctx["grad_output"][mb_id]
		inputs = self.ctx["input"][mb_id]
		go, inp = _as_rows(grad_output), _as_rows(inputs)
		kernels.gemm(go, inp, a_t=True, b_t=True, out=self._main_grad(self.weight), epilogue=kernels.EPI_F32_ACC)
		if self.bias is not None:
			kernels.colsum_(go, self._main_grad(self.bias))
		self.ctx["grad_output"][mb_id] = None
		self.ctx["input"][mb_id] = None


LinearDW.register_dx_function(LinearDX)

# module class -> its split-backward replacement (the reference also maps nn.Conv1d; convolutions are not
# part of the transformer-stage path this build covers)
MappingDW = {nn.Linear: LinearDW}


def replace_layer_with_layer_dw(model, only=None):
	"""Replace, in place, every module whose class is in ``MappingDW`` by its split-backward
	equivalent (elf/zb_utils.py:490-513)."""
	for name, module in list(model.named_modules()):
		if type(module) in MappingDW and not isinstance(module, LayerDW) and (only is None or type(module) in only):
			parent = model if "." not in name else model.get_submodule(name[: name.rfind(".")])
			setattr(parent, name.split(".")[-1], MappingDW[type(module)](module))


def replace_linear_with_linear_dw(model, device=None):
	"""Older name of ``replace_layer_with_layer_dw(model, only=[nn.Linear])`` (elf/zb_utils.py:449-485)."""
	replace_layer_with_layer_dw(model, only=[nn.Linear])
