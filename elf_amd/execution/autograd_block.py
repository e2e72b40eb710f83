"""Stage executor for any ``nn.Module``: the reference's PipelineBlock compute ops
(elf/execution/block.py:210-391, 624-694) as the reference runs them - the module's own forward under
autograd - with every ``nn.Linear`` swapped for ``LinearDW`` (elf_amd.zb_utils), so that the dense
contractions of F, B (input gradients only) and W (deferred weight gradients, fp32 accumulation) run on
the HIP GEMM of libelf_stage.so.  Everything that is not a linear layer is executed by PyTorch.

It is what ``Pipeline`` builds for a stage that is not a chain of ``TransformerBlock`` / ``LlamaBlock``
modules (those run entirely inside the library through ``HipStageBlock``), and it accepts stages with
several inputs and outputs.  There is no CPU path: construction needs the GPU and the library.
"""

import logging
from contextlib import contextmanager

import torch
from torch.utils.checkpoint import checkpoint

from .. import _lib
from ..scheduling import OpOptions
from ..zb_utils import LayerDW, replace_layer_with_layer_dw
from .block import StageBlockBase

logger = logging.getLogger("block")

__all__ = ["AutogradStageBlock"]


class AutogradStageBlock(StageBlockBase):
	def __init__(self, model, id_, placement, signature, pp_group=None, dp_group=None, recv_pgs=None, send_pgs=None, **_unused):
		if not torch.cuda.is_available():
			raise _lib.ElfStageError("AutogradStageBlock needs an MI355X: its linear layers run on the HIP GEMM")
		_lib.load()
		self._init_common(model, id_, placement, signature, pp_group, dp_group, recv_pgs, send_pgs)
		replace_layer_with_layer_dw(self.model)
		logger.info(f"{self}: generic stage ({type(model).__name__}): linear layers on the HIP GEMM, the rest through PyTorch autograd")

	def _layers_dw(self):
		return [m for m in self.model.modules() if isinstance(m, LayerDW)]

	# ------------------------------------------------------------------ remat (elf/execution/remat.py:26-74)
	@contextmanager
	def _selective_remat(self, strategy, mb_id):
		picked = [m for n, m in self.model.named_modules() if strategy(n, m)]
		restore = []
		for module in picked:
			original = module.forward
			restore.append(("forward" in module.__dict__, module.__dict__.get("forward")))

			def wrapped(*args, _original=original, **kwargs):
				return checkpoint(_original, *args, **kwargs, use_reentrant=False)

			module.forward = wrapped
		try:
			yield
		finally:
			for module, (had_own, own) in zip(picked, restore):
				# stashed inputs that the checkpoint will produce again are not kept
				for sub in module.modules():
					if isinstance(sub, LayerDW) and len(sub.ctx["input"]) > mb_id and sub.ctx["input"][mb_id] is not None and not getattr(sub.ctx["input"][mb_id], "is_model_input", False):
						sub.delete("input", mb_id)
				if had_own:
					module.forward = own
				else:
					del module.forward  # back to the class's method

	# ------------------------------------------------------------------ compute ops
	def _run(self, inputs, name):
		with self._timed(name):
			y = self.model(*inputs)
		return y if isinstance(y, tuple) else (y,)

	def forward(self, mb_id, **options):
		inputs = []
		for var in self.input_variables:
			x = var.wait_and_pop(mb_id)
			if x.is_floating_point() or x.is_complex():
				x.requires_grad_(True)
			inputs.append(x)
		strategy = options.get(OpOptions.REMAT_STRATEGY) or (lambda *_: False)
		with self._selective_remat(strategy, mb_id):
			y = self._run(inputs, f"forward({self.id}:{mb_id})")
			for m in self._layers_dw():
				m.move_last_computed("input", mb_id)
		for targets, value in zip(self.output_variables, y):
			for dst in targets:
				dst.set(dst.to_send, mb_id, value.detach())
		for var, value in zip(self.input_variables, inputs):
			var.set(var.saved, mb_id, value)
		for targets, value in zip(self.output_variables, y):
			targets[0].set(targets[0].saved, mb_id, value)
		if self.is_last:
			return [targets[0].get(targets[0].to_send, mb_id) for targets in self.output_variables]

	def backward_inputs(self, mb_id, **options):
		inputs = [var.get(var.saved, mb_id) for var in self.input_variables]
		outputs = [targets[0].get(targets[0].saved, mb_id) for targets in self.output_variables]
		grads = []
		for targets in self.output_variables:
			g = targets[0].wait_and_pop(mb_id)
			for dst in targets[1:]:
				g = g + dst.wait_and_pop(mb_id)
			grads.append(g)
		ra = bool(options.get(OpOptions.RECOMPUTE_ACTIVATIONS, False))
		rg = bool(options.get(OpOptions.RECOMPUTE_GRADIENTS, False))
		with self._timed(f"backward_inputs({self.id}:{mb_id})"):
			for i, (out, g) in enumerate(zip(outputs, grads)):
				assert out.shape == g.shape, f"Output and grad shapes do not match: {out.shape} != {g.shape}"
				torch.autograd.backward(out, g, retain_graph=i != len(outputs) - 1)
		input_grads = [x.grad.data for x in inputs if x.requires_grad]
		for m in self._layers_dw():
			m.move_last_computed("grad_output", mb_id)
			if rg and not m.is_empty("grad_output"):
				m.delete("grad_output", mb_id)
			if getattr(m, "last_input", None) is not None:  # a checkpoint ran the forward again
				m.move_last_computed("input", mb_id)
			if ra and not m.is_empty("input"):
				m.delete("input", mb_id)
		for var, value in zip([v for v, x in zip(self.input_variables, inputs) if x.requires_grad], input_grads):
			var.set(var.to_send, mb_id, value)
		if ra:
			for var, value in zip(self.input_variables, inputs):
				var.set(var.saved, mb_id, value)
		if rg:
			for targets, value in zip(self.output_variables, grads):
				targets[0].set(targets[0].to_process, mb_id, value)

	def backward_params(self, mb_id, **options):
		with self._timed(f"backward_params({self.id}:{mb_id})"):
			for m in self._layers_dw():
				if not m.is_empty("grad_output"):
					m.backward(mb_id)

	def recompute_forward(self, mb_id, **options):
		inputs = [var.get(var.saved, mb_id) for var in self.input_variables]
		if not options.get(OpOptions.SAVE, False):
			with torch.no_grad():
				self._run(inputs, f"recompute_forward({self.id}:{mb_id})")
		else:
			y = self._run(inputs, f"recompute_forward({self.id}:{mb_id})")
			for var, value in zip(self.input_variables, inputs):
				var.set(var.saved, mb_id, value)
			for targets, value in zip(self.output_variables, y):
				targets[0].set(targets[0].saved, mb_id, value)
		for m in self._layers_dw():
			m.move_last_computed("input", mb_id)

	def recompute_backward_inputs(self, mb_id, **options):
		"""The smallest backward that reaches every split layer, to refill their output gradients
		(elf/zb_utils.py:584-604): differentiate with respect to the split layers' own parameters,
		the leaves that hang directly under their autograd nodes; their gradients come back as None
		(the split functions return none for parameters) and nothing else is accumulated."""
		for var in self.input_variables:
			var.get(var.saved, mb_id)
		outputs = [targets[0].get(targets[0].saved, mb_id) for targets in self.output_variables]
		grads = [targets[0].get(targets[0].to_process, mb_id) for targets in self.output_variables]
		leaves = [p for m in self._layers_dw() for p in (m.weight, getattr(m, "bias", None)) if p is not None and p.requires_grad]
		with self._timed(f"recompute_backward_inputs({self.id}:{mb_id})"):
			for i, (out, g) in enumerate(zip(outputs, grads)):
				if leaves:
					torch.autograd.grad(out, inputs=leaves, grad_outputs=g, allow_unused=True, retain_graph=i != len(outputs) - 1)
		for m in self._layers_dw():
			m.move_last_computed("grad_output", mb_id)

	# ------------------------------------------------------------------ gradients
	def scale_grads(self, batch_size):
		"""Every gradient divided by the batch size (block.py:518-527).  Split layers accumulate in fp32
		``main_grad``; their ``.grad`` in the parameter's dtype is written here."""
		inv = 1.0 / float(batch_size)
		for p in self.model.parameters():
			g32 = getattr(p, "main_grad", None)
			if g32 is not None:
				g32.mul_(inv)
				p.grad = g32.to(p.dtype)
			elif p.grad is not None:
				p.grad.data.mul_(inv)

	def zero_grad(self):
		for p in self.model.parameters():
			if getattr(p, "main_grad", None) is not None:
				p.main_grad.zero_()
			p.grad = None

	def _grad_buffers(self):
		return [getattr(p, "main_grad", None) if getattr(p, "main_grad", None) is not None else p.grad for p in self.model.parameters() if getattr(p, "main_grad", None) is not None or p.grad is not None]

	def clear(self):
		for m in self._layers_dw():
			m.clear()
