"""The split-backward operator plug-in (elf_amd.zb_utils: LinearDX / LayerDW / LinearDW / MappingDW /
replace_layer_with_layer_dw, reference elf/zb_utils.py:9-256, 487-513) on the HIP GEMM, and the generic
stage executor built on it (AutogradStageBlock), against closed forms and plain PyTorch autograd."""

import copy

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from tests.helpers import assert_close

pytestmark = pytest.mark.gpu


def _bf16(t):
	return t.to(torch.bfloat16).cuda()


def test_two_chained_linears_closed_form():
	"""The numbers of the reference's tests/distributed/distributed_test_block.py:16-55 (two chained 2x2
	linears with biases, x = [1, 2], incoming gradient [1, 1]), embedded in the top-left corner of 64-wide
	layers and in token 0 of 64: y0 = [5.1, 11.2], y1 = [9.57, 12.93], dX1 = [1.2, 1.4], dW1 = [[5.1, 11.2]] * 2,
	db1 = [1, 1], dX0 = [5.4, 8.0], dW0 = [[1.2, 2.4], [1.4, 2.8]], db0 = [1.2, 1.4]; B leaves the
	parameter gradients to W."""
	from elf_amd.zb_utils import LinearDW

	def layer(W, b):
		lin = nn.Linear(64, 64).to(torch.bfloat16).cuda()
		with torch.no_grad():
			lin.weight.zero_()
			lin.bias.zero_()
			lin.weight[:2, :2] = torch.tensor(W)
			lin.bias[:2] = torch.tensor(b)
		return LinearDW(lin)

	l0, l1 = layer([[1.0, 2.0], [3.0, 4.0]], [0.1, 0.2]), layer([[0.5, 0.6], [0.7, 0.8]], [0.3, 0.4])
	x = torch.zeros(64, 64, dtype=torch.bfloat16, device="cuda")
	x[0, :2] = torch.tensor([1.0, 2.0])
	x.requires_grad_(True)
	y0 = l0(x)
	y1 = l1(y0)
	tol = dict(rtol=1e-2, atol=1e-2)  # bf16 storage of 5.1, 11.2, ...
	assert torch.allclose(y0[0, :2].float().cpu(), torch.tensor([5.1, 11.2]), **tol)
	assert torch.allclose(y1[0, :2].float().cpu(), torch.tensor([9.57, 12.93]), **tol)
	dy = torch.zeros_like(y1)
	dy[0, :2] = 1.0
	y1.backward(dy)
	assert torch.allclose(x.grad[0, :2].float().cpu(), torch.tensor([5.4, 8.0]), **tol)
	assert float(x.grad[1:].abs().max()) == 0.0 and float(x.grad[0, 2:].abs().max()) == 0.0
	for l in (l0, l1):
		assert l.weight.grad is None and getattr(l.weight, "main_grad", None) is None  # B leaves dW to W
		l.move_last_computed("input", 0)
		l.move_last_computed("grad_output", 0)
		l.backward(0)
		assert l.is_empty("input") and l.is_empty("grad_output")  # W consumed the stash
	assert torch.allclose(l1.weight.main_grad[:2, :2].cpu(), torch.tensor([[5.1, 11.2], [5.1, 11.2]]), **tol)
	assert torch.allclose(l1.bias.main_grad[:2].cpu(), torch.tensor([1.0, 1.0]))
	assert torch.allclose(l0.weight.main_grad[:2, :2].cpu(), torch.tensor([[1.2, 2.4], [1.4, 2.8]]), **tol)
	assert torch.allclose(l0.bias.main_grad[:2].cpu(), torch.tensor([1.2, 1.4]), **tol)
	assert float(l0.weight.main_grad[2:].abs().max()) == 0.0 and float(l0.weight.main_grad[:, 2:].abs().max()) == 0.0


@pytest.mark.parametrize("bias", [False, True])
def test_b_then_w_equals_fused_autograd(bias):
	"""F, then B (input gradient only), then W over three micro-batches = plain autograd of F.linear in
	fp32 on the same bf16 values; 3-D inputs; a layer used twice in one forward sums its output gradients."""
	from elf_amd.zb_utils import LinearDW

	g = torch.Generator().manual_seed(0)
	lin = nn.Linear(192, 320, bias=bias)
	with torch.no_grad():
		lin.weight.copy_(torch.randn(lin.weight.shape, generator=g) * 0.05)
		if bias:
			lin.bias.copy_(torch.randn(320, generator=g) * 0.1)
	lin = lin.to(torch.bfloat16).cuda()
	dw = LinearDW(lin)
	ref_w = lin.weight.detach().float().requires_grad_(True)
	ref_b = lin.bias.detach().float().requires_grad_(True) if bias else None
	for mb in range(3):
		x = _bf16(torch.randn(2, 64, 192, generator=g)).requires_grad_(True)
		gy = _bf16(torch.randn(2, 64, 320, generator=g))
		y = dw(x)
		y.backward(gy)
		dw.move_last_computed("input", mb)
		dw.move_last_computed("grad_output", mb)
		xr = x.detach().float().requires_grad_(True)
		yr = F.linear(xr, ref_w, ref_b)
		yr.backward(gy.float())
		assert_close(y, yr.detach(), f"y[{mb}]")
		assert_close(x.grad, xr.grad, f"dx[{mb}]")
	for mb in (2, 0, 1):  # W in any order
		dw.backward(mb)
	assert_close(dw.weight.main_grad, ref_w.grad, "dW over three micro-batches")
	if bias:
		assert_close(dw.bias.main_grad, ref_b.grad, "db over three micro-batches")
	# a layer called twice in one forward: the stash holds the sum of both output gradients and the LAST input,
	# as in the reference (elf/zb_utils.py:136-151, 118-121)
	sq = LinearDW(nn.Linear(128, 128, bias=False).to(torch.bfloat16).cuda())
	x = _bf16(torch.randn(64, 128, generator=g)).requires_grad_(True)
	y = sq(sq(x))
	gy = _bf16(torch.randn(64, 128, generator=g))
	y.backward(gy)
	inner_out_grad = (gy.float() @ sq.weight.float()).to(torch.bfloat16)
	assert_close(sq.last_grad_output, inner_out_grad.float() + gy.float(), "summed output gradients", rel_max=2e-2)


def test_layer_dw_queues_and_module_replacement():
	from elf_amd._lib import ElfStageError
	from elf_amd.zb_utils import LayerDW, LinearDW, MappingDW, replace_layer_with_layer_dw

	dw = LinearDW(nn.Linear(64, 64).to(torch.bfloat16).cuda())
	t = torch.zeros(1)
	dw.set("input", 2, t)
	assert len(dw.ctx["input"]) == 3 and not dw.is_empty("input") and dw.is_empty("grad_output") and dw._state() == "(1,0)"
	with pytest.raises(ValueError):
		dw.set("input", 2, t)
	dw.delete("input", 2)
	with pytest.raises(ValueError):
		dw.delete("input", 2)
	with pytest.raises(ValueError):
		dw.delete("grad_output", 7)
	dw.move_last_computed("input", 0)  # nothing computed: a no-op
	assert dw.is_empty("input")
	dw.last_input = t
	dw.move_last_computed("input", 1)
	assert dw.ctx["input"][1] is t and dw.last_input is None
	dw.clear()
	assert dw.ctx == {"input": [], "grad_output": []}
	with pytest.raises(NotImplementedError):
		LayerDW.backward(dw, 0)
	assert LayerDW._dx_function_registry[LinearDW].__name__ == "LinearDX" and MappingDW[nn.Linear] is LinearDW

	model = nn.Sequential(nn.Linear(64, 128), nn.Tanh(), nn.Sequential(nn.Linear(128, 64), nn.LayerNorm(64)))
	w0 = model[0].weight
	replace_layer_with_layer_dw(model)
	assert isinstance(model[0], LinearDW) and isinstance(model[2][0], LinearDW) and isinstance(model[2][1], nn.LayerNorm)
	assert model[0].weight is w0, "the replacement shares the wrapped layer's parameters"
	replace_layer_with_layer_dw(model)  # idempotent
	other = nn.Sequential(nn.Linear(64, 64))
	replace_layer_with_layer_dw(other, only=[nn.Conv1d])
	assert type(other[0]) is nn.Linear
	with pytest.raises(ElfStageError):
		LinearDW(nn.Linear(64, 100))  # not a multiple of 64: no tile of the HIP GEMM fits
	with pytest.raises(ElfStageError):
		dw(torch.zeros(64, 64, device="cuda"))  # fp32 input
	with pytest.raises(ElfStageError):
		dw(torch.zeros(10, 64, dtype=torch.bfloat16, device="cuda"))  # 10 tokens


class _Mixer(nn.Module):
	"""A stage that is not a transformer block: two inputs, biased linears, LayerNorm, tanh, two outputs."""

	def __init__(self, d=128, h=256):
		super().__init__()
		self.inp = nn.Linear(d, h)
		self.gate = nn.Linear(d, h)
		self.norm = nn.LayerNorm(h)
		self.body = nn.Sequential(nn.Linear(h, h), nn.Tanh(), nn.Linear(h, d))
		self.skip = nn.Linear(d, d, bias=False)

	def forward(self, a, b):
		h = self.norm(self.inp(a) * torch.sigmoid(self.gate(b)))
		return self.body(h) + self.skip(a), h


def _mixer(seed):
	torch.manual_seed(seed)
	m = _Mixer()
	with torch.no_grad():
		for p in m.parameters():
			if p.dim() == 2:
				p.mul_(0.5)
	return m.to(torch.bfloat16)


@pytest.mark.parametrize("variant", ["plain", "remat_body", "activations_bwd", "full_bwd"])
def test_autograd_stage_block_on_a_generic_module(variant):
	"""F / B / W (and the remat variants) of a stage with two inputs and two outputs through
	AutogradStageBlock against plain autograd in fp32 over the same bf16 weights: outputs, both input
	gradients, every parameter gradient (split layers in fp32 main_grad, the norm in .grad)."""
	from elf_amd.execution import AutogradStageBlock
	from elf_amd.partitioners.utils import Signature
	from elf_amd.scheduling import OpOptions
	from elf_amd.zb_utils import LinearDW

	model = _mixer(3)
	ref = copy.deepcopy(model).float().cuda()
	sig = Signature(["a", "b"], ["y", "h"], [0, 0], [[2], [2]])
	placement = [0, 1, 2]
	blk = AutogradStageBlock(model, 1, placement, sig)
	assert sum(isinstance(m, LinearDW) for m in blk.model.modules()) == 5
	g = torch.Generator().manual_seed(5)
	n_mb, T = 2, 64
	data = [[_bf16(torch.randn(T, 128, generator=g)) for _ in range(2)] for _ in range(n_mb)]
	grads = [[_bf16(torch.randn(T, 128, generator=g)), _bf16(torch.randn(T, 256, generator=g) * 0.1)] for _ in range(n_mb)]
	blk.zero_grad()
	for m in range(n_mb):
		for var, x in zip(blk.input_variables, data[m]):
			var.set(var.to_process, m, (None, x.clone()))
		opts = {OpOptions.REMAT_STRATEGY: (lambda name, module: name == "body")} if variant == "remat_body" else {}
		blk.forward(m, **opts)
		if variant == "remat_body":
			assert all(l.ctx["input"][m] is None for l in blk.model.body if isinstance(l, LinearDW)), "inputs inside the checkpointed module are not kept"
	want_out, want_dx = [], []
	for m in range(n_mb):
		a, b = (x.float().requires_grad_(True) for x in data[m])
		y, h = ref(a, b)
		torch.autograd.backward([y, h], [gr.float() for gr in grads[m]])
		want_out.append((y.detach(), h.detach()))
		want_dx.append((a.grad, b.grad))
	for m in range(n_mb):
		for targets, gr, want in zip(blk.output_variables, grads[m], want_out[m]):
			assert_close(targets[0].get(targets[0].to_send, m), want, f"{variant} output[{m}]")
			targets[0].set(targets[0].to_process, m, (None, gr))
		if variant == "activations_bwd":
			blk.backward_inputs(m, **{OpOptions.RECOMPUTE_ACTIVATIONS: True})
			assert all(l.ctx["input"][m] is None and l.ctx["grad_output"][m] is not None for l in blk._layers_dw())
			blk.recompute_forward(m)
		elif variant == "full_bwd":
			blk.backward_inputs(m, **{OpOptions.RECOMPUTE_ACTIVATIONS: True, OpOptions.RECOMPUTE_GRADIENTS: True})
			assert all(l.ctx["input"][m] is None and l.ctx["grad_output"][m] is None for l in blk._layers_dw())
			norm_grad = blk.model.norm.weight.grad.clone()
			blk.recompute_forward(m, **{OpOptions.SAVE: True})
			blk.recompute_backward_inputs(m)
			assert torch.equal(blk.model.norm.weight.grad, norm_grad), "the gradient recompute must not add to non-split parameters again"
		else:
			blk.backward_inputs(m)
		for var, want in zip(blk.input_variables, want_dx[m]):
			assert_close(var.get(var.to_send, m), want, f"{variant} dx[{m}]")
		blk.backward_params(m)
		assert all(l.ctx["input"][m] is None and l.ctx["grad_output"][m] is None for l in blk._layers_dw())
	ref_params = dict(ref.named_parameters())
	for name, p in blk.model.named_parameters():
		got = p.main_grad if getattr(p, "main_grad", None) is not None else p.grad
		assert got is not None, name
		assert_close(got, ref_params[name].grad, f"{variant} grad {name}")
	blk.scale_grads(4)
	for name, p in blk.model.named_parameters():
		assert p.grad.dtype == torch.bfloat16
		assert_close(p.grad, ref_params[name].grad / 4, f"{variant} scaled grad {name}")


@pytest.mark.parametrize("scheduler,placement", [("afab", [0, 0]), ("1f1b", [0, 1]), ("zbh1", [0, 1])])
def test_pipeline_builds_generic_stages_for_other_modules(scheduler, placement):
	"""Pipeline over two stages that are not transformer blocks: they run through AutogradStageBlock (the
	split linears on the HIP GEMM) under AFAB on one rank and under 1F1B / ZB-H1 as two ranks played by one
	process, and give the loss and gradients of the un-pipelined model."""
	from elf_amd.execution import AutogradStageBlock
	from elf_amd.pipeline import Pipeline

	class Stage(nn.Module):
		def __init__(self):
			super().__init__()
			self.net = nn.Sequential(nn.Linear(128, 256), nn.GELU(), nn.LayerNorm(256), nn.Linear(256, 128))

		def forward(self, x):
			return x + self.net(x)

	torch.manual_seed(11)
	stages = [Stage().to(torch.bfloat16), Stage().to(torch.bfloat16)]
	refs = [copy.deepcopy(s).float().cuda() for s in stages]
	g = torch.Generator().manual_seed(12)
	mb, n_mb = 64, 4
	x = _bf16(torch.randn(mb * n_mb, 128, generator=g))
	tgt = _bf16(torch.randn(mb * n_mb, 128, generator=g))

	def loss_fn(pred, target, reduction="sum"):
		return F.mse_loss(pred.float(), target.float(), reduction=reduction)

	pipe = Pipeline(stages, x[:mb], scheduler=scheduler, partitioner=False, placement=placement, all_ranks=len(set(placement)) > 1)
	assert all(isinstance(b, AutogradStageBlock) for b in pipe.blocks)
	pipe.zero_grad()
	result, loss = pipe(x, tgt, loss_fn, split_size=mb)
	out = refs[1](refs[0](x.float()))
	want_loss = F.mse_loss(out, tgt.float(), reduction="sum") / (128 * mb * n_mb)
	want_loss.backward()
	assert_close(torch.cat([r.float() for r in result]), out.detach(), "pipeline output")
	assert abs(float(loss) - float(want_loss.detach())) <= 2e-2 * float(want_loss.detach())
	for stage, ref in zip(stages, refs):
		ref_params = dict(ref.named_parameters())
		for name, p in stage.named_parameters():
			assert_close(p.grad, ref_params[name].grad, f"grad {name}")
