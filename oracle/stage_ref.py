"""TEST INFRASTRUCTURE - CPU restatement ("oracle") of the reference stage in plain PyTorch.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this file, and
only as the checker / the timed CPU baseline.  Nothing in elf_amd/ imports it.

What is restated, and from where (paths are into the reference repository):

* ``SplitLinear`` / ``SplitLinearFn``  - LinearDX / LinearDW, elf/zb_utils.py:9-40, 198-256:
  forward ``F.linear``; B returns ``dY @ W`` and stashes ``dY``; W does ``dW += dY^T X``.
* ``gpt_block``   - TransformerBlock, benchmarks/models/simple.py:437-468 (+ MultiHeadAttention
  :389-434, FeedForward :44-52) with dropout off (the reference's own checker runs ``model.eval()``,
  benchmarks/benchmark_utils.py:229), bias-free linears, an explicit ``causal`` flag.
* ``llama_block`` - NO reference module exists (its model zoo has no RMSNorm/RoPE/SwiGLU/GQA);
  textbook definitions: RMSNorm x*rsqrt(mean(x^2)+eps)*g, RoPE half-split with
  inv_freq = theta^(-2i/D), grouped-query attention = repeat K/V heads, SwiGLU silu(g)*u.
* ``RefStage``    - PipelineBlock F / B / W / RF / RB* and their slot semantics,
  elf/execution/block.py:210-391, 624-694; full-stage checkpointing elf/execution/remat.py:26-74.
  ``ends`` adds what the first / last stage of the reference's FullTransformer own
  (benchmarks/models/simple.py:496-509): ``embed`` = nn.Embedding in front of the blocks (a plain
  autograd leaf: its gradient accumulates in B), ``head`` = bias-free nn.Linear behind them (a
  split linear like the others), ``normf_g`` / ``normf_b`` = an optional final norm (no reference
  module; textbook definition as for the blocks' norms).

Parity pins (tests/test_oracle_cpu.py): SplitLinear against the closed-form 2x2 example held by
the reference's tests/distributed/distributed_test_block.py:16-55; B-then-W against fused
autograd on ``F.linear``; attention against a brute-force fp64 loop and against
``F.scaled_dot_product_attention`` (enable_gqa / is_causal); RMSNorm / LayerNorm / RoPE / SwiGLU
against closed forms; sum over micro-batches of dW == full-batch dW; remat variants == no remat.
"""

import math

import torch
import torch.nn.functional as F
from torch.utils.checkpoint import checkpoint

ARCH_GPT, ARCH_LLAMA = 0, 1


# --------------------------------------------------------------------------------------------
# split backward of a linear layer (zb_utils.py:9-40, 215-256)
class SplitLinear:
	"""Weight [out, in] plus the per-micro-batch queues of the reference's LayerDW.ctx."""

	def __init__(self, weight):
		self.weight = weight  # leaf tensor
		self.inputs = {}      # mb -> X
		self.grad_outputs = {}  # mb -> dY
		self.last_input = None
		self.last_grad_output = None
		self.grad = None      # accumulated dW (fp32 unless acc_dtype says otherwise)

	def __call__(self, x):
		return SplitLinearFn.apply(x, self.weight, self)

	def move_last(self, queue, mb):
		last = self.last_input if queue == "input" else self.last_grad_output
		if last is None:
			return
		q = self.inputs if queue == "input" else self.grad_outputs
		if mb in q:
			raise ValueError(f"{queue} at index {mb} already set")
		q[mb] = last
		if queue == "input":
			self.last_input = None
		else:
			self.last_grad_output = None

	def backward_params(self, mb, acc_dtype=torch.float32):
		go = self.grad_outputs.pop(mb)
		inp = self.inputs.pop(mb)
		go2 = go.reshape(-1, go.shape[-1])
		in2 = inp.reshape(-1, inp.shape[-1])
		gw = torch.mm(go2.t().to(acc_dtype), in2.to(acc_dtype)) if acc_dtype != go2.dtype else torch.mm(go2.t(), in2)
		if self.grad is None:
			self.grad = gw
		else:
			self.grad.add_(gw)


class SplitLinearFn(torch.autograd.Function):
	@staticmethod
	def forward(ctx, x, weight, owner):
		ctx.owner = owner
		owner.last_input = x.detach()
		ctx.save_for_backward(x.detach())  # forces checkpoint() to recompute it
		return F.linear(x, weight)

	@staticmethod
	def backward(ctx, gy):
		o = ctx.owner
		o.last_grad_output = gy if o.last_grad_output is None else o.last_grad_output + gy
		return gy @ o.weight.detach(), None, None


# --------------------------------------------------------------------------------------------
# ops
def _up(t):
	"""Math runs in fp32 for bf16 / fp16 / fp32 inputs and stays in fp64 for fp64 inputs."""
	return t if t.dtype == torch.float64 else t.float()


def rms_norm(x, g, eps):
	xf = _up(x)
	return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * _up(g)).to(x.dtype)


def layer_norm(x, g, b, eps):
	return F.layer_norm(_up(x), (x.shape[-1],), _up(g), _up(b), eps).to(x.dtype)


def rope_tables(S, D, theta, device):
	"""cos/sin [S, D/2] in fp32 from fp64 angles: a = pos * theta^(-2i/D)."""
	inv = theta ** (-torch.arange(0, D // 2, dtype=torch.float64, device=device) / (D // 2))
	ang = torch.arange(S, dtype=torch.float64, device=device)[:, None] * inv[None, :]
	return ang.cos().float(), ang.sin().float()  # the tables themselves are fp32, as in the HIP path


def rope(x, cos, sin):
	"""x: [B, S, H, D]; half-split rotation (out_lo = lo*cos - hi*sin, out_hi = hi*cos + lo*sin)."""
	D = x.shape[-1]
	lo, hi = _up(x[..., : D // 2]), _up(x[..., D // 2 :])
	c, s = cos[None, :, None, :].to(lo.dtype), sin[None, :, None, :].to(lo.dtype)
	return torch.cat([lo * c - hi * s, hi * c + lo * s], dim=-1).to(x.dtype)


def attention(q, k, v, causal, use_sdpa=False):
	"""q: [B,S,Hq,D], k/v: [B,S,Hkv,D] -> [B,S,Hq,D]; softmax(QK^T/sqrt(D)) V, fp32 softmax."""
	B, S, Hq, D = q.shape
	G = Hq // k.shape[2]
	qt, kt, vt = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
	if use_sdpa:
		o = F.scaled_dot_product_attention(qt, kt, vt, is_causal=causal, enable_gqa=G > 1)
		return o.transpose(1, 2)
	kt = kt.repeat_interleave(G, dim=1)
	vt = vt.repeat_interleave(G, dim=1)
	s = (_up(qt) @ _up(kt).transpose(-1, -2)) / math.sqrt(D)
	if causal:
		s = s.masked_fill(~torch.ones(S, S, dtype=torch.bool, device=q.device).tril(), float("-inf"))
	p = torch.softmax(s, dim=-1)
	return (p @ _up(vt)).to(q.dtype).transpose(1, 2)


# --------------------------------------------------------------------------------------------
# blocks.  `p` is a dict: norm weights are plain leaf tensors, linears are SplitLinear objects.
# cfg["_ckpt"] (set per forward by RefStage) names the kinds of sub-module whose forward runs under
# checkpoint(use_reentrant=False), as RematManager.apply_selective_remat wraps the modules a
# remat_strategy selects (elf/execution/remat.py:42-58): "norm", "attn", "act".
def _sub(cfg, kind, fn, *args):
	if kind in cfg.get("_ckpt", ()):
		return checkpoint(fn, *args, use_reentrant=False)
	return fn(*args)


def gpt_block(x, p, cfg, use_sdpa=False):
	B, S, d = x.shape
	H, D = cfg["n_heads"], cfg["head_dim"]
	y = _sub(cfg, "norm", layer_norm, x, p["norm1_g"], p["norm1_b"], cfg["eps"])
	qkv = p["wqkv"](y)
	q, k, v = qkv.split([H * D, H * D, H * D], dim=-1)
	o = _sub(cfg, "attn", attention, q.reshape(B, S, H, D), k.reshape(B, S, H, D), v.reshape(B, S, H, D), cfg["causal"], use_sdpa)
	x2 = x + p["wo"](o.reshape(B, S, H * D))
	y = _sub(cfg, "norm", layer_norm, x2, p["norm2_g"], p["norm2_b"], cfg["eps"])
	return x2 + p["w2"](_sub(cfg, "act", F.gelu, p["w1"](y)))


def llama_block(x, p, cfg, use_sdpa=False):
	B, S, d = x.shape
	Hq, Hkv, D, Fh = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["ffn"]
	cos, sin = cfg["_rope"]
	y = _sub(cfg, "norm", rms_norm, x, p["norm1_g"], cfg["eps"])
	qkv = p["wqkv"](y)
	q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
	q = rope(q.reshape(B, S, Hq, D), cos, sin)
	k = rope(k.reshape(B, S, Hkv, D), cos, sin)
	o = _sub(cfg, "attn", attention, q, k, v.reshape(B, S, Hkv, D), cfg["causal"], use_sdpa)
	x2 = x + p["wo"](o.reshape(B, S, Hq * D))
	y = _sub(cfg, "norm", rms_norm, x2, p["norm2_g"], cfg["eps"])
	gu = p["w1"](y)
	return x2 + p["w2"](F.silu(gu[..., :Fh]) * gu[..., Fh:])


PARAM_NAMES = ["norm1_g", "norm1_b", "wqkv", "wo", "norm2_g", "norm2_b", "w1", "w2"]
LINEARS = ("wqkv", "wo", "w1", "w2")


def param_shapes(cfg):
	d, Hq, Hkv, D, Fh = cfg["d_model"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["ffn"]
	llama = cfg["arch"] == ARCH_LLAMA
	shapes = {
		"norm1_g": (d,), "norm1_b": (d,), "wqkv": ((Hq + 2 * Hkv) * D, d), "wo": (d, Hq * D),
		"norm2_g": (d,), "norm2_b": (d,), "w1": ((2 * Fh if llama else Fh), d), "w2": (d, Fh),
	}
	if llama:
		del shapes["norm1_b"], shapes["norm2_b"]
	return shapes


def make_params(cfg, seed=0, dtype=torch.bfloat16, perturb_norm=True):
	"""Seeded stage parameters on CPU: linears N(0, 0.02); norm gains 1 (+ a small seeded
	perturbation so that gain / bias gradients are exercised), biases 0 (+ perturbation)."""
	g = torch.Generator(device="cpu").manual_seed(seed)
	blocks = []
	for _ in range(cfg["n_blocks"]):
		blk = {}
		for name, shape in param_shapes(cfg).items():
			if name in LINEARS:
				t = torch.randn(shape, generator=g) * 0.02
			elif name.endswith("_g"):
				t = torch.ones(shape) + (0.1 * torch.randn(shape, generator=g) if perturb_norm else 0)
			else:
				t = 0.1 * torch.randn(shape, generator=g) if perturb_norm else torch.zeros(shape)
			blk[name] = t.to(dtype)
		blocks.append(blk)
	return blocks


def make_boundary(cfg, n_mb, seed=1, dtype=torch.bfloat16):
	"""Seeded N(0,1) incoming activations X[mb] and gradients dY[mb], each [mb, seq, d]."""
	g = torch.Generator(device="cpu").manual_seed(seed)
	shape = (cfg["mb"], cfg["seq"], cfg["d_model"])
	xs = [torch.randn(shape, generator=g).to(dtype) for _ in range(n_mb)]
	dys = [torch.randn(shape, generator=g).to(dtype) for _ in range(n_mb)]
	return xs, dys


# --------------------------------------------------------------------------------------------
class RefStage:
	"""Plain-PyTorch stage with the reference's F / B / W / RF / RB* semantics.

	compute_dtype: dtype the blocks run in (float32 = the fp32-accumulated truth from the same
	bf16-rounded weights; bfloat16 = what the reference itself would run).
	acc_dtype: dtype of the dW accumulators (the reference accumulates in the parameter dtype,
	zb_utils.py:241-244; the HIP path in fp32)."""

	def __init__(self, cfg, params, compute_dtype=torch.float32, acc_dtype=torch.float32, device="cpu", use_sdpa=False, ends=None):
		self.cfg = dict(cfg)
		self.device = device
		self.compute_dtype = compute_dtype
		self.acc_dtype = acc_dtype
		self.use_sdpa = use_sdpa
		if cfg["arch"] == ARCH_LLAMA:
			self.cfg["_rope"] = rope_tables(cfg["seq"], cfg["head_dim"], cfg["rope_theta"], device)
		self.blocks = []
		for blk in params:
			b = {}
			for name, t in blk.items():
				leaf = t.to(device=device, dtype=compute_dtype).clone().requires_grad_(name not in LINEARS)
				b[name] = SplitLinear(leaf) if name in LINEARS else leaf
			self.blocks.append(b)
		self.saved_in, self.saved_out, self.kept_grad = {}, {}, {}
		self.block_fn = llama_block if cfg["arch"] == ARCH_LLAMA else gpt_block
		self.ends = {}
		for name, t in (ends or {}).items():
			leaf = t.to(device=device, dtype=compute_dtype).clone().requires_grad_(name != "head")
			self.ends[name] = SplitLinear(leaf) if name == "head" else leaf

	def _linears(self):
		return [b[n] for b in self.blocks for n in LINEARS] + ([self.ends["head"]] if "head" in self.ends else [])

	def _model(self, x):
		if "embed" in self.ends:
			x = F.embedding(x, self.ends["embed"])
		for b in self.blocks:
			x = self.block_fn(x, b, self.cfg, self.use_sdpa)
		if "normf_g" in self.ends:
			e = self.ends
			if self.cfg["arch"] == ARCH_LLAMA:
				x = _sub(self.cfg, "norm", rms_norm, x, e["normf_g"], self.cfg["eps"])
			else:
				x = _sub(self.cfg, "norm", layer_norm, x, e["normf_g"], e["normf_b"], self.cfg["eps"])
		if "head" in self.ends:
			x = self.ends["head"](x)
		return x

	def _as_input(self, x):
		if "embed" in self.ends:
			return x.to(device=self.device)  # token ids: no gradient
		return x.to(device=self.device, dtype=self.compute_dtype).detach().requires_grad_(True)

	# F (block.py:210-263)
	def forward(self, mb, x, remat_root=False, remat=()):
		"""``remat``: kinds of sub-module ("norm", "attn", "act") checkpointed in this forward."""
		x = self._as_input(x)
		self.cfg["_ckpt"] = tuple(remat)
		y = checkpoint(self._model, x, use_reentrant=False) if remat_root else self._model(x)
		self.cfg["_ckpt"] = ()
		for lin in self._linears():
			lin.move_last("input", mb)
			if remat_root:
				lin.inputs.pop(mb, None)  # recomputed inside B (remat.py:60-72)
		self.saved_in[mb], self.saved_out[mb] = x, y
		return y.detach()

	# B (block.py:624-694)
	def backward_inputs(self, mb, dy, recompute_activations=False, recompute_gradients=False):
		x, y = self.saved_in.pop(mb), self.saved_out.pop(mb)
		dy = dy.to(device=self.device, dtype=self.compute_dtype)
		torch.autograd.backward(y, dy)
		for lin in self._linears():
			lin.move_last("grad_output", mb)
			if recompute_gradients:
				lin.grad_outputs.pop(mb, None)
			if lin.last_input is not None:  # checkpoint re-ran the forward
				lin.move_last("input", mb)
			if recompute_activations:
				lin.inputs.pop(mb, None)
		if recompute_activations:
			self.saved_in[mb] = x
		if recompute_gradients:
			self.kept_grad[mb] = dy
		return x.grad.detach() if x.is_floating_point() else None

	# RF (block.py:308-338)
	def recompute_forward(self, mb, save=False):
		x = self.saved_in.pop(mb)
		if save:
			x = self._as_input(x)
			y = self._model(x)
			self.saved_in[mb], self.saved_out[mb] = x, y
		else:
			with torch.no_grad():
				self._model(x)
		for lin in self._linears():
			lin.move_last("input", mb)

	# RB* (block.py:340-374; zb_utils.py:584-604): only the linears' dY are refreshed, parameter
	# gradients of the norms must not be accumulated a second time.
	def recompute_backward_inputs(self, mb):
		x, y, dy = self.saved_in.pop(mb), self.saved_out.pop(mb), self.kept_grad.pop(mb)
		# only the graph walk matters (it refills the split linears' dY); no .grad is touched
		torch.autograd.grad(y, [x] if x.is_floating_point() else [self.ends["embed"]], dy, allow_unused=True)
		for lin in self._linears():
			lin.move_last("grad_output", mb)

	# W (block.py:376-391)
	def backward_params(self, mb):
		for lin in self._linears():
			if lin.grad_outputs:
				lin.backward_params(mb, self.acc_dtype)

	def scale_grads(self, batch_size):
		for name, g in self.grads().items():
			g /= batch_size

	def grads(self):
		"""{"<block>.<name>": accumulated gradient}"""
		out = {}
		for i, b in enumerate(self.blocks):
			for name, v in b.items():
				g = v.grad
				if g is not None:
					out[f"{i}.{name}"] = g
		for name, v in self.ends.items():
			if v.grad is not None:
				out[f"ends.{name}"] = v.grad
		return out

	def zero_grad(self):
		for b in self.blocks:
			for v in b.values():
				v.grad = None
		for v in self.ends.values():
			v.grad = None
