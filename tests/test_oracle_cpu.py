"""Pins of the oracle (oracle/stage_ref.py) itself, so that a plausible mistake in it - a dropped
term, a wrong sign or index, a transposed operand - fails here before the oracle is trusted as
the checker of the HIP path.  Everything runs on CPU in float64/float32."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import stage_ref as R


def test_split_linear_closed_form_from_reference_test_inputs():
	"""Numbers of the reference's tests/distributed/distributed_test_block.py:16-55 (two chained
	2x2 linears; biases folded into the input here since stage linears are bias-free):
	Y = X W^T, dX = dY W, dW = dY^T X."""
	W0 = torch.tensor([[1.0, 2.0], [3.0, 4.0]])
	W1 = torch.tensor([[0.5, 0.6], [0.7, 0.8]])
	l0, l1 = R.SplitLinear(W0.clone()), R.SplitLinear(W1.clone())
	x = torch.tensor([[1.0, 2.0]], requires_grad=True)
	y0 = l0(x) + torch.tensor([0.1, 0.2])
	y1 = l1(y0) + torch.tensor([0.3, 0.4])
	assert torch.allclose(y0, torch.tensor([[5.1, 11.2]])) and torch.allclose(y1, torch.tensor([[9.57, 12.93]]))
	y1.backward(torch.tensor([[1.0, 1.0]]))
	assert torch.allclose(x.grad, torch.tensor([[5.4, 8.0]]))  # dX0 = (dY1 W1) W0
	for l in (l0, l1):
		l.move_last("input", 0)
		l.move_last("grad_output", 0)
		assert l.grad is None  # B leaves the weight gradient to W
		l.backward_params(0)
	assert torch.allclose(l1.grad, torch.tensor([[5.1, 11.2], [5.1, 11.2]]))
	assert torch.allclose(l0.grad, torch.tensor([[1.2, 2.4], [1.4, 2.8]]))
	assert not l0.inputs and not l0.grad_outputs  # W consumed the stash
	with pytest.raises(KeyError):
		l0.backward_params(0)


def test_b_then_w_equals_fused_autograd():
	torch.manual_seed(0)
	W = torch.randn(7, 5, dtype=torch.float64)
	x = torch.randn(3, 4, 5, dtype=torch.float64, requires_grad=True)
	gy = torch.randn(3, 4, 7, dtype=torch.float64)
	lin = R.SplitLinear(W.clone())
	lin(x).backward(gy)
	lin.move_last("input", 2)
	lin.move_last("grad_output", 2)
	lin.backward_params(2, acc_dtype=torch.float64)
	Wr = W.clone().requires_grad_(True)
	xr = x.detach().clone().requires_grad_(True)
	F.linear(xr, Wr).backward(gy)
	assert torch.allclose(x.grad, xr.grad) and torch.allclose(lin.grad, Wr.grad)
	# accumulation over micro-batches and the "already set" rule of the slot lists
	lin(x.detach().requires_grad_(True)).backward(gy)
	lin.move_last("input", 3)
	lin.move_last("grad_output", 3)
	lin.last_input = x.detach()
	with pytest.raises(ValueError):
		lin.move_last("input", 3)
	lin.backward_params(3, acc_dtype=torch.float64)
	assert torch.allclose(lin.grad, 2 * Wr.grad)


def _attention_bruteforce(q, k, v, causal):
	B, S, Hq, D = q.shape
	G = Hq // k.shape[2]
	out = torch.zeros(B, S, Hq, D, dtype=torch.float64)
	for b in range(B):
		for h in range(Hq):
			for i in range(S):
				last = i if causal else S - 1
				w = [math.exp(sum(float(q[b, i, h, t]) * float(k[b, j, h // G, t]) for t in range(D)) / math.sqrt(D)) for j in range(last + 1)]
				z = sum(w)
				for j in range(last + 1):
					out[b, i, h] += (w[j] / z) * v[b, j, h // G].double()
	return out


@pytest.mark.parametrize("causal", [False, True])
def test_attention_against_bruteforce_and_sdpa(causal):
	torch.manual_seed(1)
	q, k, v = torch.randn(2, 6, 4, 8, dtype=torch.float64), torch.randn(2, 6, 2, 8, dtype=torch.float64), torch.randn(2, 6, 2, 8, dtype=torch.float64)
	got = R.attention(q, k, v, causal)
	assert torch.allclose(got, _attention_bruteforce(q, k, v, causal), atol=1e-6)
	qf, kf, vf = torch.randn(2, 33, 8, 16), torch.randn(2, 33, 2, 16), torch.randn(2, 33, 2, 16)
	assert torch.allclose(R.attention(qf, kf, vf, causal), R.attention(qf, kf, vf, causal, use_sdpa=True), atol=2e-5)


def test_norms_rope_swiglu_closed_forms():
	torch.manual_seed(2)
	x = torch.randn(5, 16, dtype=torch.float64)
	g, b = torch.randn(16, dtype=torch.float64), torch.randn(16, dtype=torch.float64)
	eps = 1e-5
	rms = R.rms_norm(x, g, eps)
	ln = R.layer_norm(x, g, b, eps)
	for i in range(5):
		ms = sum(float(t) ** 2 for t in x[i]) / 16
		mu = sum(float(t) for t in x[i]) / 16
		var = sum((float(t) - mu) ** 2 for t in x[i]) / 16
		for j in range(16):
			assert abs(float(rms[i, j]) - float(x[i, j]) / math.sqrt(ms + eps) * float(g[j])) < 1e-5
			assert abs(float(ln[i, j]) - ((float(x[i, j]) - mu) / math.sqrt(var + eps) * float(g[j]) + float(b[j]))) < 1e-5
	# RoPE: position 0 is the identity, norms of (lo_i, hi_i) pairs are preserved, angle = pos * theta^(-2i/D)
	S, D, theta = 7, 8, 5e5
	cos, sin = R.rope_tables(S, D, theta, "cpu")
	t = torch.randn(1, S, 3, D, dtype=torch.float64)
	r = R.rope(t, cos, sin)
	assert torch.allclose(r[:, 0], t[:, 0], atol=1e-6)
	assert torch.allclose(r[..., : D // 2] ** 2 + r[..., D // 2 :] ** 2, t[..., : D // 2] ** 2 + t[..., D // 2 :] ** 2, atol=1e-5)
	pos, i = 5, 2
	a = pos * theta ** (-2 * i / D)
	want_lo = float(t[0, pos, 1, i]) * math.cos(a) - float(t[0, pos, 1, i + D // 2]) * math.sin(a)
	want_hi = float(t[0, pos, 1, i + D // 2]) * math.cos(a) + float(t[0, pos, 1, i]) * math.sin(a)
	assert abs(float(r[0, pos, 1, i]) - want_lo) < 1e-5 and abs(float(r[0, pos, 1, i + D // 2]) - want_hi) < 1e-5
	# relative-position property: <rope(q)_m, rope(k)_n> depends on m - n only
	q1, k1 = torch.randn(D, dtype=torch.float64), torch.randn(D, dtype=torch.float64)
	qq = R.rope(q1.expand(1, S, 1, D), cos, sin)[0, :, 0]
	kk = R.rope(k1.expand(1, S, 1, D), cos, sin)[0, :, 0]
	assert abs(float(qq[3] @ kk[1]) - float(qq[6] @ kk[4])) < 1e-4


CFG = {
	"gpt": {"arch": R.ARCH_GPT, "n_blocks": 2, "d_model": 32, "n_heads": 4, "n_kv_heads": 4, "head_dim": 8, "ffn": 48, "seq": 8, "mb": 2, "causal": False, "eps": 1e-5, "rope_theta": 0.0},
	"llama": {"arch": R.ARCH_LLAMA, "n_blocks": 2, "d_model": 32, "n_heads": 4, "n_kv_heads": 2, "head_dim": 8, "ffn": 40, "seq": 8, "mb": 2, "causal": True, "eps": 1e-5, "rope_theta": 5e5},
}


def _plain_module_grads(cfg, params, xs, dys):
	"""The same blocks written with nn.functional only (no SplitLinear, no stage executor), run
	un-pipelined on the whole batch: the reference's own parity criterion is "pipeline == plain
	model" (benchmarks/benchmark_utils.py:215-292)."""
	ps = [{k: v.double().clone().requires_grad_(True) for k, v in blk.items()} for blk in params]
	x = torch.cat(xs).double().requires_grad_(True)
	h = x
	B, S = h.shape[0], cfg["seq"]
	Hq, Hkv, D, Fh = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["ffn"]
	for p in ps:
		if cfg["arch"] == R.ARCH_GPT:
			y = F.layer_norm(h, (h.shape[-1],), p["norm1_g"], p["norm1_b"], cfg["eps"])
		else:
			y = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + cfg["eps"]) * p["norm1_g"]
		qkv = y @ p["wqkv"].t()
		q, k, v = [t.reshape(B, S, -1, D) for t in qkv.split([Hq * D, Hkv * D, Hkv * D], -1)]
		if cfg["arch"] == R.ARCH_LLAMA:
			cos, sin = [t.double() for t in R.rope_tables(S, D, cfg["rope_theta"], "cpu")]
			rot = lambda t: torch.cat([t[..., : D // 2] * cos[None, :, None] - t[..., D // 2 :] * sin[None, :, None], t[..., D // 2 :] * cos[None, :, None] + t[..., : D // 2] * sin[None, :, None]], -1)
			q, k = rot(q), rot(k)
		o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=cfg["causal"], enable_gqa=Hq != Hkv)
		h2 = h + o.transpose(1, 2).reshape(B, S, Hq * D) @ p["wo"].t()
		if cfg["arch"] == R.ARCH_GPT:
			y = F.layer_norm(h2, (h2.shape[-1],), p["norm2_g"], p["norm2_b"], cfg["eps"])
			h = h2 + F.gelu(y @ p["w1"].t()) @ p["w2"].t()
		else:
			y = h2 * torch.rsqrt(h2.pow(2).mean(-1, keepdim=True) + cfg["eps"]) * p["norm2_g"]
			gu = y @ p["w1"].t()
			h = h2 + (F.silu(gu[..., :Fh]) * gu[..., Fh:]) @ p["w2"].t()
	h.backward(torch.cat(dys).double())
	return h.detach(), x.grad, {f"{i}.{k}": v.grad for i, p in enumerate(ps) for k, v in p.items()}


@pytest.mark.parametrize("kind", ["gpt", "llama"])
def test_stage_equals_unpipelined_model_and_sums_over_microbatches(kind):
	cfg = CFG[kind]
	params = R.make_params(cfg, seed=3, dtype=torch.float64)
	xs, dys = R.make_boundary(cfg, 3, seed=4, dtype=torch.float64)
	ref = R.RefStage(cfg, params, compute_dtype=torch.float64, acc_dtype=torch.float64)
	ys = [ref.forward(m, xs[m]) for m in range(3)]
	dxs = [ref.backward_inputs(m, dys[m]) for m in (2, 0, 1)]  # any order
	for m in (1, 2, 0):
		ref.backward_params(m)
	y_all, dx_all, grads = _plain_module_grads(cfg, params, xs, dys)
	assert torch.allclose(torch.cat(ys), y_all, atol=1e-9)
	assert torch.allclose(torch.cat([dxs[1], dxs[2], dxs[0]]), dx_all, atol=1e-9)
	got = ref.grads()
	assert set(got) == set(grads)
	for name in grads:
		assert torch.allclose(got[name], grads[name], atol=1e-8), name


@pytest.mark.parametrize("kind", ["gpt", "llama"])
def test_remat_variants_give_the_same_gradients(kind):
	cfg = CFG[kind]
	params = R.make_params(cfg, seed=5, dtype=torch.float64)
	xs, dys = R.make_boundary(cfg, 1, seed=6, dtype=torch.float64)

	def run(variant):
		ref = R.RefStage(cfg, params, compute_dtype=torch.float64, acc_dtype=torch.float64)
		y = ref.forward(0, xs[0], remat_root=variant == "full_fwd", remat={"simple": ("norm", "act"), "selective": ("attn",)}.get(variant, ()))
		if variant == "activations_bwd":
			dx = ref.backward_inputs(0, dys[0], recompute_activations=True)
			assert all(not lin.inputs and lin.grad_outputs for lin in ref._linears())
			ref.recompute_forward(0)
		elif variant == "full_bwd":
			dx = ref.backward_inputs(0, dys[0], recompute_activations=True, recompute_gradients=True)
			assert all(not lin.inputs and not lin.grad_outputs for lin in ref._linears())
			ref.recompute_forward(0, save=True)
			ref.recompute_backward_inputs(0)
		else:
			dx = ref.backward_inputs(0, dys[0])
		ref.backward_params(0)
		return y, dx, ref.grads()

	y0, dx0, g0 = run("plain")
	for variant in ("full_fwd", "activations_bwd", "full_bwd", "simple", "selective"):
		y, dx, g = run(variant)
		assert torch.allclose(y, y0, atol=1e-10) and torch.allclose(dx, dx0, atol=1e-10)
		for name in g0:
			assert torch.allclose(g[name], g0[name], atol=1e-9), f"{variant} {name}"


def test_product_modules_agree_with_the_oracle_blocks():
	"""elf_amd.models' torch forward (what a generic executor would call) == oracle blocks."""
	from elf_amd import models
	from tests.helpers import cfg_from_stage, oracle_params_from_stage, perturb_norms

	for stage in (models.gpt_stage(2, 32, 4, 48, 8, causal=True, dtype=torch.float32), models.llama_stage(2, 32, 4, 2, 40, 8, head_dim=8, dtype=torch.float32)):
		perturb_norms(stage)
		cfg = cfg_from_stage(stage, 2)
		ref = R.RefStage(cfg, oracle_params_from_stage(stage))
		x = torch.randn(2, 8, 32)
		assert torch.allclose(stage(x), ref.forward(0, x), atol=2e-5)


@pytest.mark.parametrize("kind", ["gpt", "llama"])
def test_stage_ends_equal_library_embedding_and_linear(kind):
	"""The oracle's first / last stage pieces against library routines on the whole batch: the
	embedding is F.embedding (its gradient an index_add of the block-0 input gradient), the head
	a plain matmul behind the (closed-form) final norm; F/B/W over 3 micro-batches in any order sum
	to the full-batch gradients, and every remat variant gives them too."""
	cfg = CFG[kind]
	V_in, V_out, d = 37, 29, cfg["d_model"]
	params = R.make_params(cfg, seed=5, dtype=torch.float64)
	g = torch.Generator().manual_seed(6)
	ends = {"embed": torch.randn(V_in, d, generator=g, dtype=torch.float64), "head": torch.randn(V_out, d, generator=g, dtype=torch.float64) * 0.1,
	        "normf_g": 1 + 0.1 * torch.randn(d, generator=g, dtype=torch.float64)}
	if kind == "gpt":
		ends["normf_b"] = 0.1 * torch.randn(d, generator=g, dtype=torch.float64)
	ids = [torch.randint(0, V_in, (cfg["mb"], cfg["seq"]), generator=g) for _ in range(3)]
	ids[0][0, :4] = 3  # repeated token
	dls = [torch.randn(cfg["mb"], cfg["seq"], V_out, generator=g, dtype=torch.float64) for _ in range(3)]

	# whole batch with library routines around the (already pinned) block chain
	emb = ends["embed"].clone().requires_grad_(True)
	head = ends["head"].clone().requires_grad_(True)
	ng = ends["normf_g"].clone().requires_grad_(True)
	nb = ends["normf_b"].clone().requires_grad_(True) if kind == "gpt" else None
	x0 = F.embedding(torch.cat(ids), emb)
	x0.retain_grad()
	inner = R.RefStage(cfg, params, compute_dtype=torch.float64, acc_dtype=torch.float64)
	h = inner._model(x0)
	hn = F.layer_norm(h, (d,), ng, nb, cfg["eps"]) if kind == "gpt" else h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + cfg["eps"]) * ng
	logits = hn @ head.t()
	logits.backward(torch.cat(dls))
	want_embed = torch.zeros(V_in, d, dtype=torch.float64).index_add_(0, torch.cat(ids).reshape(-1), x0.grad.reshape(-1, d))
	assert torch.allclose(emb.grad, want_embed, atol=1e-10)

	for variant in ("plain", "full_fwd", "full_bwd"):
		ref = R.RefStage(cfg, params, compute_dtype=torch.float64, acc_dtype=torch.float64, ends=ends)
		ys = [ref.forward(m, ids[m], remat_root=variant == "full_fwd") for m in range(3)]
		assert torch.allclose(torch.cat(ys), logits.detach(), atol=1e-9)
		for m in (2, 0, 1):
			fb = variant == "full_bwd"
			assert ref.backward_inputs(m, dls[m], recompute_activations=fb, recompute_gradients=fb) is None
			if fb:
				ref.recompute_forward(m, save=True)
				ref.recompute_backward_inputs(m)
			ref.backward_params(m)
		got = ref.grads()
		assert torch.allclose(got["ends.embed"], emb.grad, atol=1e-8), variant
		assert torch.allclose(got["ends.head"], head.grad, atol=1e-8), variant
		assert torch.allclose(got["ends.normf_g"], ng.grad, atol=1e-8), variant
		if kind == "gpt":
			assert torch.allclose(got["ends.normf_b"], nb.grad, atol=1e-8), variant
		inner_grads = {f"{i}.{k}": (v.weight.grad if isinstance(v, R.SplitLinear) else v.grad) for i, b in enumerate(inner.blocks) for k, v in b.items()}
		for name, gr in inner_grads.items():
			if gr is not None:  # norm gains / biases of the blocks (their linears are split: no autograd .grad)
				assert torch.allclose(got[name], gr, atol=1e-8), (variant, name)


def test_loss_oracle_against_fp64_loops():
	"""-log softmax(x)[t] and its gradient softmax(x) - onehot(t), row by row in fp64 Python loops:
	pins sum / mean / none reductions, ignored rows and the engine's division by elements per sample."""
	from oracle import loss_ref as L

	torch.manual_seed(3)
	mb, S, V = 2, 5, 7
	x = (torch.randn(mb, S, V) * 3).to(torch.bfloat16)
	t = torch.randint(0, V, (mb, S))
	t[0, 1] = -100
	t[1, 4] = -100
	rows, grads = [], []
	for b in range(mb):
		for s in range(S):
			v = [float(x[b, s, c]) for c in range(V)]
			mx = max(v)
			den = sum(math.exp(a - mx) for a in v)
			if t[b, s] == -100:
				rows.append(0.0)
				grads.append([0.0] * V)
				continue
			rows.append(mx + math.log(den) - v[int(t[b, s])])
			grads.append([math.exp(a - mx) / den - (1.0 if c == int(t[b, s]) else 0.0) for c, a in enumerate(v)])
	live = sum(1 for r in t.view(-1) if r != -100)
	assert L.cross_entropy_ref(x, t, "none").tolist() == pytest.approx(rows, rel=1e-5, abs=1e-6)
	assert float(L.cross_entropy_ref(x, t, "sum")) == pytest.approx(sum(rows), rel=1e-5)
	assert float(L.cross_entropy_ref(x, t, "mean")) == pytest.approx(sum(rows) / live, rel=1e-5)
	loss, g = L.compute_loss_ref(x, t)
	assert g.dtype == torch.bfloat16 and g.shape == x.shape
	assert float(loss) == pytest.approx(sum(rows) / S, rel=1e-5)
	want = torch.tensor(grads).view(mb, S, V) / S
	assert torch.allclose(g.float(), want, rtol=1e-2, atol=1e-4)  # bf16 rounding of the gradient
