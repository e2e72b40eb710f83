"""Shared helpers of the parity tests (oracle <-> product glue)."""

import os
import torch

from oracle import stage_ref as R


def cfg_from_stage(stage, mb):
	b0 = stage[0]
	llama = type(b0).__name__ == "LlamaBlock"
	return {
		"arch": R.ARCH_LLAMA if llama else R.ARCH_GPT, "n_blocks": len(stage), "d_model": b0.dim, "n_heads": b0.attn.num_heads,
		"n_kv_heads": b0.attn.num_kv_heads, "head_dim": b0.attn.head_dim, "ffn": b0.ffn_dim, "seq": stage.seq_len, "mb": mb,
		"causal": bool(b0.causal), "eps": b0.eps, "rope_theta": getattr(b0, "rope_theta", 0.0),
	}


def oracle_params_from_stage(stage):
	"""Per block, the oracle's fused parameter dict read from the product module (bf16 values)."""
	out = []
	for b in stage:
		llama = type(b).__name__ == "LlamaBlock"
		p = {
			"norm1_g": b.norm1.weight, "norm2_g": b.norm2.weight,
			"wqkv": torch.cat([b.attn.q_proj.weight, b.attn.k_proj.weight, b.attn.v_proj.weight], 0), "wo": b.proj.weight,
		}
		if llama:
			p["w1"] = torch.cat([b.mlp.gate_proj.weight, b.mlp.up_proj.weight], 0)
			p["w2"] = b.mlp.down_proj.weight
		else:
			p["norm1_b"], p["norm2_b"] = b.norm1.bias, b.norm2.bias
			p["w1"], p["w2"] = b.mlp.fc1.weight, b.mlp.fc2.weight
		out.append({k: v.detach().clone() for k, v in p.items()})
	return out


def product_grads(stage, which="main_grad"):
	"""{"<block>.<oracle name>": gradient} from the product module, fused like the oracle's."""
	out = {}
	for i, b in enumerate(stage):
		llama = type(b).__name__ == "LlamaBlock"
		g = lambda p: getattr(p, which)
		out[f"{i}.norm1_g"], out[f"{i}.norm2_g"] = g(b.norm1.weight), g(b.norm2.weight)
		out[f"{i}.wqkv"] = torch.cat([g(b.attn.q_proj.weight), g(b.attn.k_proj.weight), g(b.attn.v_proj.weight)], 0)
		out[f"{i}.wo"] = g(b.proj.weight)
		if llama:
			out[f"{i}.w1"] = torch.cat([g(b.mlp.gate_proj.weight), g(b.mlp.up_proj.weight)], 0)
			out[f"{i}.w2"] = g(b.mlp.down_proj.weight)
		else:
			out[f"{i}.norm1_b"], out[f"{i}.norm2_b"] = g(b.norm1.bias), g(b.norm2.bias)
			out[f"{i}.w1"], out[f"{i}.w2"] = g(b.mlp.fc1.weight), g(b.mlp.fc2.weight)
	return out


def perturb_norms(stage, seed=7):
	"""Non-trivial norm gains / biases so that their gradients are exercised."""
	g = torch.Generator(device="cpu").manual_seed(seed)
	with torch.no_grad():
		for b in stage:
			for n in (b.norm1, b.norm2):
				n.weight.copy_((1 + 0.1 * torch.randn(n.weight.shape, generator=g)).to(n.weight.dtype))
				if getattr(n, "bias", None) is not None:
					n.bias.copy_((0.1 * torch.randn(n.bias.shape, generator=g)).to(n.bias.dtype))


def assert_close(got, ref, what, rel_max=2e-2, rel_fro=1e-2):
	got, ref = got.float().cpu(), ref.float().cpu()
	assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
	assert torch.isfinite(got).all(), f"{what}: non-finite values"
	scale = ref.abs().max().item() + 1e-12
	err = (got - ref).abs().max().item()
	fro = ((got - ref).norm() / (ref.norm() + 1e-12)).item()
	if os.environ.get("ELF_TEST_MARGINS"):  # how far inside the bounds each comparison lands (pytest -s)
		print(f"[margin] {what}: max {err / scale:.4f} of {rel_max}, fro {fro:.4f} of {rel_fro}", flush=True)
	assert err <= rel_max * scale, f"{what}: max abs err {err:.4g} > {rel_max} * {scale:.4g}"
	assert fro <= rel_fro, f"{what}: relative Frobenius error {fro:.4g} > {rel_fro}"
	return err / scale, fro


def assert_close_dev(got, ref, what, rel_max=2e-2, rel_fro=1e-2):
	"""``assert_close`` without leaving the device (for tensors of hundreds of MB)."""
	assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
	diff = got.float() - ref.float()
	assert torch.isfinite(diff).all().item(), f"{what}: non-finite values"
	scale = ref.abs().max().item() + 1e-12
	err = diff.abs().max().item()
	fro = (diff.double().norm() / (ref.double().norm() + 1e-12)).item()
	if os.environ.get("ELF_TEST_MARGINS"):
		print(f"[margin] {what}: max {err / scale:.4f} of {rel_max}, fro {fro:.4f} of {rel_fro}", flush=True)
	assert err <= rel_max * scale, f"{what}: max abs err {err:.4g} > {rel_max} * {scale:.4g}"
	assert fro <= rel_fro, f"{what}: relative Frobenius error {fro:.4g} > {rel_fro}"
	return err / scale, fro
