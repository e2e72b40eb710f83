"""Transformer-block stage modules: parameter containers with a plain-PyTorch forward.

``TransformerBlock`` has the structure and attribute names of the reference model zoo's block
(benchmarks/models/simple.py:437-468: norm1, norm2, attn.{q,k,v}_proj, proj, mlp.fc1/fc2, bias-free
linears, GELU), with dropout removed (parity runs use p = 0) and an explicit ``causal`` flag.
``LlamaBlock`` (RMSNorm, RoPE half-split, grouped-query attention, SwiGLU) has no counterpart in
the reference.  ``StageModule`` is a chain of such blocks = what one pipeline stage owns.

The torch ``forward`` here is what a generic (module-agnostic) executor would call; on an MI355X
the stage runs through ``elf_amd.execution.HipStageBlock`` instead, which reads these modules'
parameters and never calls their forward.
"""

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

__all__ = ["TransformerBlock", "LlamaBlock", "StageModule", "EndStage", "RMSNorm", "gpt_stage", "llama_stage", "gpt_end_stage"]


class Attention(nn.Module):
	"""softmax(q k^T / sqrt(D)) v over [B, H, S, D] tensors (grouped-query when k/v have fewer heads)."""

	def __init__(self, head_dim, causal=False):
		super().__init__()
		self.head_dim, self.causal = head_dim, causal

	def forward(self, q, k, v):
		return F.scaled_dot_product_attention(q, k, v, is_causal=self.causal, enable_gqa=q.shape[1] != k.shape[1])


class MultiHeadAttention(nn.Module):
	def __init__(self, dim, num_heads, num_kv_heads=None, head_dim=None, causal=False, rope_theta=None):
		super().__init__()
		self.num_heads = num_heads
		self.num_kv_heads = num_kv_heads or num_heads
		self.head_dim = head_dim or dim // num_heads
		self.q_proj = nn.Linear(dim, self.num_heads * self.head_dim, bias=False)
		self.k_proj = nn.Linear(dim, self.num_kv_heads * self.head_dim, bias=False)
		self.v_proj = nn.Linear(dim, self.num_kv_heads * self.head_dim, bias=False)
		self.attn = Attention(self.head_dim, causal)
		self.rope_theta = rope_theta

	def _rope(self, x):
		# x: [B, S, H, D]; half-split rotation with fp64 angles
		S, D = x.shape[1], x.shape[-1]
		inv = self.rope_theta ** (-torch.arange(0, D // 2, dtype=torch.float64, device=x.device) / (D // 2))
		ang = torch.arange(S, dtype=torch.float64, device=x.device)[:, None] * inv[None, :]
		cos, sin = ang.cos().float()[None, :, None, :], ang.sin().float()[None, :, None, :]
		lo, hi = x[..., : D // 2].float(), x[..., D // 2 :].float()
		return torch.cat([lo * cos - hi * sin, hi * cos + lo * sin], dim=-1).to(x.dtype)

	def forward(self, x):
		B, S, _ = x.shape
		q = self.q_proj(x).reshape(B, S, self.num_heads, self.head_dim)
		k = self.k_proj(x).reshape(B, S, self.num_kv_heads, self.head_dim)
		v = self.v_proj(x).reshape(B, S, self.num_kv_heads, self.head_dim)
		if self.rope_theta is not None:
			q, k = self._rope(q), self._rope(k)
		o = self.attn(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
		return o.transpose(1, 2).reshape(B, S, self.num_heads * self.head_dim)


class FeedForward(nn.Module):
	def __init__(self, hidden_size, ffn_dim):
		super().__init__()
		self.fc1 = nn.Linear(hidden_size, ffn_dim, bias=False)
		self.activation = nn.GELU()
		self.fc2 = nn.Linear(ffn_dim, hidden_size, bias=False)

	def forward(self, x):
		return self.fc2(self.activation(self.fc1(x)))


class TransformerBlock(nn.Module):
	"""x + proj(attn(norm1 x)), then + mlp(norm2 .): the GPT-style block of the reference."""

	arch = "gpt"

	def __init__(self, dim, num_heads=4, ffn_dim=None, causal=False, eps=1e-5):
		super().__init__()
		self.dim, self.num_heads, self.ffn_dim, self.causal, self.eps = dim, num_heads, ffn_dim or 4 * dim, causal, eps
		self.norm1 = nn.LayerNorm(dim, eps=eps)
		self.norm2 = nn.LayerNorm(dim, eps=eps)
		self.attn = MultiHeadAttention(dim, num_heads, causal=causal)
		self.proj = nn.Linear(dim, dim, bias=False)
		self.mlp = FeedForward(dim, self.ffn_dim)

	def forward(self, x):
		x = x + self.proj(self.attn(self.norm1(x)))
		return x + self.mlp(self.norm2(x))


class RMSNorm(nn.Module):
	def __init__(self, dim, eps=1e-5):
		super().__init__()
		self.eps = eps
		self.weight = nn.Parameter(torch.ones(dim))

	def forward(self, x):
		xf = x.float()
		return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight.float()).to(x.dtype)


class SwiGLU(nn.Module):
	def __init__(self, hidden_size, ffn_dim):
		super().__init__()
		self.gate_proj = nn.Linear(hidden_size, ffn_dim, bias=False)
		self.up_proj = nn.Linear(hidden_size, ffn_dim, bias=False)
		self.down_proj = nn.Linear(ffn_dim, hidden_size, bias=False)

	def forward(self, x):
		return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


class LlamaBlock(nn.Module):
	arch = "llama"

	def __init__(self, dim, num_heads, num_kv_heads, ffn_dim, head_dim=None, causal=True, rope_theta=5e5, eps=1e-5):
		super().__init__()
		self.dim, self.num_heads, self.num_kv_heads, self.ffn_dim = dim, num_heads, num_kv_heads, ffn_dim
		self.causal, self.rope_theta, self.eps = causal, rope_theta, eps
		self.norm1 = RMSNorm(dim, eps)
		self.norm2 = RMSNorm(dim, eps)
		self.attn = MultiHeadAttention(dim, num_heads, num_kv_heads, head_dim, causal, rope_theta)
		self.proj = nn.Linear(num_heads * self.attn.head_dim, dim, bias=False)
		self.mlp = SwiGLU(dim, ffn_dim)

	def forward(self, x):
		x = x + self.proj(self.attn(self.norm1(x)))
		return x + self.mlp(self.norm2(x))


class StageModule(nn.Sequential):
	"""The blocks one pipeline stage owns (all of one architecture and shape)."""

	def __init__(self, blocks, seq_len):
		super().__init__(*blocks)
		self.seq_len = seq_len


class EndStage(nn.Module):
	"""First and / or last stage of a decoder: token embedding in front of the blocks, (final norm
	and) output head behind them, with the attribute names of the reference's FullTransformer
	(benchmarks/models/simple.py:470-509: ``embed``, ``head``; it has no final norm, ``norm_f`` is an
	option for Llama-style models)."""

	def __init__(self, blocks, vocab_in=None, vocab_out=None, final_norm=False):
		super().__init__()
		b0 = blocks[0]
		self.blocks = blocks
		self.seq_len = blocks.seq_len
		self.embed = nn.Embedding(vocab_in, b0.dim) if vocab_in else None
		self.norm_f = None
		if final_norm:
			assert vocab_out, "a final norm needs an output head"
			self.norm_f = RMSNorm(b0.dim, b0.eps) if isinstance(b0, LlamaBlock) else nn.LayerNorm(b0.dim, eps=b0.eps)
		self.head = nn.Linear(b0.dim, vocab_out, bias=False) if vocab_out else None

	def forward(self, x):
		if self.embed is not None:
			x = self.embed(x)
		x = self.blocks(x)
		if self.norm_f is not None:
			x = self.norm_f(x)
		return self.head(x) if self.head is not None else x


def _init(module, seed, dtype):
	g = torch.Generator(device="cpu").manual_seed(seed)
	for m in module.modules():
		if isinstance(m, (nn.Linear, nn.Embedding)):
			with torch.no_grad():
				m.weight.copy_(torch.randn(m.weight.shape, generator=g) * 0.02)
	return module.to(dtype)


def gpt_stage(n_blocks, dim, num_heads, ffn_dim, seq_len, causal=False, seed=0, dtype=torch.bfloat16):
	return _init(StageModule([TransformerBlock(dim, num_heads, ffn_dim, causal) for _ in range(n_blocks)], seq_len), seed, dtype)


def llama_stage(n_blocks, dim, num_heads, num_kv_heads, ffn_dim, seq_len, head_dim=None, rope_theta=5e5, seed=0, dtype=torch.bfloat16):
	blocks = [LlamaBlock(dim, num_heads, num_kv_heads, ffn_dim, head_dim, True, rope_theta) for _ in range(n_blocks)]
	return _init(StageModule(blocks, seq_len), seed, dtype)


def gpt_end_stage(n_blocks, dim, num_heads, ffn_dim, seq_len, vocab_in=None, vocab_out=None, causal=True, final_norm=False, seed=0, dtype=torch.bfloat16):
	"""GPT-style first / last / only stage: (embedding +) blocks (+ final norm + head)."""
	blocks = StageModule([TransformerBlock(dim, num_heads, ffn_dim, causal) for _ in range(n_blocks)], seq_len)
	return _init(EndStage(blocks, vocab_in, vocab_out, final_norm), seed, dtype)
