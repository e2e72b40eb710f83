"""Thin torch-tensor wrappers over the kernel-level C-ABI entry points.

torch is used for device memory and streams only; every op below is one call into
libelf_stage.so on ``torch.cuda.current_stream()``.
"""

import ctypes
import math

import torch

from . import _lib

EPI_BF16, EPI_BF16_RESID, EPI_F32_ACC, EPI_F32_STORE = 0, 1, 2, 3
NORM_RMS, NORM_LAYER = 0, 1


def _stream():
	return torch.cuda.current_stream().cuda_stream


def _ptr(t):
	return 0 if t is None else t.data_ptr()


def _need(t, dtype, name):
	if not t.is_cuda:
		raise _lib.ElfStageError(f"{name}: tensor must live on the GPU (this path has no CPU implementation)")
	if t.dtype != dtype:
		raise _lib.ElfStageError(f"{name}: expected {dtype}, got {t.dtype}")
	if t.dim() >= 2 and t.stride(-1) != 1:
		raise _lib.ElfStageError(f"{name}: innermost dimension must be contiguous")


def gemm(a, b, *, a_t=False, b_t=False, out=None, epilogue=EPI_BF16, residual=None, residual_ld=None, tile_cfg=0, k_splits=0):
	"""C[M,N] (+)= sum_k A(m,k) B(n,k).  a: [M,K] (or [K,M] if a_t); b: [N,K] (or [K,N] if b_t).
	``residual_ld=0``: ``residual`` is one row of N values added to every row (a bias)."""
	_need(a, torch.bfloat16, "gemm.a")
	_need(b, torch.bfloat16, "gemm.b")
	K, M = (a.shape[0], a.shape[1]) if a_t else (a.shape[1], a.shape[0])
	Kb, N = (b.shape[0], b.shape[1]) if b_t else (b.shape[1], b.shape[0])
	if K != Kb:
		raise _lib.ElfStageError(f"gemm: reduction sizes differ ({K} vs {Kb})")
	if out is None:
		dt = torch.bfloat16 if epilogue in (EPI_BF16, EPI_BF16_RESID) else torch.float32
		out = (torch.zeros if epilogue == EPI_F32_ACC else torch.empty)((M, N), dtype=dt, device=a.device)
	lib = _lib.load()
	rc = lib.elf_gemm_bf16(int(a_t), int(b_t), M, N, K, _ptr(a), a.stride(0), _ptr(b), b.stride(0), _ptr(out), out.stride(0),
	                       epilogue, _ptr(residual), (residual.stride(0) if residual_ld is None else residual_ld) if residual is not None else 0, tile_cfg, k_splits, _stream())
	_lib.check(rc, "elf_gemm_bf16")
	return out


class _DwProblem(ctypes.Structure):
	"""``elf_dw_problem`` of include/elf_stage.h."""

	_fields_ = [("dY", ctypes.c_void_p), ("lddy", ctypes.c_int64), ("X", ctypes.c_void_p), ("ldx", ctypes.c_int64), ("acc", ctypes.c_void_p),
	            ("grad_bf16", ctypes.c_void_p), ("M", ctypes.c_int), ("N", ctypes.c_int)]


def gemm_dw_group(problems, *, scale=0.0):
	"""The weight gradients of several linear layers over the same tokens in one launch.  ``problems``: tuples
	``(dy [K, M] bf16, x [K, N] bf16, acc [M, N] fp32)`` or ``(dy, x, acc, grad_bf16 [M, N] bf16)``: ``acc += dy.T @ x``;
	with ``scale`` every ``acc`` is then multiplied by it and ``grad_bf16`` receives its bf16 rounding."""
	arr = (_DwProblem * len(problems))()
	K = problems[0][0].shape[0] if problems else 0
	for q, pr in zip(arr, problems):
		dy, x, acc = pr[0], pr[1], pr[2]
		g16 = pr[3] if len(pr) > 3 else None
		_need(dy, torch.bfloat16, "gemm_dw_group.dy")
		_need(x, torch.bfloat16, "gemm_dw_group.x")
		_need(acc, torch.float32, "gemm_dw_group.acc")
		M, N = dy.shape[1], x.shape[1]
		if dy.shape[0] != K or x.shape[0] != K:
			raise _lib.ElfStageError(f"gemm_dw_group: every problem reduces over the same {K} rows")
		if tuple(acc.shape) != (M, N) or not acc.is_contiguous() or (g16 is not None and (tuple(g16.shape) != (M, N) or not g16.is_contiguous())):
			raise _lib.ElfStageError(f"gemm_dw_group: accumulators are dense [{M}, {N}]")
		if g16 is not None:
			_need(g16, torch.bfloat16, "gemm_dw_group.grad_bf16")
		q.dY, q.lddy, q.X, q.ldx, q.acc, q.grad_bf16, q.M, q.N = _ptr(dy), dy.stride(0), _ptr(x), x.stride(0), _ptr(acc), _ptr(g16), M, N
	rc = _lib.load().elf_gemm_dw_group(len(problems), ctypes.cast(arr, ctypes.c_void_p), K, float(scale), _stream())
	_lib.check(rc, "elf_gemm_dw_group")


def gemm_turn_giveups():
	"""Waves of split-K GEMM launches on the current device that added out of turn since the library was loaded."""
	n = ctypes.c_uint64()
	_lib.check(_lib.load().elf_gemm_turn_giveups(ctypes.byref(n)), "elf_gemm_turn_giveups")
	return n.value


ACT_GELU, ACT_SWIGLU = 0, 1


def gemm_act(a, w, act):
	"""(pre, out): pre = a @ w.T; out = gelu(pre) (act 0) or silu(pre[:, :F]) * pre[:, F:] (act 1, w = [gate; up])."""
	_need(a, torch.bfloat16, "gemm_act.a")
	_need(w, torch.bfloat16, "gemm_act.w")
	M, K = a.shape
	N = w.shape[0]
	if w.shape[1] != K:
		raise _lib.ElfStageError(f"gemm_act: reduction sizes differ ({K} vs {w.shape[1]})")
	F = N // 2 if act == ACT_SWIGLU else N
	pre = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
	out = torch.empty((M, F), dtype=torch.bfloat16, device=a.device)
	rc = _lib.load().elf_gemm_act_bf16(act, M, F, K, _ptr(a), a.stride(0), _ptr(w), w.stride(0), _ptr(pre), N, _ptr(out), F, _stream())
	_lib.check(rc, "elf_gemm_act_bf16")
	return pre, out


def gemm_rope(a, w, cs, S, n_rot_heads, D, fused=True):
	"""a @ w.T with the rotary embedding applied to the first ``n_rot_heads`` heads of width ``D`` of the result
	(rows are tokens at position row % S); ``fused=False`` forces the GEMM + RoPE kernel pair (same bits)."""
	_need(a, torch.bfloat16, "gemm_rope.a")
	_need(w, torch.bfloat16, "gemm_rope.w")
	M, K = a.shape
	N = w.shape[0]
	if not fused:
		return rope_apply_(gemm(a, w), cs, S, n_rot_heads, D)
	c = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
	rc = _lib.load().elf_gemm_rope_bf16(M, N, K, _ptr(a), a.stride(0), _ptr(w), w.stride(0), _ptr(c), N, _ptr(cs), S, n_rot_heads, D, _stream())
	_lib.check(rc, "elf_gemm_rope_bf16")
	return c


def gemm_swiglu_bwd(dy, w2, gu, fused=True):
	"""dgu [M, 2F]: gradient of gu = [g | u] for d = dy @ w2 (dy [M, K], w2 [K, F]); ``fused=False`` forces the
	GEMM + activation-backward pair (same bits)."""
	for t, n in ((dy, "dy"), (w2, "w2"), (gu, "gu")):
		_need(t, torch.bfloat16, "gemm_swiglu_bwd." + n)
	M, K = dy.shape
	F = w2.shape[1]
	if w2.shape[0] != K or tuple(gu.shape) != (M, 2 * F):
		raise _lib.ElfStageError(f"gemm_swiglu_bwd: shapes {tuple(dy.shape)}, {tuple(w2.shape)}, {tuple(gu.shape)} do not fit")
	dgu = torch.empty_like(gu)
	if not fused:
		d = gemm(dy, w2, b_t=True)
		return swiglu_bwd(d, gu)
	scratch = torch.empty((M, F), dtype=torch.bfloat16, device=dy.device)
	rc = _lib.load().elf_gemm_swiglu_bwd_bf16(M, F, K, _ptr(dy), dy.stride(0), _ptr(w2), w2.stride(0), _ptr(gu), 2 * F, _ptr(dgu), 2 * F, _ptr(scratch), _stream())
	_lib.check(rc, "elf_gemm_swiglu_bwd_bf16")
	return dgu


def norm_fwd(kind, x, gamma, beta=None, eps=1e-5):
	_need(x, torch.bfloat16, "norm.x")
	T, d = x.shape
	y = torch.empty_like(x)
	stats = torch.empty((T, 2), dtype=torch.float32, device=x.device)
	rc = _lib.load().elf_norm_fwd(kind, _ptr(x), _ptr(gamma), _ptr(beta), _ptr(y), _ptr(stats), T, d, eps, _stream())
	_lib.check(rc, "elf_norm_fwd")
	return y, stats


def norm_bwd(kind, dy, x, gamma, stats, dgamma, dbeta=None, dres=None):
	T, d = x.shape
	lib = _lib.load()
	ws = torch.empty(lib.elf_norm_bwd_workspace_floats(T, d), dtype=torch.float32, device=x.device)
	dx = torch.empty_like(x)
	rc = lib.elf_norm_bwd(kind, _ptr(dy), _ptr(x), _ptr(gamma), _ptr(stats), _ptr(dres), _ptr(dx), _ptr(dgamma), _ptr(dbeta), _ptr(ws), T, d, _stream())
	_lib.check(rc, "elf_norm_bwd")
	return dx


def norm_bwd_noalloc(kind, dy, x, gamma, stats, dgamma, dx, dbeta=None, dres=None):
	"""``norm_bwd`` through the entry point that allocates nothing: the caller brings ``dx`` too."""
	T, d = x.shape
	rc = _lib.load().elf_norm_bwd_noalloc(kind, _ptr(dy), _ptr(x), _ptr(gamma), _ptr(stats), _ptr(dres), _ptr(dx), _ptr(dgamma), _ptr(dbeta), T, d, _stream())
	_lib.check(rc, "elf_norm_bwd_noalloc")
	return dx


def gelu_fwd(x):
	y = torch.empty_like(x)
	_lib.check(_lib.load().elf_gelu_fwd(_ptr(x), _ptr(y), x.numel(), _stream()), "elf_gelu_fwd")
	return y


def gelu_bwd(dy, x):
	dx = torch.empty_like(x)
	_lib.check(_lib.load().elf_gelu_bwd(_ptr(dy), _ptr(x), _ptr(dx), x.numel(), _stream()), "elf_gelu_bwd")
	return dx


def swiglu_fwd(gu):
	T, F2 = gu.shape
	h = torch.empty((T, F2 // 2), dtype=gu.dtype, device=gu.device)
	_lib.check(_lib.load().elf_swiglu_fwd(_ptr(gu), _ptr(h), T, F2 // 2, _stream()), "elf_swiglu_fwd")
	return h


def swiglu_bwd(dh, gu):
	T, F2 = gu.shape
	dgu = torch.empty_like(gu)
	_lib.check(_lib.load().elf_swiglu_bwd(_ptr(dh), _ptr(gu), _ptr(dgu), T, F2 // 2, _stream()), "elf_swiglu_bwd")
	return dgu


def rope_table(S, D, theta, device="cuda"):
	cs = torch.empty((S, D // 2, 2), dtype=torch.float32, device=device)
	_lib.check(_lib.load().elf_rope_table(_ptr(cs), S, D, float(theta), _stream()), "elf_rope_table")
	return cs


def rope_apply_(buf, cs, S, n_heads, D, backward=False):
	T, ld = buf.shape[0], buf.stride(0)
	_lib.check(_lib.load().elf_rope_apply(_ptr(buf), _ptr(cs), T, S, ld, n_heads, D, int(backward), _stream()), "elf_rope_apply")
	return buf


def scale_grads_(acc_f32, out_bf16, scale):
	_lib.check(_lib.load().elf_scale_grads(_ptr(acc_f32), _ptr(out_bf16), acc_f32.numel(), float(scale), _stream()), "elf_scale_grads")


def add(a, b):
	out = torch.empty_like(a)
	_lib.check(_lib.load().elf_add_bf16(_ptr(a), _ptr(b), _ptr(out), a.numel(), _stream()), "elf_add_bf16")
	return out


def colsum_(x, out_f32):
	"""out_f32 [N] += x.sum(0) for x: bf16 [T, N]."""
	_need(x, torch.bfloat16, "colsum.x")
	_need(out_f32, torch.float32, "colsum.out")
	lib = _lib.load()
	ws = torch.empty(max(1, lib.elf_colsum_workspace_floats(x.shape[0], x.shape[1])), dtype=torch.float32, device=x.device)
	_lib.check(lib.elf_colsum_bf16(_ptr(x), x.stride(0), _ptr(out_f32), x.shape[0], x.shape[1], _ptr(ws), _stream()), "elf_colsum_bf16")
	return out_f32


def embedding_fwd(ids, table):
	"""ids: int64 [T] (any shape, flattened); table: bf16 [V, d] -> bf16 [T, d]."""
	_need(table, torch.bfloat16, "embedding.table")
	if ids.dtype != torch.int64 or not ids.is_cuda:
		raise _lib.ElfStageError("embedding.ids must be an int64 GPU tensor")
	ids = ids.contiguous()
	out = torch.empty(ids.numel(), table.shape[1], dtype=torch.bfloat16, device=table.device)
	_lib.check(_lib.load().elf_embedding_fwd(_ptr(ids), _ptr(table), _ptr(out), ids.numel(), table.shape[1], table.shape[0], _stream()), "elf_embedding_fwd")
	return out


def embedding_bwd_(ids, dx, dtable):
	"""dtable (fp32 [V, d]) += scatter of dx (bf16 [T, d]) by ids."""
	_need(dx, torch.bfloat16, "embedding.dx")
	_need(dtable, torch.float32, "embedding.dtable")
	ids = ids.contiguous()
	_lib.check(_lib.load().elf_embedding_bwd(_ptr(ids), _ptr(dx), _ptr(dtable), ids.numel(), dtable.shape[1], dtable.shape[0], _stream()), "elf_embedding_bwd")
	return dtable


def attn_fwd(qkv, B, S, Hq, Hkv, D, causal, scale=None):
	"""qkv: [B*S, (Hq+2*Hkv)*D] packed projections. Returns (o [B*S, Hq*D], lse [B,Hq,S])."""
	_need(qkv, torch.bfloat16, "attn.qkv")
	T, ld = qkv.shape[0], qkv.stride(0)
	scale = scale if scale is not None else 1.0 / math.sqrt(D)
	o = torch.empty((T, Hq * D), dtype=torch.bfloat16, device=qkv.device)
	lse = torch.empty((B, Hq, S), dtype=torch.float32, device=qkv.device)
	q, k, v = qkv[:, : Hq * D], qkv[:, Hq * D : (Hq + Hkv) * D], qkv[:, (Hq + Hkv) * D :]
	rc = _lib.load().elf_attn_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), ld, ld, ld, o.stride(0), B, S, Hq, Hkv, D, int(causal), scale, _stream())
	_lib.check(rc, "elf_attn_fwd")
	return o, lse


def attn_bwd(qkv, o, do, lse, B, S, Hq, Hkv, D, causal, scale=None, rope_cs=None):
	"""Returns dqkv packed like qkv.  ``rope_cs``: the q and k heads of ``qkv`` are rotated (``rope_apply_`` with this
	table); dq and dk then come out with the rotation's backward applied."""
	T, ld = qkv.shape[0], qkv.stride(0)
	scale = scale if scale is not None else 1.0 / math.sqrt(D)
	lib = _lib.load()
	ws = torch.empty(lib.elf_attn_bwd_workspace_bytes(B, S, Hq, D, int(causal)), dtype=torch.uint8, device=qkv.device)
	dqkv = torch.empty_like(qkv)
	q, k, v = qkv[:, : Hq * D], qkv[:, Hq * D : (Hq + Hkv) * D], qkv[:, (Hq + Hkv) * D :]
	dq, dk, dv = dqkv[:, : Hq * D], dqkv[:, Hq * D : (Hq + Hkv) * D], dqkv[:, (Hq + Hkv) * D :]
	args = (_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(ws),
	        ld, ld, ld, o.stride(0), do.stride(0), dqkv.stride(0), dqkv.stride(0), dqkv.stride(0), B, S, Hq, Hkv, D, int(causal), scale)
	if rope_cs is None:
		_lib.check(lib.elf_attn_bwd(*args, _stream()), "elf_attn_bwd")
	else:
		_lib.check(lib.elf_attn_bwd_rope(*args, _ptr(rope_cs), _stream()), "elf_attn_bwd_rope")
	return dqkv
