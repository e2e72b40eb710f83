"""Parity of every HIP kernel (through the C ABI) against a plain PyTorch fp32 evaluation of
the same op on the same bf16-rounded inputs.  Tolerance: the path's bf16 bar (rel 2e-2 of the
reference's max magnitude per tensor), plus a much tighter Frobenius-norm bound that catches
systematic errors (a dropped term, a wrong sign or index)."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

REL_MAX = 2e-2   # elementwise, relative to max |ref|
REL_FRO = 6e-3   # Frobenius, bf16 output rounding is ~2^-9 relative


def _close(got, ref, rel_max=REL_MAX, rel_fro=REL_FRO, what=""):
	got = got.float()
	ref = ref.float()
	assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
	assert torch.isfinite(got).all(), f"{what}: non-finite output"
	scale = ref.abs().max().item() + 1e-12
	err = (got - ref).abs().max().item()
	fro = ((got - ref).norm() / (ref.norm() + 1e-12)).item()
	assert err <= rel_max * scale, f"{what}: max err {err:.4g} vs scale {scale:.4g}"
	assert fro <= rel_fro, f"{what}: relative Frobenius error {fro:.4g}"


def _randn(*shape, seed=0, scale=1.0):
	g = torch.Generator(device="cpu").manual_seed(seed)
	return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16).cuda()


@pytest.fixture(scope="module")
def K():
	from elf_amd import kernels

	return kernels


@pytest.mark.parametrize("layout", ["nt", "nn", "tn"])
@pytest.mark.parametrize("shape", [(256, 256, 64), (512, 768, 256), (1024, 2304, 768), (2048, 1024, 4096)])
@pytest.mark.parametrize("tile_cfg", [0, 1, 2, 3, 5, 7, 8])
def test_gemm_layouts(K, layout, shape, tile_cfg):
	M, N, Kd = shape
	if tile_cfg in (1, 5, 7) and (M % 256 or N % 256):
		pytest.skip("tile does not divide")
	if tile_cfg == 8 and N % 256:
		pytest.skip("the 128x256 direct-to-LDS tile needs N % 256 == 0")
	A = _randn(M, Kd, seed=1)
	B = _randn(N, Kd, seed=2, scale=0.05)
	ref = A.float() @ B.float().t()
	if layout == "nt":
		out = K.gemm(A, B, tile_cfg=tile_cfg)
	elif layout == "nn":
		out = K.gemm(A, B.t().contiguous(), b_t=True, tile_cfg=tile_cfg)
	else:
		out = K.gemm(A.t().contiguous(), B.t().contiguous(), a_t=True, b_t=True, tile_cfg=tile_cfg)
	_close(out, ref, what=f"gemm {layout} {shape} cfg{tile_cfg}")


def test_gemm_epilogues(K):
	M, N, Kd = 512, 768, 512
	A = _randn(M, Kd, seed=3)
	B = _randn(N, Kd, seed=4, scale=0.05)
	R = _randn(M, N, seed=5)
	ref = A.float() @ B.float().t()
	_close(K.gemm(A, B, epilogue=K.EPI_BF16_RESID, residual=R), ref + R.float(), what="resid")
	_close(K.gemm(A, B, epilogue=K.EPI_F32_STORE), ref, rel_fro=1e-5, rel_max=1e-5, what="f32 store")
	# fp32 accumulation across calls (the deferred weight-gradient pattern), with and without split-K
	for ks in (1, 4):
		acc = torch.full((M, N), 0.25, dtype=torch.float32, device="cuda")
		for _ in range(3):
			K.gemm(A, B, out=acc, epilogue=K.EPI_F32_ACC, k_splits=ks)
		_close(acc, 3 * ref + 0.25, rel_fro=1e-5, rel_max=1e-5, what=f"f32 acc ks={ks}")


@pytest.mark.parametrize("tile_cfg", [7, 8])
@pytest.mark.parametrize("layout", ["nt", "tn", "nn"])
def test_gemm_direct_to_lds_epilogues_and_k_split(K, tile_cfg, layout):
	"""The direct-to-LDS kernels (256x256 and 128x256 tiles): every epilogue, short K (1 and
	2 slices: the loop's loads past the end of K), and the K split with fp32 atomics."""
	M, N = (384, 768) if tile_cfg == 8 else (512, 768)
	for Kd in (64, 128, 1024):
		A = _randn(M, Kd, seed=21)
		B = _randn(N, Kd, seed=22, scale=0.05)
		R = _randn(M, N, seed=23)
		ref = A.float() @ B.float().t()
		if layout == "nt":
			kw = dict(tile_cfg=tile_cfg)
			a, b = A, B
		elif layout == "nn":
			kw = dict(tile_cfg=tile_cfg, b_t=True)
			a, b = A, B.t().contiguous()
		else:
			kw = dict(tile_cfg=tile_cfg, a_t=True, b_t=True)
			a, b = A.t().contiguous(), B.t().contiguous()
		_close(K.gemm(a, b, **kw), ref, what=f"bf16 K={Kd}")
		_close(K.gemm(a, b, epilogue=K.EPI_BF16_RESID, residual=R, **kw), ref + R.float(), what=f"resid K={Kd}")
		_close(K.gemm(a, b, epilogue=K.EPI_F32_STORE, **kw), ref, rel_fro=1e-5, rel_max=1e-5, what=f"f32 store K={Kd}")
		for ks in (1, 2, 4):
			acc = torch.full((M, N), 0.25, dtype=torch.float32, device="cuda")
			for _ in range(2):
				K.gemm(a, b, out=acc, epilogue=K.EPI_F32_ACC, k_splits=ks, **kw)
			_close(acc, 2 * ref + 0.25, rel_fro=1e-5, rel_max=1e-5, what=f"f32 acc K={Kd} ks={ks}")


@pytest.mark.parametrize("dims,ks", [((1024, 1536, 8192), 0), ((768, 768, 8192), 0), ((2304, 768, 8192), 0), ((2048, 2048, 4096), 0), ((512, 768, 4096), 8), ((4096, 6144, 8192), 0), ((2048, 2304, 2048), 4)])
def test_gemm_k_split_is_bit_reproducible(K, dims, ks):
	"""Weight-gradient GEMMs whose tiles are shared by several workgroups along K (all tiles split, only the
	tail of the last round split, an explicit split): the workgroups of a tile add in turn, so repeated runs
	into equal accumulators give equal bits, and the sum is the unsplit one within fp32 rounding."""
	M, N, Kd = dims
	A = _randn(Kd, M, seed=71)
	B = _randn(Kd, N, seed=72, scale=0.05)
	start = torch.randn(M, N, device="cuda", generator=torch.Generator(device="cuda").manual_seed(73))
	runs = []
	for _ in range(4):
		acc = start.clone()
		K.gemm(A, B, a_t=True, b_t=True, out=acc, epilogue=K.EPI_F32_ACC, k_splits=ks)
		runs.append(acc)
	for r in runs[1:]:
		assert torch.equal(r, runs[0]), "split-K accumulation must not depend on the order in which workgroups finish"
	one = start.clone()
	K.gemm(A, B, a_t=True, b_t=True, out=one, epilogue=K.EPI_F32_ACC, k_splits=1)
	assert ((runs[0] - one).norm() / one.norm()).item() <= 1e-5


@pytest.mark.parametrize("shape", [(256, 256, 128), (512, 768, 256), (4096, 1280, 1152), (8192, 4096, 1024), (2048, 28672, 256)])
def test_persistent_forward_gemm_equals_the_tile_kernel_bit_for_bit(K, monkeypatch, shape):
	"""Forward GEMMs on 256x256 tiles run as persistent workgroups that walk several tiles and store from registers
	(operands swapped on the MFMA, permuted weight rows); the one-tile-per-workgroup kernel with its LDS-staged epilogue
	(ELF_NO_PERSISTENT_GEMM=1) forms the same products in the same order: equal bits for every epilogue, from one tile
	per workgroup (1, 6 tiles) to several with a ragged last round (80, 512, 896 tiles), also against fp32 torch."""
	M, N, Kd = shape
	a, w, r, bias = _randn(M, Kd, seed=61), _randn(N, Kd, seed=62, scale=0.05), _randn(M, N, seed=63), _randn(1, N, seed=64)
	F = N // 2
	S, D = 256, 128
	cs = K.rope_table(S, D, 5e5)
	n_rot = (N // D) // 2

	def run():
		return (K.gemm(a, w, tile_cfg=7), K.gemm(a, w, tile_cfg=7, epilogue=K.EPI_BF16_RESID, residual=r),
		        K.gemm(a, w, tile_cfg=7, epilogue=K.EPI_BF16_RESID, residual=bias, residual_ld=0), *K.gemm_act(a, w, K.ACT_SWIGLU), K.gemm_rope(a, w, cs, S, n_rot, D))

	new = run()
	monkeypatch.setenv("ELF_NO_PERSISTENT_GEMM", "1")
	old = run()
	monkeypatch.delenv("ELF_NO_PERSISTENT_GEMM")
	for i, (x, y) in enumerate(zip(new, old)):
		assert torch.equal(x, y), f"output {i} of the persistent kernel differs from the tile kernel's at {shape}"
	ref = a.float() @ w.float().t()
	_close(new[0], ref, what="persistent bf16")
	_close(new[1], ref + r.float(), what="persistent residual")
	_close(new[2], ref + bias.float(), what="persistent bias row")
	_close(new[4], torch.nn.functional.silu(new[3][:, :F].float()) * new[3][:, F:].float(), what="persistent swiglu")


def test_gemm_strided_views(K):
	# operands that are column slices of wider buffers (leading dimension > row length)
	big = _randn(512, 1024, seed=6)
	A = big[:, 128:640]                      # [512, 512], ld 1024
	Bw = _randn(256, 512, seed=7, scale=0.05)
	out = torch.zeros(512, 512, dtype=torch.bfloat16, device="cuda")
	K.gemm(A, Bw, out=out[:, 256:])          # writes a column slice
	_close(out[:, 256:], A.float() @ Bw.float().t(), what="strided")
	assert out[:, :256].abs().max().item() == 0


def test_gemm_rejects_bad_shapes(K):
	from elf_amd._lib import ElfStageError

	A = _randn(100, 64)
	B = _randn(64, 64)
	with pytest.raises(ElfStageError):
		K.gemm(A, B)
	with pytest.raises(ElfStageError):
		K.gemm(_randn(64, 72), _randn(64, 72))  # K not a multiple of 64
	with pytest.raises(ElfStageError):
		K.gemm(A.cpu(), B)


@pytest.mark.parametrize("d", [256, 768, 1024, 2048, 4096, 8192])
@pytest.mark.parametrize("kind", ["rms", "ln"])
def test_norm_fwd_bwd(K, d, kind):
	T = 515 if d <= 2048 else 130  # ragged row count on purpose
	x = _randn(T, d, seed=10) * 1.5 + 0.25
	x = x.to(torch.bfloat16)
	gamma = (1 + 0.1 * torch.randn(d, generator=torch.Generator().manual_seed(11))).to(torch.bfloat16).cuda()
	beta = (0.1 * torch.randn(d, generator=torch.Generator().manual_seed(12))).to(torch.bfloat16).cuda()
	dy = _randn(T, d, seed=13)
	dres = _randn(T, d, seed=14)
	eps = 1e-5
	xr = x.float().requires_grad_(True)
	gr = gamma.float().requires_grad_(True)
	br = beta.float().requires_grad_(True)
	if kind == "rms":
		yr = xr * torch.rsqrt(xr.pow(2).mean(-1, keepdim=True) + eps) * gr
	else:
		yr = torch.nn.functional.layer_norm(xr, (d,), gr, br, eps)
	yr.backward(dy.float())
	k = K.NORM_RMS if kind == "rms" else K.NORM_LAYER
	y, stats = K.norm_fwd(k, x, gamma, beta if kind == "ln" else None, eps)
	_close(y, yr.detach(), what="norm fwd")
	dgamma = torch.full((d,), 0.5, dtype=torch.float32, device="cuda")
	dbeta = torch.full((d,), -0.5, dtype=torch.float32, device="cuda")
	dx = K.norm_bwd(k, dy, x, gamma, stats, dgamma, dbeta if kind == "ln" else None, dres)
	_close(dx, xr.grad + dres.float(), what="norm dx")
	_close(dgamma - 0.5, gr.grad, rel_fro=1e-4, rel_max=1e-3, what="dgamma")
	if kind == "ln":
		_close(dbeta + 0.5, br.grad, rel_fro=1e-4, rel_max=1e-3, what="dbeta")
	dx2 = K.norm_bwd(k, dy, x, gamma, stats, dgamma, dbeta if kind == "ln" else None, None)
	_close(dx2, xr.grad, what="norm dx no residual")


def test_gelu_swiglu(K):
	x = _randn(300, 1024, seed=20) * 2
	x = x.to(torch.bfloat16)
	dy = _randn(300, 1024, seed=21)
	xr = x.float().requires_grad_(True)
	yr = torch.nn.functional.gelu(xr)
	yr.backward(dy.float())
	_close(K.gelu_fwd(x), yr.detach(), what="gelu")
	_close(K.gelu_bwd(dy, x), xr.grad, what="gelu bwd")
	F = 512
	gu = x  # [300, 2F]
	dh = _randn(300, F, seed=22)
	gur = gu.float().requires_grad_(True)
	hr = torch.nn.functional.silu(gur[:, :F]) * gur[:, F:]
	hr.backward(dh.float())
	_close(K.swiglu_fwd(gu), hr.detach(), what="swiglu")
	_close(K.swiglu_bwd(dh, gu), gur.grad, what="swiglu bwd")


@pytest.mark.parametrize("act", ["gelu", "swiglu"])
@pytest.mark.parametrize("shape", [(2048, 6144, 128), (1024, 4096, 192), (1536, 8192, 64), (320, 1024, 128)])
def test_gemm_with_activation_epilogue(K, act, shape):
	"""Up-projection with its activation (SwiGLU: in the GEMM epilogue; GELU: GEMM + activation kernel
	behind the same entry point): against fp32 torch, and bit for bit against the GEMM followed by the
	activation kernel.  Shapes: 256x256 tiles, 128x256 tiles, a single K slice, and one the fused tiles
	do not cover (the library then runs the two kernels itself)."""
	M, N, Kd = shape
	A = _randn(M, Kd, seed=41)
	W = _randn(N, Kd, seed=42, scale=0.12)
	code = K.ACT_GELU if act == "gelu" else K.ACT_SWIGLU
	pre, out = K.gemm_act(A, W, code)
	ref_pre = A.float() @ W.float().t()
	_close(pre, ref_pre, what="pre-activation")
	p32 = pre.float()
	if act == "gelu":
		ref_out = torch.nn.functional.gelu(p32)
		two = K.gelu_fwd(K.gemm(A, W))
	else:
		F = N // 2
		ref_out = torch.nn.functional.silu(p32[:, :F]) * p32[:, F:]
		two = K.swiglu_fwd(K.gemm(A, W))
	_close(out, ref_out, what="activated")
	assert torch.equal(pre, K.gemm(A, W)), "pre-activation differs from the plain GEMM"
	assert torch.equal(out, two), "fused activation differs from the separate kernel"


@pytest.mark.parametrize("shape", [(8192, 2048, 256), (4096, 3072, 64), (512, 1024, 128)])
def test_gemm_with_swiglu_backward_epilogue(K, shape):
	"""dX of the down projection with the SwiGLU's backward in the GEMM epilogue: against fp32 torch autograd
	of silu(g) * u, and bit for bit against the GEMM followed by the activation-backward kernel.  Shapes: two the
	fused tiles cover (one with a single K slice) and one they do not (the library runs the two kernels itself)."""
	M, F, Kd = shape
	dY = _randn(M, Kd, seed=51)
	W2 = _randn(Kd, F, seed=52, scale=0.1)
	gu = _randn(M, 2 * F, seed=53)
	dgu = K.gemm_swiglu_bwd(dY, W2, gu)
	two = K.gemm_swiglu_bwd(dY, W2, gu, fused=False)
	assert torch.equal(dgu, two), "fused activation backward differs from the separate kernels"
	d = (dY.float() @ W2.float()).to(torch.bfloat16).float()
	g32 = gu.float().requires_grad_(True)
	(torch.nn.functional.silu(g32[:, :F]) * g32[:, F:]).backward(d)
	_close(dgu, g32.grad, what="gradient of [g | u]")


@pytest.mark.parametrize("shape", [(8192, 6144, 256, 4096, 32, 8, 128), (4096, 2048, 64, 1024, 12, 4, 64), (2048, 4096, 128, 512, 5, 3, 128), (512, 1024, 128, 256, 4, 2, 128)])
def test_gemm_with_rope_epilogue(K, shape):
	"""The packed q | k | v projection with the rotary embedding of its q and k heads in the GEMM epilogue:
	bit for bit against the GEMM followed by the RoPE kernel, and against an fp32 rotation (fp64 angles) of
	the rounded projection.  Shapes: 256x256 tiles with heads of 128 (the Llama-3-8B projection), 128x256
	tiles with heads of 64, an odd number of rotated heads (the v heads start in the middle of a tile), and
	one the fused tiles do not cover (the library runs the two kernels itself)."""
	M, N, Kd, S, Hq, Hkv, D = shape
	assert (Hq + 2 * Hkv) * D <= N
	A = _randn(M, Kd, seed=61)
	W = _randn(N, Kd, seed=62, scale=0.1)
	cs = K.rope_table(S, D, 5e5)
	got = K.gemm_rope(A, W, cs, S, Hq + Hkv, D)
	two = K.gemm_rope(A, W, cs, S, Hq + Hkv, D, fused=False)
	assert torch.equal(got, two), "fused rotation differs from the separate kernel"
	plain = K.gemm(A, W)
	nrot = (Hq + Hkv) * D
	assert torch.equal(got[:, nrot:], plain[:, nrot:]), "columns after the rotated heads must be the plain projection"
	ref = _rope_ref(plain[:, :nrot].float().view(M, Hq + Hkv, D), S, D, 5e5).reshape(M, nrot)
	_close(got[:, :nrot], ref, what="rotated projection")


def test_gemm_with_activation_strided_outputs(K):
	# outputs that are column slices of wider buffers, as a caller that packs activations would pass
	from elf_amd import _lib

	M, F, Kd = 1024, 2048, 128
	A = _randn(M, Kd, seed=43)
	W = _randn(2 * F, Kd, seed=44, scale=0.12)
	pre = torch.zeros(M, 2 * F + 64, dtype=torch.bfloat16, device="cuda")
	out = torch.zeros(M, F + 64, dtype=torch.bfloat16, device="cuda")
	rc = _lib.load().elf_gemm_act_bf16(K.ACT_SWIGLU, M, F, Kd, A.data_ptr(), Kd, W.data_ptr(), Kd, pre.data_ptr(), pre.stride(0),
	                                   out.data_ptr(), out.stride(0), torch.cuda.current_stream().cuda_stream)
	_lib.check(rc, "elf_gemm_act_bf16")
	p2, o2 = K.gemm_act(A, W, K.ACT_SWIGLU)
	assert torch.equal(pre[:, : 2 * F], p2) and torch.equal(out[:, :F], o2)
	assert pre[:, 2 * F :].abs().max().item() == 0 and out[:, F:].abs().max().item() == 0


def _rope_ref(x, S, D, theta):
	# x: [T, H, D] fp32; half-split rotation, angles in fp64
	T = x.shape[0]
	pos = (torch.arange(T, device=x.device) % S).double()
	inv = theta ** (-torch.arange(0, D // 2, device=x.device).double() / (D // 2))
	ang = pos[:, None] * inv[None, :]
	cos, sin = ang.cos().float()[:, None, :], ang.sin().float()[:, None, :]
	a, b = x[..., : D // 2], x[..., D // 2 :]
	return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)


def test_rope(K):
	S, B, Hq, Hkv, D, theta = 256, 2, 4, 2, 128, 5e5
	T = B * S
	qkv = _randn(T, (Hq + 2 * Hkv) * D, seed=30)
	cs = K.rope_table(S, D, theta)
	ref = qkv.float().clone()
	nrot = Hq + Hkv
	ref[:, : nrot * D] = _rope_ref(ref[:, : nrot * D].reshape(T, nrot, D), S, D, theta).reshape(T, -1)
	out = qkv.clone()
	K.rope_apply_(out, cs, S, nrot, D)
	_close(out, ref, what="rope fwd")
	assert torch.equal(out[:, nrot * D :], qkv[:, nrot * D :]), "v columns must be untouched"
	# backward = inverse rotation: rotating the forward result back returns the input
	back = out.clone()
	K.rope_apply_(back, cs, S, nrot, D, backward=True)
	_close(back, qkv, what="rope inverse")


def test_scale_and_add(K):
	acc = torch.randn(1000003, device="cuda")
	ref = acc.clone() * 0.125
	out = torch.empty(1000003, dtype=torch.bfloat16, device="cuda")
	K.scale_grads_(acc, out, 0.125)
	assert torch.equal(acc, ref)
	assert torch.equal(out, ref.to(torch.bfloat16))
	a, b = _randn(4096, 64, seed=40), _randn(4096, 64, seed=41)
	assert torch.equal(K.add(a, b), (a.float() + b.float()).to(torch.bfloat16))


def _attn_ref(qkv, B, S, Hq, Hkv, D, causal, do=None):
	T = B * S
	x = qkv.float().requires_grad_(True)
	q = x[:, : Hq * D].reshape(B, S, Hq, D).transpose(1, 2)
	k = x[:, Hq * D : (Hq + Hkv) * D].reshape(B, S, Hkv, D).transpose(1, 2)
	v = x[:, (Hq + Hkv) * D :].reshape(B, S, Hkv, D).transpose(1, 2)
	G = Hq // Hkv
	k = k.repeat_interleave(G, dim=1)
	v = v.repeat_interleave(G, dim=1)
	s = (q @ k.transpose(-1, -2)) / math.sqrt(D)
	if causal:
		mask = torch.ones(S, S, dtype=torch.bool, device=x.device).tril()
		s = s.masked_fill(~mask, float("-inf"))
	lse = torch.logsumexp(s, dim=-1)
	o = (torch.softmax(s, dim=-1) @ v).transpose(1, 2).reshape(T, Hq * D)
	if do is not None:
		o.backward(do.float())
		return o.detach(), lse.detach(), x.grad
	return o.detach(), lse.detach(), None


@pytest.mark.parametrize("cfg", [
	(1, 128, 2, 2, 64, False), (2, 256, 4, 4, 64, False), (2, 256, 4, 2, 128, True),
	(1, 512, 8, 2, 128, True), (1, 384, 2, 1, 64, True), (2, 128, 4, 4, 128, False),
	(1, 1024, 4, 1, 128, True), (1, 1024, 3, 3, 64, False), (1, 640, 2, 2, 128, True),
])
def test_attention_fwd_bwd(K, cfg):
	B, S, Hq, Hkv, D, causal = cfg
	T = B * S
	qkv = _randn(T, (Hq + 2 * Hkv) * D, seed=50)
	do = _randn(T, Hq * D, seed=51)
	o_ref, lse_ref, dqkv_ref = _attn_ref(qkv, B, S, Hq, Hkv, D, causal, do)
	o, lse = K.attn_fwd(qkv, B, S, Hq, Hkv, D, causal)
	_close(o, o_ref, what=f"attn fwd {cfg}")
	_close(lse, lse_ref, rel_fro=1e-3, rel_max=1e-2, what="lse")
	dqkv = K.attn_bwd(qkv, o, do, lse, B, S, Hq, Hkv, D, causal)
	for name, sl in (("dq", slice(0, Hq * D)), ("dk", slice(Hq * D, (Hq + Hkv) * D)), ("dv", slice((Hq + Hkv) * D, None))):
		_close(dqkv[:, sl], dqkv_ref[:, sl], rel_fro=1.5e-2, what=f"attn {name} {cfg}")
	# no atomics anywhere in the backward: a second run gives the same bits
	assert torch.equal(dqkv, K.attn_bwd(qkv, o, do, lse, B, S, Hq, Hkv, D, causal))
	# the backward of a rotary embedding on q and k, applied where dQ and dK are stored: the bits of the plain
	# backward followed by the RoPE kernel's backward pass
	cs = K.rope_table(S, D, 5e5)
	fused = K.attn_bwd(qkv, o, do, lse, B, S, Hq, Hkv, D, causal, rope_cs=cs)
	assert torch.equal(fused, K.rope_apply_(dqkv.clone(), cs, S, Hq + Hkv, D, backward=True))


@pytest.mark.parametrize("D,causal,ramp,gain", [(128, True, 6.0, 1.0), (128, False, 6.0, 1.0), (64, True, 6.0, 1.0), (128, True, 0.0, 6.0),
                                               (128, False, -6.0, 3.0), (64, False, 0.0, 6.0)])
def test_attention_forward_with_scores_that_climb_along_the_keys(K, D, causal, ramp, gain):
	"""The forward's softmax takes its exponentials against a reference point that follows the running maximum only
	when it has to.  Here it has to, again and again: a component of k that grows (ramp > 0) or falls (ramp < 0) with the
	key position against a constant component of q moves the row maxima by many powers of two from tile to tile, and
	gain scales everything to scores of several hundred.  Output and log-sum-exp against the fp32 softmax."""
	B, S, Hq, Hkv = 2, 1024, 4, 2
	T = B * S
	qkv = _randn(T, (Hq + 2 * Hkv) * D, seed=60).float() * gain
	pos = (torch.arange(T, device="cuda") % S).float() / S  # 0 .. 1 along each sequence
	for h in range(Hq):
		qkv[:, h * D] = 4.0
	for h in range(Hkv):
		qkv[:, (Hq + h) * D] = ramp * pos * math.sqrt(D)  # adds ramp * 4 * pos to every score: up to 35 powers of two
	qkv = qkv.to(torch.bfloat16)
	o_ref, lse_ref, _ = _attn_ref(qkv, B, S, Hq, Hkv, D, causal)
	o, lse = K.attn_fwd(qkv, B, S, Hq, Hkv, D, causal)
	assert torch.isfinite(o.float()).all() and torch.isfinite(lse).all()
	_close(o, o_ref, what=f"attn fwd, climbing scores D={D} causal={causal} ramp={ramp} gain={gain}")
	_close(lse, lse_ref, rel_fro=1e-3, rel_max=1e-2, what="lse")
	assert torch.equal(o, K.attn_fwd(qkv, B, S, Hq, Hkv, D, causal)[0])


@pytest.mark.parametrize("T,N,ld", [(8192, 768, 768), (1000, 2304, 2304), (7, 64, 128), (4096, 8, 8), (333, 4104, 4104)])
def test_colsum_is_exact_to_rounding_and_repeatable(K, T, N, ld):
	"""The bias gradient of a split linear layer: column sums of a bf16 [T, N] view (row stride ld) added to an fp32
	accumulator, equal bits from run to run (one writer per column, slices added in a fixed order)."""
	buf = _randn(T, ld, seed=91)
	x = buf[:, :N]
	start = torch.randn(N, device="cuda", generator=torch.Generator(device="cuda").manual_seed(92))
	runs = []
	for _ in range(3):
		acc = start.clone()
		K.colsum_(x, acc)
		runs.append(acc)
	assert torch.equal(runs[0], runs[1]) and torch.equal(runs[0], runs[2])
	want = start.double() + x.double().sum(0)
	assert ((runs[0].double() - want).abs().max() / want.abs().max()).item() <= 1e-5


def test_split_k_on_one_stream_never_gives_up_its_turn_and_wide_splits_are_refused(K):
	"""Back-to-back split-K launches on one stream keep their turns (the counter of waves that added out of turn does not
	move, which is what bit-reproducible weight gradients rest on), and a split count that would not fit the 8 bits the
	turn counters give it is refused."""
	from elf_amd import _lib

	M, N, Kd = 768, 768, 8192
	A, B = _randn(Kd, M, seed=130), _randn(Kd, N, seed=131, scale=0.05)
	before = K.gemm_turn_giveups()
	runs = []
	for _ in range(3):
		acc = torch.zeros(M, N, device="cuda")
		for cfg in (7, 8, 1):
			K.gemm(A, B, a_t=True, b_t=True, out=acc, epilogue=K.EPI_F32_ACC, k_splits=4, tile_cfg=cfg)
		runs.append(acc)
	torch.cuda.synchronize()
	assert K.gemm_turn_giveups() == before
	assert torch.equal(runs[0], runs[1]) and torch.equal(runs[0], runs[2])
	with pytest.raises(_lib.ElfStageError):
		K.gemm(A, B, a_t=True, b_t=True, out=runs[0], epilogue=K.EPI_F32_ACC, k_splits=256, tile_cfg=7)


def _dw_problems(shapes, Kd, seed):
	"""(dy [Kd, M], x [Kd, N], acc [M, N] with what earlier micro-batches left in it) per (M, N)."""
	out = []
	for i, (M, N) in enumerate(shapes):
		g = torch.Generator(device="cuda").manual_seed(seed + i)
		out.append((_randn(Kd, M, seed=seed + 10 * i), _randn(Kd, N, seed=seed + 10 * i + 1, scale=0.05), torch.randn(M, N, generator=g, device="cuda")))
	return out


def test_grouped_weight_gradients_equal_the_single_launches(K):
	"""Several layers' dW += dY^T X in one launch (the W pass of a stage) against one elf_gemm_bf16 call per layer that
	splits K the same way: whole tiles (K too short to split); the GPT-2-small layers at K = 4096, whose 108 tiles are all
	in the launch's only round and split two ways; and a large layer (256 whole tiles, one round) followed by two small
	ones whose 36 tiles make up the last round and are split four ways.  Bit for bit, run after run, no turn given up; and
	against fp32 torch."""
	before = K.gemm_turn_giveups()
	for shapes, Kd, splits in (
		(((256, 512), (768, 256), (512, 768), (256, 256)), 512, (1, 1, 1, 1)),
		(((768, 3072), (3072, 768), (768, 768), (2304, 768)), 4096, (2, 2, 2, 2)),
		(((4096, 4096), (768, 768), (768, 2304)), 4096, (1, 4, 4)),
	):
		print(f"[case] gemm_dw_group {shapes} K={Kd}", flush=True)
		problems = _dw_problems(shapes, Kd, seed=400)
		start = [acc.clone() for _, _, acc in problems]
		want = []
		for (dy, x, _), acc0, ks in zip(problems, start, splits):
			acc = acc0.clone()
			K.gemm(dy, x, a_t=True, b_t=True, out=acc, epilogue=K.EPI_F32_ACC, tile_cfg=7, k_splits=ks)
			want.append(acc)
		runs = []
		for _ in range(3):
			accs = [a.clone() for a in start]
			K.gemm_dw_group([(dy, x, acc) for (dy, x, _), acc in zip(problems, accs)])
			runs.append(accs)
		torch.cuda.synchronize()
		for i, (dy, x, _) in enumerate(problems):
			assert torch.equal(runs[0][i], want[i]), f"layer {i} {shapes[i]}: grouped launch differs from the single one"
			assert torch.equal(runs[1][i], want[i]) and torch.equal(runs[2][i], want[i]), f"layer {i}: not reproducible"
			ref = start[i].double() + dy.double().t() @ x.double()
			assert ((want[i].double() - ref).abs().max() / ref.abs().max()).item() <= 1e-5
	assert K.gemm_turn_giveups() == before


@pytest.mark.parametrize("shapes", [((2048, 2048), (2048, 2048), (2048, 2048), (3072, 3072)), ((4608, 4608),), ((768, 768),)], ids=["small_layers", "one_large_layer", "one_small_layer"])
def test_grouped_weight_gradients_with_the_split_boundary_inside_a_layer(K, shapes):
	"""The launch's last round may begin in the middle of a layer: 3 x 64 + 144 tiles (80 of the last layer's tiles split
	three ways; small layers, laid on the XCDs as contiguous runs), one layer of 324 tiles (68 split three ways; its own
	tile walk), and a lone 9-tile layer (all split).  Against fp64 torch, twice with equal bits, with the scale folded in."""
	Kd = 4096
	problems = _dw_problems(shapes, Kd, seed=700)
	before = K.gemm_turn_giveups()
	runs = []
	for _ in range(2):
		accs = [acc.clone() for _, _, acc in problems]
		g16 = [torch.empty_like(a, dtype=torch.bfloat16) for a in accs]
		K.gemm_dw_group([(dy, x, acc, h) for (dy, x, _), acc, h in zip(problems, accs, g16)], scale=0.25)
		runs.append((accs, g16))
	torch.cuda.synchronize()
	assert K.gemm_turn_giveups() == before
	for i, (dy, x, start) in enumerate(problems):
		ref = (start.double() + dy.double().t() @ x.double()) * 0.25
		got = runs[0][0][i]
		assert ((got.double() - ref).abs().max() / ref.abs().max()).item() <= 1e-5, f"layer {i} {shapes[i]}"
		assert torch.equal(runs[0][1][i], got.to(torch.bfloat16)), f"layer {i}: bf16 copy"
		assert torch.equal(runs[1][0][i], got) and torch.equal(runs[1][1][i], runs[0][1][i]), f"layer {i}: not reproducible"


def test_grouped_weight_gradients_with_the_gradient_scale(K):
	"""scale != 0: the accumulators leave multiplied by the scale with their bf16 copies written, from the epilogue for
	whole tiles and by a small kernel behind the launch for split ones (here: none split, all split, and a whole layer
	followed by a split one): all equal the unscaled launch followed by elf_scale_grads bit for bit."""
	for shapes, Kd in ((((256, 512), (768, 256)), 512), (((768, 3072), (768, 768)), 8192), (((4096, 4096), (768, 768)), 4096)):
		problems = _dw_problems(shapes, Kd, seed=500)
		plain = [acc.clone() for _, _, acc in problems]
		K.gemm_dw_group([(dy, x, acc) for (dy, x, _), acc in zip(problems, plain)])
		plain16 = [torch.empty_like(a, dtype=torch.bfloat16) for a in plain]
		for a, h in zip(plain, plain16):
			K.scale_grads_(a, h, 1 / 32)
		folded = [acc.clone() for _, _, acc in problems]
		folded16 = [torch.full_like(a, 7.0, dtype=torch.bfloat16) for a in folded]
		K.gemm_dw_group([(dy, x, acc, h) for (dy, x, _), acc, h in zip(problems, folded, folded16)], scale=1 / 32)
		torch.cuda.synchronize()
		for i in range(len(problems)):
			assert torch.equal(folded[i], plain[i]) and torch.equal(folded16[i], plain16[i]), f"layer {i} {shapes[i]} K={Kd}"


def test_grouped_weight_gradients_refuse_what_the_tiles_cannot_hold(K):
	from elf_amd import _lib

	ok = _dw_problems(((256, 256),), 512, seed=600)
	with pytest.raises(_lib.ElfStageError):
		K.gemm_dw_group(ok * 17)
	with pytest.raises(_lib.ElfStageError):
		K.gemm_dw_group(_dw_problems(((256, 320),), 512, seed=601))
	with pytest.raises(_lib.ElfStageError):
		K.gemm_dw_group(ok, scale=0.5)  # a scaling pass needs somewhere to put the bf16 gradients


def test_split_k_gemms_on_two_streams_stay_correct(K):
	"""Weight-gradient GEMMs launched concurrently on two streams share the turn counters of their split tiles; whatever
	the interleaving, every sum must be the right one to fp32 rounding (a workgroup that finds its counter taken by
	the other launch adds out of turn)."""
	M, N, Kd = 768, 768, 8192
	A = [_randn(Kd, M, seed=110 + i) for i in range(2)]
	B = [_randn(Kd, N, seed=120 + i, scale=0.05) for i in range(2)]
	ref = [A[i].float().t() @ B[i].float() for i in range(2)]
	acc = [torch.zeros(M, N, device="cuda") for _ in range(2)]
	streams = [torch.cuda.Stream(), torch.cuda.Stream()]
	torch.cuda.synchronize()
	reps = 12
	for _ in range(reps):
		for i in range(2):
			with torch.cuda.stream(streams[i]):
				K.gemm(A[i], B[i], a_t=True, b_t=True, out=acc[i], epilogue=K.EPI_F32_ACC, k_splits=4, tile_cfg=7 if i == 0 else 8)
	torch.cuda.synchronize()
	for i in range(2):
		assert ((acc[i] - reps * ref[i]).norm() / (reps * ref[i]).norm()).item() <= 1e-5
