"""Properties that do not depend on size, checked at the benchmark's full shapes (Llama-3-8B-shaped
stage: 8192 tokens per micro-batch, d_model 4096, 32 query / 8 kv heads of 128, FFN 14336; and the
Llama-3-70B-shaped one: d_model 8192, 64 query / 8 kv heads, FFN 28672, one sequence of 8192).  Each
property is one a wrong tile index, a dropped K slice, a mis-masked attention tile or a lost
accumulation would break.  Whole stages at these shapes against the oracle are in
tests/test_benchmark_shapes_gpu.py."""

import pytest
import torch

pytestmark = pytest.mark.gpu

T, D_MODEL, HQ, HKV, HD, FFN, SEQ = 8192, 4096, 32, 8, 128, 14336, 4096


def _randn(*shape, seed=0, scale=1.0):
	g = torch.Generator(device="cuda").manual_seed(seed)
	return (torch.randn(*shape, generator=g, device="cuda") * scale).to(torch.bfloat16)


@pytest.fixture(scope="module")
def K():
	from elf_amd import kernels

	return kernels


# the Llama-3-8B FFN shapes (256x256 tiles; for tn the dW shape whose 896 tiles get a K-split tail), the
# down projection's (an A operand of 235 MB: the tile walk in bands of 16 tile rows; for tn the 14336 x 4096
# weight gradient, whose split tail is the walk's partly filled last round) and the GPT-2-small ones
# (N = 768: 128x256 tiles; dW with 36 tiles: K split over all of them)
# and the Llama-3-70B FFN shapes (N = 57344: 7168 tiles, a 940 MB weight; K = 28672; for tn a 1.9 GB fp32 result)
@pytest.mark.parametrize("dims", [(T, FFN, D_MODEL), (T, D_MODEL, FFN), (T, 768, 3072), (T, 57344, 8192), (T, 8192, 28672)])
@pytest.mark.parametrize("layout", ["nt", "nn", "tn"])
def test_gemm_row_and_column_probes_at_full_size(K, layout, dims):
	"""C = A B^T (for tn the matching dW shape, K = tokens): 64 sampled rows and columns of the result
	equal their fp32 dot products; a one-hot A row selects a B column exactly."""
	M, N, Kd = dims if layout != "tn" else (dims[2], dims[1], dims[0])
	A = _randn(M, Kd, seed=1)
	B = _randn(N, Kd, seed=2, scale=0.05)
	A[7].zero_()
	A[7, 1234] = 1.0  # row 7 of C must be column 1234 of B, bit for bit
	if layout == "nt":
		C = K.gemm(A, B)
	elif layout == "nn":
		C = K.gemm(A, B.t().contiguous(), b_t=True)
	else:
		C = torch.zeros(M, N, dtype=torch.float32, device="cuda")
		K.gemm(A.t().contiguous(), B.t().contiguous(), a_t=True, b_t=True, out=C, epilogue=K.EPI_F32_ACC)
	assert torch.equal(C[7].to(torch.bfloat16), B[:, 1234])
	rows = torch.randint(0, M, (64,), generator=torch.Generator().manual_seed(3)).cuda()
	cols = torch.randint(0, N, (64,), generator=torch.Generator().manual_seed(4)).cuda()
	ref_r = A[rows].float() @ B.float().t()
	ref_c = A.float() @ B[cols].float().t()
	for got, ref in ((C[rows].float(), ref_r), (C[:, cols].float(), ref_c)):
		assert (got - ref).abs().max().item() <= 2e-2 * ref.abs().max().item()
		assert ((got - ref).norm() / ref.norm()).item() <= 5e-3


@pytest.mark.parametrize("dims", [(6144, 3072, 14336), (10240, 2048, 8192), (8192, 3072, 14336)])
def test_gemm_band_walk_with_a_partly_filled_last_round(K, dims):
	"""A operands of 160 MB and more take the tile walk in bands of 16 tile rows; 288, 320 and 384 tiles
	leave 1, 2 and 4 blocks of 8 x 4 tiles for the last round, which the 8 XCDs then share.  Every
	element against an fp32 product of the same bf16 operands."""
	M, N, Kd = dims
	A = _randn(M, Kd, seed=11)
	B = _randn(N, Kd, seed=12, scale=0.05)
	ref = A.float() @ B.float().t()
	for C in (K.gemm(A, B), K.gemm(A, B.t().contiguous(), b_t=True)):
		err = (C.float() - ref).abs()
		assert err.max().item() <= 2e-2 * ref.abs().max().item()
		assert (err.norm() / ref.norm()).item() <= 5e-3


def test_gemm_fp32_accumulation_is_additive_at_full_size(K):
	"""The deferred weight-gradient epilogue: three calls into one fp32 buffer = 3 x one call,
	and the K-split variant (fp32 atomics) agrees with the unsplit one."""
	dY = _randn(T, D_MODEL, seed=5, scale=0.1)
	X = _randn(T, FFN, seed=6)
	one = torch.zeros(D_MODEL, FFN, dtype=torch.float32, device="cuda")
	K.gemm(dY, X, a_t=True, b_t=True, out=one, epilogue=K.EPI_F32_ACC, k_splits=1)
	acc = torch.zeros_like(one)
	for _ in range(3):
		K.gemm(dY, X, a_t=True, b_t=True, out=acc, epilogue=K.EPI_F32_ACC, k_splits=1)
	assert ((acc - 3 * one).abs().max() <= 1e-5 * one.abs().max()).item()
	split = torch.zeros_like(one)
	K.gemm(dY, X, a_t=True, b_t=True, out=split, epilogue=K.EPI_F32_ACC, k_splits=4)
	assert ((split - one).norm() / one.norm()).item() <= 1e-5


@pytest.mark.parametrize("shape", [(2, 4096, 32, 8), (1, 8192, 32, 8), (1, 8192, 64, 8)])
def test_attention_properties_at_full_size(K, shape):
	"""Causal GQA attention at batch 2 x seq 4096 (Llama-3-8B-shaped stage), 1 x 8192 (its long-sequence
	variant) and 1 x 8192 with 64 query heads (70B-shaped): (1) with V = 1 every output is 1 (rows of P sum
	to one); (2) changing keys / values / queries after position p leaves outputs up to p unchanged
	bit for bit; (3) dQ, dK, dV are linear in dO; (4) with dO = 0 all gradients vanish."""
	B, SEQ, HQ, HKV = shape
	print(f"[case] attention properties B={B} S={SEQ} Hq={HQ} Hkv={HKV}", flush=True)
	nq, nkv = HQ * HD, HKV * HD
	qkv = _randn(B * SEQ, nq + 2 * nkv, seed=7, scale=0.5)
	ones = qkv.clone()
	ones[:, nq + nkv:] = 1.0
	o, _ = K.attn_fwd(ones, B, SEQ, HQ, HKV, HD, True)
	assert (o.float() - 1.0).abs().max().item() <= 1e-2
	o_ref, lse = K.attn_fwd(qkv, B, SEQ, HQ, HKV, HD, True)
	p = 2500
	pert = qkv.clone()
	pert.view(B, SEQ, -1)[:, p + 1:] = _randn(B, SEQ - p - 1, nq + 2 * nkv, seed=8)
	o_pert, lse_pert = K.attn_fwd(pert, B, SEQ, HQ, HKV, HD, True)
	assert torch.equal(o_pert.view(B, SEQ, -1)[:, :p + 1], o_ref.view(B, SEQ, -1)[:, :p + 1])
	assert torch.equal(lse_pert[:, :, :p + 1], lse[:, :, :p + 1])
	do1 = _randn(B * SEQ, nq, seed=9)
	do2 = _randn(B * SEQ, nq, seed=10)
	g1 = K.attn_bwd(qkv, o_ref, do1, lse, B, SEQ, HQ, HKV, HD, True).float()
	g2 = K.attn_bwd(qkv, o_ref, do2, lse, B, SEQ, HQ, HKV, HD, True).float()
	g12 = K.attn_bwd(qkv, o_ref, (do1.float() + do2.float()).to(torch.bfloat16), lse, B, SEQ, HQ, HKV, HD, True).float()
	for name, sl in (("dq", slice(0, nq)), ("dk", slice(nq, nq + nkv)), ("dv", slice(nq + nkv, None))):
		want = g1[:, sl] + g2[:, sl]
		assert ((g12[:, sl] - want).norm() / want.norm()).item() <= 1.5e-2, name
	g0 = K.attn_bwd(qkv, o_ref, torch.zeros_like(do1), lse, B, SEQ, HQ, HKV, HD, True)
	assert g0.abs().max().item() == 0.0
	# causality of the backward: a gradient that arrives only at positions <= p gives no dK / dV after p
	do_head = do1.clone()
	do_head.view(B, SEQ, -1)[:, p + 1:] = 0
	gh = K.attn_bwd(qkv, o_ref, do_head, lse, B, SEQ, HQ, HKV, HD, True).view(B, SEQ, -1)
	assert gh[:, p + 1:].abs().max().item() == 0.0


@pytest.mark.parametrize("SEQ,Hq", [(4096, 4), (8192, 4), (8192, 8)])
def test_attention_one_kv_group_at_full_sequence_length(K, SEQ, Hq):
	"""One grouped-query group (4 or 8 query heads on 1 kv head) at the full sequence length, against fp32
	torch: 32 or 64 key tiles per query row, so the backward sums the deepest stack of per-tile dQ
	partials the benchmark shapes have.  Tolerances of the small-shape kernel tests."""
	import math

	print(f"[case] attention one kv group S={SEQ} Hq={Hq}", flush=True)
	B, Hkv = 1, 1
	qkv = _randn(B * SEQ, (Hq + 2 * Hkv) * HD, seed=11)
	do = _randn(B * SEQ, Hq * HD, seed=12)
	x = qkv.float().requires_grad_(True)
	q = x[:, : Hq * HD].reshape(SEQ, Hq, HD).transpose(0, 1)
	k = x[:, Hq * HD : (Hq + 1) * HD].reshape(SEQ, 1, HD).transpose(0, 1)
	v = x[:, (Hq + 1) * HD :].reshape(SEQ, 1, HD).transpose(0, 1)
	s = (q @ k.transpose(-1, -2)) / math.sqrt(HD)
	s = s.masked_fill(~torch.ones(SEQ, SEQ, dtype=torch.bool, device="cuda").tril(), float("-inf"))
	o_ref = (torch.softmax(s, dim=-1) @ v).transpose(0, 1).reshape(SEQ, Hq * HD)
	o_ref.backward(do.float())
	o, lse = K.attn_fwd(qkv, B, SEQ, Hq, Hkv, HD, True)
	g = K.attn_bwd(qkv, o, do, lse, B, SEQ, Hq, Hkv, HD, True).float()

	def close(got, ref, what):
		scale = ref.abs().max().item()
		assert (got - ref).abs().max().item() <= 2e-2 * scale, what
		assert ((got - ref).norm() / ref.norm()).item() <= 1.5e-2, what

	close(o.float(), o_ref.detach(), "o")
	close(g[:, : Hq * HD], x.grad[:, : Hq * HD], "dq")
	close(g[:, Hq * HD : (Hq + 1) * HD], x.grad[:, Hq * HD : (Hq + 1) * HD], "dk")
	close(g[:, (Hq + 1) * HD :], x.grad[:, (Hq + 1) * HD :], "dv")


def test_bandwidth_kernels_at_full_size(K):
	"""RMSNorm output has unit RMS under gamma = 1; SwiGLU of (g, u) with u = 1 is silu(g); RoPE
	keeps the norm of every (x_i, x_{i+D/2}) pair and its backward undoes its forward; the gradient
	scale is exact in fp32."""
	x = _randn(T, D_MODEL, seed=11) * 3.0
	x = x.to(torch.bfloat16)
	y, stats = K.norm_fwd(K.NORM_RMS, x, torch.ones(D_MODEL, dtype=torch.bfloat16, device="cuda"), None, 1e-5)
	rms = y.float().pow(2).mean(-1).sqrt()
	assert (rms - 1).abs().max().item() <= 5e-3
	gu = _randn(T, 2 * FFN, seed=12)
	gu[:, FFN:] = 1.0
	h = K.swiglu_fwd(gu)
	assert (h.float() - torch.nn.functional.silu(gu[:, :FFN].float())).abs().max().item() <= 2e-2
	qkv = _randn(2 * SEQ, (HQ + 2 * HKV) * HD, seed=13)
	before = qkv.clone()
	cs = K.rope_table(SEQ, HD, 5e5)
	K.rope_apply_(qkv, cs, SEQ, HQ + HKV, HD)
	v0 = before[:, : (HQ + HKV) * HD].float().view(2 * SEQ, HQ + HKV, 2, HD // 2)
	v1 = qkv[:, : (HQ + HKV) * HD].float().view(2 * SEQ, HQ + HKV, 2, HD // 2)
	n0, n1 = v0.pow(2).sum(2), v1.pow(2).sum(2)
	assert ((n1 - n0).abs() <= 2e-2 * n0 + 1e-3).all().item()
	assert torch.equal(qkv[:, (HQ + HKV) * HD:], before[:, (HQ + HKV) * HD:])  # V untouched
	K.rope_apply_(qkv, cs, SEQ, HQ + HKV, HD, backward=True)
	assert (qkv.float() - before.float()).abs().max().item() <= 3e-2 * before.float().abs().max().item()
	acc = torch.randn(D_MODEL, FFN, device="cuda", generator=torch.Generator(device="cuda").manual_seed(14))
	want = acc / 32
	out = torch.empty(D_MODEL, FFN, dtype=torch.bfloat16, device="cuda")
	K.scale_grads_(acc, out, 1.0 / 32)
	assert torch.equal(acc, want) and torch.equal(out, want.to(torch.bfloat16))


def test_cross_entropy_at_the_llama_vocabulary(K):
	"""One micro-batch of logits at the Llama-3 vocabulary (8192 x 128256): rows whose logits are zero
	except b at the target have the closed-form loss log(1 + (V-1) e^-b); every gradient row sums to
	zero (softmax - onehot) within bf16 rounding; a sample of random rows matches the CPU oracle."""
	import math

	from elf_amd import losses
	from oracle import loss_ref as L

	V, b = 128256, 5.0
	g = torch.Generator(device="cuda").manual_seed(21)
	x = (torch.randn(T, V, device="cuda", generator=g) * 2.0).to(torch.bfloat16)
	t = torch.randint(0, V, (T,), device="cuda", generator=g)
	x[:256] = 0
	x[torch.arange(256, device="cuda"), t[:256]] = b
	loss, grad = losses.cross_entropy.loss_and_grad(x, t, reduction="sum", scale=1.0)
	rows = losses.cross_entropy(x, t, reduction="none")
	assert float(loss) == pytest.approx(float(rows.double().sum()), rel=1e-5)
	assert torch.allclose(rows[:256], torch.full((256,), math.log1p((V - 1) * math.exp(-b)), device="cuda"), rtol=1e-5)
	row_sums = grad.float().sum(-1)
	assert row_sums.abs().max().item() <= 2e-2  # |sum| of V values each rounded to bf16
	pick = torch.arange(256, T, 131, device="cuda")
	xs, ts = x[pick].cpu(), t[pick].cpu()
	assert torch.allclose(rows[pick].cpu(), L.cross_entropy_ref(xs, ts, "none"), rtol=1e-5, atol=2e-5)
	xf = xs.float().requires_grad_()
	L.cross_entropy_ref(xf, ts, "sum").backward()
	err = (grad[pick].float().cpu() - xf.grad).abs()
	assert bool((err <= xf.grad.abs() * 2.0**-7 + 1e-6).all())
