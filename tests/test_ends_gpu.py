"""First / last stage of a decoder on the native executor: token embedding in front of the blocks,
(final norm,) output head behind them (reference modules: FullTransformer.embed / .head,
benchmarks/models/simple.py:470-524), against the oracle stage; and the reference's own small
configuration (4-layer GPT-style decoder, d 256, 4 heads, FFN 1024, seq 128, vocabulary 1000,
micro-batch 4 x 8, cross-entropy) run through ``Pipeline`` as two stages on one rank against plain
fp32 autograd over the same weights.  Tolerances: the stage bar (rel 2e-2 of max, 1e-2 Frobenius)."""

import pytest
import torch
import torch.nn.functional as F

from tests.helpers import assert_close, cfg_from_stage, oracle_params_from_stage, perturb_norms, product_grads

pytestmark = pytest.mark.gpu


def test_embedding_kernels_match_torch():
	from elf_amd import kernels as K

	V, d, T = 1000, 256, 4096
	g = torch.Generator().manual_seed(1)
	table = (torch.randn(V, d, generator=g) * 0.5).to(torch.bfloat16).cuda()
	ids = torch.randint(0, V, (T,), generator=g).cuda()
	ids[:64] = 7  # a token that repeats: its gradient rows must add up
	out = K.embedding_fwd(ids, table)
	assert torch.equal(out, table[ids])
	bad = ids.clone()
	bad[3], bad[5] = -1, V
	out_bad = K.embedding_fwd(bad, table)
	assert out_bad[3].abs().max().item() == 0 and out_bad[5].abs().max().item() == 0 and torch.equal(out_bad[6:], out[6:])
	dx = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
	dtab = torch.full((V, d), 0.25, dtype=torch.float32, device="cuda")
	K.embedding_bwd_(ids, dx, dtab)
	want = torch.full((V, d), 0.25, dtype=torch.float32, device="cuda").index_add_(0, ids, dx.float())
	assert_close(dtab, want, "embedding dtable", rel_max=1e-5, rel_fro=1e-5)
	again = torch.full((V, d), 0.25, dtype=torch.float32, device="cuda")
	K.embedding_bwd_(ids, dx, again)
	assert torch.equal(again, dtab), "a table row has one writer that adds its tokens in order: equal bits from run to run"
	K.embedding_bwd_(bad, dx, dtab.zero_())
	assert dtab.abs().sum().item() > 0  # out-of-range ids are skipped, the rest still lands


@pytest.mark.parametrize("V,d,T", [(50, 4096, 1000), (3, 8192, 777), (128256, 1024, 8192)])
def test_embedding_backward_ragged_sizes_and_heavy_repeats(V, d, T):
	"""Token counts that are not multiples of the workgroup size, rows wider than one pass of the workgroup, a
	vocabulary so small that every row collects hundreds of tokens: the sum in the kernel's fixed order, exactly."""
	from elf_amd import kernels as K

	g = torch.Generator().manual_seed(V + d)
	ids = torch.randint(0, V, (T,), generator=g).cuda()
	dx = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
	start = torch.randn(V, d, generator=g).cuda()
	got = start.clone()
	K.embedding_bwd_(ids, dx, got)
	# the kernel's order of additions, row by row: the positions behind a token's first occurrence in runs of 64, run k to
	# partial sum k % 4, each partial in ascending position, the partials folded left to right, then the row's old value
	touched = torch.unique(ids)
	want = start.clone()
	for tok in touched[:64].tolist():
		pos = (ids == tok).nonzero().flatten().tolist()
		parts = [torch.zeros(d, device="cuda") for _ in range(4)]
		for t in pos:
			parts[((t - pos[0]) // 64) % 4] += dx[t].float()
		want[tok] += ((parts[0] + parts[1]) + parts[2]) + parts[3]
		assert torch.equal(got[tok], want[tok]), f"row {tok}"
	full = start.clone().index_add_(0, ids, dx.float())
	assert_close(got, full, "embedding dtable", rel_max=1e-5, rel_fro=1e-5)
	untouched = torch.ones(V, dtype=torch.bool, device="cuda")
	untouched[touched] = False
	assert torch.equal(got[untouched], start[untouched])


@pytest.mark.parametrize("dist", ["all_equal", "zipf"])
def test_embedding_backward_with_padding_like_and_zipf_ids(dist):
	"""8192 tokens of width 4096 (the benchmark's token count) where one id fills the batch (padding) or ids follow a Zipf
	law (natural text): the row of a frequent id is summed by four waves per 512-column slice in a fixed order - exact
	against fp32 sums in that order - and the call stays in the time of a few passes over dx."""
	from elf_amd import kernels as K

	V, d, T = 32000, 4096, 8192
	g = torch.Generator().manual_seed(11)
	if dist == "all_equal":
		ids = torch.full((T,), 17, dtype=torch.int64)
	else:
		p = 1.0 / torch.arange(1, V + 1, dtype=torch.float64)
		ids = torch.multinomial(p / p.sum(), T, replacement=True, generator=g)
	ids = ids.cuda()
	dx = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
	got = torch.zeros(V, d, device="cuda")
	K.embedding_bwd_(ids, dx, got)
	torch.cuda.synchronize()
	top = int(torch.mode(ids).values.item())
	pos = (ids == top).nonzero().flatten()
	run = ((pos - pos[0]) // 64) % 4
	parts = []
	for w in range(4):  # fp32 adds in the kernel's order: four interleaved runs of positions, each ascending, folded left to right
		acc = torch.zeros(d, device="cuda")
		for r in dx[pos[run == w]].float().split(1):
			acc += r[0]
		parts.append(acc)
	want = ((parts[0] + parts[1]) + parts[2]) + parts[3]
	assert torch.equal(got[top], want), f"row of the most frequent id ({pos.numel()} occurrences)"
	full = torch.zeros(V, d, device="cuda").index_add_(0, ids, dx.float())
	assert_close(got, full, f"embedding dtable ({dist})", rel_max=1e-5, rel_fro=1e-5)
	e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
	e0.record()
	for _ in range(5):
		K.embedding_bwd_(ids, dx, got)
	e1.record()
	torch.cuda.synchronize()
	us = e0.elapsed_time(e1) / 5 * 1e3
	print(f"[embedding_bwd {dist}] {us:.0f} us per call, {T * d * 2 / us / 1e3:.0f} GB/s of dx", flush=True)
	assert us < 2000, f"embedding_bwd took {us:.0f} us on {dist} ids"


def _end_stage(kind, vocab_in, vocab_out, final_norm, seed):
	from elf_amd import models

	if kind == "gpt":
		st = models.gpt_end_stage(1, 256, 4, 512, 128, vocab_in=vocab_in, vocab_out=vocab_out, causal=True, final_norm=final_norm, seed=seed)
	else:
		blocks = models.StageModule([models.LlamaBlock(256, 2, 1, 512, 128, True, 5e5)], 128)
		st = models._init(models.EndStage(blocks, vocab_in, vocab_out, final_norm), seed, torch.bfloat16)
	perturb_norms(st.blocks)
	if st.norm_f is not None:
		with torch.no_grad():
			st.norm_f.weight.add_(0.1 * torch.randn(st.norm_f.weight.shape).to(torch.bfloat16))
	return st


def _ends_params(st):
	out = {}
	if st.embed is not None:
		out["embed"] = st.embed.weight.detach().clone()
	if st.head is not None:
		out["head"] = st.head.weight.detach().clone()
	if st.norm_f is not None:
		out["normf_g"] = st.norm_f.weight.detach().clone()
		if getattr(st.norm_f, "bias", None) is not None:
			out["normf_b"] = st.norm_f.bias.detach().clone()
	return out


def _ends_grads(st):
	out = {}
	for name, mod in (("embed", st.embed), ("head", st.head), ("normf_g", st.norm_f)):
		if mod is not None:
			out[f"ends.{name}"] = mod.weight.main_grad
	if st.norm_f is not None and getattr(st.norm_f, "bias", None) is not None:
		out["ends.normf_b"] = st.norm_f.bias.main_grad
	return out


@pytest.mark.parametrize("case", [("gpt", 1000, None, False), ("gpt", None, 1000, False), ("gpt", None, 1024, True), ("llama", 512, 320, True)])
@pytest.mark.parametrize("variant", ["plain", "full_fwd", "full_bwd"])
def test_first_and_last_stage_match_oracle(case, variant):
	"""F, B, W (and the remat variants) of a stage with an embedding and / or a head, driven
	directly through the block's ops with hand-fed boundaries."""
	from elf_amd.execution import HipStageBlock
	from elf_amd.partitioners.utils import sequential_signatures
	from elf_amd.scheduling import OpOptions
	from oracle import stage_ref as R

	kind, vin, vout, fnorm = case
	mb, nmb, S, d = 2, 2, 128, 256
	st = _end_stage(kind, vin, vout, fnorm, seed=31)
	cfg = cfg_from_stage(st.blocks, mb)
	ref = R.RefStage(cfg, oracle_params_from_stage(st.blocks), device="cuda", ends=_ends_params(st))
	placement = [0, 1, 2]
	blk = HipStageBlock(st, 1, placement, sequential_signatures(placement)[1], mb_size=mb)
	blk.zero_grad()
	g = torch.Generator().manual_seed(5)
	xs = [torch.randint(0, vin, (mb, S), generator=g).cuda() if vin else torch.randn(mb, S, d, generator=g).to(torch.bfloat16).cuda() for _ in range(nmb)]
	dys = [(torch.randn(mb, S, vout or d, generator=g) * (0.1 if vout else 1.0)).to(torch.bfloat16).cuda() for _ in range(nmb)]
	blk.set_boundary(inputs=xs, grads=dys, keep_sent=True)
	root = (lambda name, module: name == "") if variant == "full_fwd" else None
	for m in range(nmb):
		blk.recv_forward(m, mb, src=0)
		blk.forward(m, **({OpOptions.REMAT_STRATEGY: root} if root else {}))
		blk.send_forward(m, dst=2)
		y = blk.sent_forward[m]
		assert tuple(y.shape) == (mb, S, vout or d)
		assert_close(y, ref.forward(m, xs[m], remat_root=root is not None), f"{case} y[{m}]")
	for m in range(nmb):
		blk.recv_backward(m, mb, src=2)
		full_bwd = variant == "full_bwd"
		blk.backward_inputs(m, **({OpOptions.RECOMPUTE_ACTIVATIONS: True, OpOptions.RECOMPUTE_GRADIENTS: True} if full_bwd else {}))
		blk.send_backward(m, dst=0)
		want_dx = ref.backward_inputs(m, dys[m], recompute_activations=full_bwd, recompute_gradients=full_bwd)
		if vin:
			assert want_dx is None and m not in blk.sent_backward
		else:
			assert_close(blk.sent_backward[m], want_dx, f"{case} dx[{m}]")
		if full_bwd:
			blk.recompute_forward(m, **{OpOptions.SAVE: True})
			blk.recompute_backward_inputs(m)
			ref.recompute_forward(m, save=True)
			ref.recompute_backward_inputs(m)
		blk.backward_params(m)
		ref.backward_params(m)
	torch.cuda.synchronize()
	got = dict(product_grads(st.blocks), **_ends_grads(st))
	want = ref.grads()
	assert set(want) <= set(got)
	for name in sorted(want):
		assert_close(got[name], want[name], f"{case} {variant} grad {name}")
	if vout and blk.vld != vout:  # the padding rows of the head never receive a gradient
		assert blk._fused_g[blk._param_loc[st.head.weight][0]][vout:].abs().max().item() == 0
	assert blk.mem_stats()["live_bytes"] == 0


@pytest.mark.parametrize("loss_kind", ["torch", "fused"])
@pytest.mark.parametrize("scheduler,placement", [("afab", [0, 0]), ("1f1b", [0, 1]), ("zbh1", [0, 1])])
def test_reference_small_configuration_through_pipeline(loss_kind, scheduler, placement):
	"""4-layer GPT-style decoder, d 256, 4 heads, FFN 1024 GELU, LayerNorm, seq 128, vocabulary 1000,
	micro-batch 4 x 8 micro-batches, cross-entropy on fp32 logits flattened over the sequence
	(FullTransformer.loss_fn, benchmarks/models/simple.py:519-523), as two stages: on one rank under
	AFAB, and as the two ranks of a pp = 2 pipeline under 1F1B and ZB-H1 (the reference's small
	configuration: its op streams for both ranks, comm ops included, interpreted by one process);
	once with that torch loss under autograd and once with the library's one-kernel cross-entropy.
	Loss and every gradient against the un-pipelined model in fp32."""
	from elf_amd import models
	from elf_amd.pipeline import Pipeline

	V, d, S, mb, nmb = 1000, 256, 128, 4, 8
	first = models.gpt_end_stage(2, d, 4, 1024, S, vocab_in=V, causal=True, seed=41)
	last = models.gpt_end_stage(2, d, 4, 1024, S, vocab_out=V, causal=True, seed=42)
	for st in (first, last):
		perturb_norms(st.blocks)

	def loss_fn(pred, target, *args, **kwargs):
		return F.cross_entropy(pred.to(torch.float32).view(-1, V), target.view(-1), *args, **kwargs)

	if loss_kind == "fused":
		from elf_amd.losses import cross_entropy as loss_fn

	# plain autograd in fp32 over the same (bf16-rounded) weights, whole batch at once
	import copy

	ref_first, ref_last = copy.deepcopy(first).float().cuda(), copy.deepcopy(last).float().cuda()
	g = torch.Generator().manual_seed(9)
	ids = torch.randint(0, V, (mb * nmb, S), generator=g).cuda()
	tgt = torch.randint(0, V, (mb * nmb, S), generator=g).cuda()
	logits = ref_last(ref_first(ids))
	want_loss = F.cross_entropy(logits.view(-1, V), tgt.view(-1), reduction="sum") / (S * mb * nmb)
	want_loss.backward()
	# the same model in the reference's own arithmetic (bf16 modules under PyTorch autograd): how far bf16 itself is from
	# the fp32 truth per parameter gradient.  Every gradient meets rel 2e-2 of its largest magnitude; the relative
	# Frobenius bound is 1e-2 or 1.25 x PyTorch's bf16 error, whichever is larger (the query / key projections of the
	# deeper blocks sit at 1.1-1.2 % in PyTorch's bf16 as well: four blocks of roundings in front of a softmax).
	bf_first, bf_last = copy.deepcopy(first).cuda(), copy.deepcopy(last).cuda()
	(F.cross_entropy(bf_last(bf_first(ids)).float().view(-1, V), tgt.view(-1), reduction="sum") / (S * mb * nmb)).backward()
	fro_bound = {}
	for tag, bf_mod, ref_mod in (("first", bf_first, ref_first), ("last", bf_last, ref_last)):
		ref_params = dict(ref_mod.named_parameters())
		for name, p in bf_mod.named_parameters():
			r = ref_params[name].grad.double()
			fro_bound[tag, name] = max(1e-2, 1.25 * ((p.grad.double() - r).norm() / (r.norm() + 1e-12)).item())
	del bf_first, bf_last

	pipe = Pipeline([first, last], ids[:mb], scheduler=scheduler, partitioner=False, placement=placement, all_ranks=len(set(placement)) > 1)
	pipe.zero_grad()
	result, loss = pipe(ids, tgt, loss_fn, split_size=mb)
	if len(set(placement)) > 1:
		from elf_amd.scheduling import OperationType as T

		kinds = [(op.op, op.rank) for op in pipe.schedule]
		for r in (0, 1):  # both ranks' streams ran, with their comm ops
			assert sum(k == (T.FORWARD, r) for k in kinds) == nmb and sum(k == (T.BACKWARD_INPUTS, r) for k in kinds) == nmb
		sends = [op for op in pipe.schedule if op.op == T.SEND_FORWARD and op.options.get("dst") is not None]
		recvs = [op for op in pipe.schedule if op.op == T.RECV_BACKWARD and op.options.get("src") is not None]
		assert len(sends) == nmb and all(op.rank == 0 for op in sends) and len(recvs) == nmb and all(op.rank == 0 for op in recvs)
		# 1F1B on the first of two ranks: two forwards in flight before the first backward
		first_b = next(i for i, k in enumerate(kinds) if k == (T.BACKWARD_INPUTS, 0))
		assert sum(k == (T.FORWARD, 0) for k in kinds[:first_b]) == 2
	assert len(result) == nmb and tuple(result[0].shape) == (mb, S, V)
	assert_close(torch.cat([r.float() for r in result]), logits.detach(), "logits")
	assert abs(float(loss) - float(want_loss.detach())) <= 1e-2 * float(want_loss.detach())
	for tag, mod, ref_mod in (("first", first, ref_first), ("last", last, ref_last)):
		ref_params = dict(ref_mod.named_parameters())
		for name, p in mod.named_parameters():
			assert_close(p.main_grad, ref_params[name].grad, f"grad {tag}.{name}", rel_fro=fro_bound[tag, name])
			assert_close(p.grad, ref_params[name].grad, f"bf16 grad {tag}.{name}", rel_fro=fro_bound[tag, name])


def test_memory_budget_with_first_and_last_stage():
	"""``Pipeline(..., memory_budget=)`` on stages that own the embedding and the head: profile_stage
	feeds token ids to the first stage and padded logits gradients to the last one, the ILP solved from
	those records rewrites the schedule under a tight budget, and the step gives the loss and gradients
	of the unconstrained one."""
	from elf_amd import losses, models
	from elf_amd.pipeline import Pipeline
	from elf_amd.scheduling import OperationType, OpOptions
	from elf_amd.scheduling.ilp import profile_stage

	V, d, S, mb, nmb = 1000, 256, 128, 4, 6
	g = torch.Generator().manual_seed(9)
	ids = torch.randint(0, V, (mb * nmb, S), generator=g).cuda()
	tgt = torch.randint(0, V, (mb * nmb, S), generator=g).cuda()

	def build(**kw):
		first = models.gpt_end_stage(2, d, 4, 1024, S, vocab_in=V, causal=True, seed=41)
		last = models.gpt_end_stage(2, d, 4, 1024, S, vocab_out=V, causal=True, seed=42)
		return Pipeline([first, last], ids[:mb], scheduler="afab", partitioner=False, placement=[0, 0], **kw), (first, last)

	plain, plain_mods = build()
	rec_first, nxt = profile_stage(plain.blocks[0], n_iter=2)
	rec_last, logits = profile_stage(plain.blocks[1], n_iter=2)
	T = mb * S
	assert tuple(nxt.shape) == (T, d) and tuple(logits.shape) == (T, V)
	assert rec_first["Minput"] == pytest.approx(T * 8 / 2**20) and rec_first["Moutput"] == pytest.approx(T * d * 2 / 2**20)
	assert rec_last["Moutput"] == pytest.approx(T * 1024 * 2 / 2**20)  # rows padded to 1024 columns
	for rec in (rec_first, rec_last):
		assert all(rec["T"][k] > 0 for k in "fbw") and rec["M"]["w"] == 0.0 and rec["M"]["f"] > rec["Mpeak_ckpt"] > 0
	plain.zero_grad()
	_, loss_plain = plain(ids, tgt, losses.cross_entropy, split_size=mb)

	# AFAB holds every micro-batch's stash at once: a budget of two thirds of that forces remat
	need = 2 * (rec_first["Mparams"] + rec_last["Mparams"]) + nmb * (rec_first["M"]["f"] + rec_last["M"]["f"])
	tight, tight_mods = build(memory_budget=0.67 * need)
	tight.zero_grad()
	_, loss_tight = tight(ids, tgt, losses.cross_entropy, split_size=mb)
	remat_ops = [op for op in tight.schedule if op.op in (OperationType.RECOMPUTE_FORWARD, OperationType.RECOMPUTE_BACKWARD_INPUTS) or op.options.get(OpOptions.REMAT_STRATEGY) is not None]
	assert remat_ops, "the budget must have forced rematerialisation"
	assert float(loss_tight) == pytest.approx(float(loss_plain), rel=1e-3)
	for mod_p, mod_t in zip(plain_mods, tight_mods):
		want = dict(mod_p.named_parameters())
		for name, p in mod_t.named_parameters():
			assert_close(p.main_grad, want[name].main_grad, f"grad {name} under the budget", rel_max=2e-3, rel_fro=2e-3)
