"""``Pipeline`` over the native stage executor (reference API: elf/pipeline.py:97-295): two stages on
one rank under AFAB, and one stage under ZB-H1, against the oracle stages driven by hand with the
same loss.  Tolerances as for the stage tests (rel 2e-2 of max, 1e-2 Frobenius)."""

import pytest
import torch
import torch.nn.functional as F

from tests.helpers import assert_close, cfg_from_stage, oracle_params_from_stage, perturb_norms, product_grads

pytestmark = pytest.mark.gpu


def _stages(n):
	from elf_amd import models

	out = []
	for i in range(n):
		st = models.llama_stage(1, 256, 2, 1, 512, 128, head_dim=128, seed=20 + i)
		perturb_norms(st)
		out.append(st)
	return out


# (scheduler, placement, total batch, split): an even split, a batch the split size does not divide (short
# last micro-batch: elf/pipeline.py:497-500) and an explicit list of sizes (elf/pipeline.py:501-503)
@pytest.mark.parametrize("case", [("afab", [0, 0], 6, 2), ("zbh1", [0], 6, 2), ("afab", [0, 0], 5, 2), ("zbh1", [0], 5, [1, 2, 2])])
def test_pipeline_step_matches_oracle(case):
	from elf_amd.pipeline import Pipeline, PipelineConfig
	from oracle import stage_ref as R

	sched, placement, total, split = case
	mb = 2
	sizes = split if isinstance(split, list) else [mb] * (total // mb) + ([total % mb] if total % mb else [])
	nmb, starts = len(sizes), [sum(sizes[:i]) for i in range(len(sizes))]
	stages = _stages(len(placement))
	refs = [R.RefStage(cfg_from_stage(st, mb), oracle_params_from_stage(st), device="cuda") for st in stages]
	S, d = stages[0].seq_len, 256
	g = torch.Generator().manual_seed(7)
	batch = torch.randn(total, S, d, generator=g).to(torch.bfloat16).cuda()
	target = torch.randn(total, S, d, generator=g).to(torch.bfloat16).cuda()

	pipe = Pipeline(stages if len(stages) > 1 else stages[0], batch[:mb], config=PipelineConfig(scheduler=sched, partitioner=False, placement=placement))
	assert pipe.is_first() and pipe.is_last() and [b.id for b in pipe.blocks] == list(range(len(placement)))
	pipe.zero_grad()
	result, loss = pipe(batch, target, F.mse_loss, split_size=split)
	assert len(result) == nmb and pipe.last_nmb == nmb
	assert set(pipe.stats) == {"total", "idle", "start_idle", "end_idle", "bubble"}
	assert list(pipe.detailed_stats["memories"]) == [str(op) for op in pipe.schedule]

	want_loss = 0.0
	for m in range(nmb):
		x = batch[starts[m]:starts[m] + sizes[m]]
		for ref in refs:
			x = ref.forward(m, x)
		y = x.detach().float().requires_grad_()
		t = target[starts[m]:starts[m] + sizes[m]].float()
		l = F.mse_loss(y, t, reduction="sum") / (S * d)
		l.backward()
		want_loss += float(l.detach())
		assert_close(result[m].reshape(sizes[m], S, d), x, f"{sched} output[{m}]")
		dy = y.grad.to(torch.bfloat16)
		for ref in reversed(refs):
			dy = ref.backward_inputs(m, dy)
		for ref in refs:
			ref.backward_params(m)
	for ref in refs:
		ref.scale_grads(total)
	assert abs(float(loss) - want_loss / total) <= 2e-2 * abs(want_loss / total)
	for st, ref in zip(stages, refs):
		got, want = product_grads(st), ref.grads()
		for name in sorted(want):
			assert_close(got[name], want[name], f"{sched} grad {name}")

	# a second step with the same batch reuses the schedule and gives the same loss
	pipe.zero_grad()
	_, loss2 = pipe(batch, target, F.mse_loss, split_size=split)
	assert abs(float(loss2) - float(loss)) <= 1e-3 * abs(float(loss))
	assert sum(p.numel() for p in pipe.parameters()) == sum(p.numel() for st in stages for p in st.parameters())
	pipe.clear()


def test_pipeline_checkpoint_round_trip(tmp_path):
	"""The reference's per-rank checkpoint layout (elf/pipeline.py:346-368), written and read back: the
	restored weights are the ones the library computes with."""
	from elf_amd.pipeline import Pipeline

	stages = _stages(2)
	mb, S, d = 2, stages[0].seq_len, 256
	batch = torch.randn(mb * 2, S, d, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).cuda()
	pipe = Pipeline(stages, batch[:mb], scheduler="afab", partitioner=False, placement=[0, 0])
	out0, _ = pipe(batch, batch, F.mse_loss, split_size=mb)
	pipe.checkpoint(epoch="e1", dir_path=str(tmp_path))
	state = torch.load(tmp_path / "e1" / "dp0_pp0.pt", weights_only=True)
	assert {"rank", "pp", "dp", "epoch", "state_dict_0", "state_dict_1"} <= set(state) and state["epoch"] == "e1"
	assert set(state["state_dict_0"]) == set(stages[0].state_dict())
	with torch.no_grad():
		for p in pipe.parameters():
			p.mul_(0.5)
	out1, _ = pipe(batch, batch, F.mse_loss, split_size=mb)
	assert not torch.equal(out1[0], out0[0])
	pipe.load_checkpoint(epoch="e1", dir_path=str(tmp_path))
	out2, _ = pipe(batch, batch, F.mse_loss, split_size=mb)
	assert all(torch.equal(a, b) for a, b in zip(out2, out0))
	pipe.save(str(tmp_path / "full.pt"))
	full = torch.load(tmp_path / "full.pt", weights_only=True)
	assert set(full) == {n for n, _ in pipe.named_parameters()} and set(pipe.gather_parameters()) == set(full)


def test_pipeline_rejects_what_this_build_does_not_run():
	from elf_amd.pipeline import Pipeline

	st = _stages(1)[0]
	with pytest.raises(NotImplementedError):
		Pipeline(st, torch.zeros(2, 128, 256), scheduler="afab", placement=[0])  # default partitioner needs a tracer
	with pytest.raises(ValueError):
		Pipeline(st, None, scheduler="afab", partitioner=False, placement=[0])  # no sample, no mb_size
	pipe = Pipeline(st, None, scheduler="afab", partitioner=False, placement=[0], mb_size=2)
	with pytest.raises(ValueError):
		pipe(torch.zeros(6, 128, 256, dtype=torch.bfloat16, device="cuda"), None, None, split_size=3)  # larger than the stage was sized for
