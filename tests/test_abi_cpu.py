"""The C-ABI library without a GPU: it loads, exports every entry point the header declares,
rejects bad arguments before touching the device, and its pinned arena follows the reference's
placement policy (checked against oracle/pinned_pool.py and hand-worked sequences)."""

import ctypes
import os
import random
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
	from elf_amd import _lib

	return _lib.load()


def _declared():
	text = open(os.path.join(ROOT, "include", "elf_stage.h")).read()
	text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
	return sorted(set(re.findall(r"\b(elf_[a-z0-9_]+)\s*\(", text)))


def test_exports_every_declared_symbol(lib):
	names = _declared()
	assert len(names) >= 40
	for n in names:
		assert hasattr(lib, n), f"{n} is declared in include/elf_stage.h but not exported"


def test_bindings_cover_the_header():
	import elf_amd.execution  # noqa: F401  (registers the stage and pool signatures)
	from elf_amd import _lib

	assert set(_declared()) == set(_lib.exported_symbols())


def test_argument_errors_without_device(lib):
	from elf_amd import _lib

	assert lib.elf_abi_version() == 1
	rc = lib.elf_gemm_bf16(0, 0, 0, 64, 64, None, 64, None, 64, None, 64, 0, None, 0, 0, 0, None)
	assert rc == -1 and b"empty problem" in lib.elf_last_error()
	rc = lib.elf_gemm_bf16(0, 0, 64, 64, 70, 16, 64, 16, 64, 16, 64, 0, None, 0, 0, 0, None)
	assert rc == -1 and b"multiple of 64" in lib.elf_last_error()
	rc = lib.elf_attn_fwd(16, 16, 16, 16, 16, 64, 64, 64, 64, 1, 100, 4, 4, 64, 0, 0.125, None)
	assert rc == -1 and b"multiple of 128" in lib.elf_last_error()
	rc = lib.elf_attn_fwd(16, 16, 16, 16, 16, 64, 64, 64, 64, 1, 128, 6, 4, 64, 0, 0.125, None)
	assert rc == -1 and b"Hkv" in lib.elf_last_error()
	rc = lib.elf_norm_fwd(0, 16, 16, None, 16, 16, 4, 100, 1e-5, None)
	assert rc == -1
	with pytest.raises(_lib.ElfStageError):
		_lib.check(rc, "elf_norm_fwd")
	assert lib.elf_norm_bwd_workspace_floats(8192, 4096) == 512 * 2 * 4096
	# bf16 dQ partials of the 32 key tiles (causal: tile kt only meets the queries from 128 kt on) + two floats per (token, head)
	stats = 2 * (2 * 4096 * 32 * 4)
	assert lib.elf_attn_bwd_workspace_bytes(2, 4096, 32, 128, 0) == 2 * (32 * 4096) * 32 * 128 * 2 + stats
	assert lib.elf_attn_bwd_workspace_bytes(2, 4096, 32, 128, 1) == 2 * sum(4096 - 128 * kt for kt in range(32)) * 32 * 128 * 2 + stats


def test_stage_create_rejects_bad_configs(lib):
	from elf_amd.execution.block import StageConfig

	h = ctypes.c_void_p()
	bad = [
		dict(arch=7), dict(n_heads=5, n_kv_heads=2), dict(head_dim=96), dict(seq=100), dict(d_model=100),
		dict(arch=0, n_heads=4, n_kv_heads=2),
	]
	base = dict(arch=1, n_blocks=1, d_model=256, n_heads=4, n_kv_heads=2, head_dim=64, ffn=512, seq=128, mb=1, causal=1, eps=1e-5, rope_theta=5e5)
	for delta in bad:
		cfg = StageConfig(**{**base, **delta})
		assert lib.elf_stage_create(ctypes.byref(cfg), ctypes.byref(h)) == -1, delta
		assert lib.elf_last_error()


def _pool(host=True):
	from elf_amd.execution import PinnedHostTensorPool

	return PinnedHostTensorPool(host_backing=host)


def test_pinned_pool_hand_worked_sequence():
	p = _pool()
	a, pa, oa = p.allocate(100, "bf16")        # new parent of 128 elements
	assert (pa, oa) == (0, 0) and p.size() == 128 * 2
	b, pb, ob = p.allocate(20, "bf16")         # carved from the remaining (100, 28)
	assert (pb, ob) == (0, 100) and p.free_segments() == [[(120, 8)]]
	c, pc, oc = p.allocate(9, "bf16")          # does not fit in 8 -> second parent of 16
	assert (pc, oc) == (1, 0) and p.free_segments() == [[(120, 8)], [(9, 7)]]
	assert p.free(a)
	assert p.free_segments()[0] == [(0, 100), (120, 8)]
	d, pd, od = p.allocate(50, "bf16")         # first fit: start of the (0, 100) hole
	assert (pd, od) == (0, 0) and p.free_segments()[0] == [(50, 50), (120, 8)]
	assert p.free(b)                            # (100, 20) merges with both neighbours
	assert p.free_segments()[0] == [(50, 78)]
	e, pe, oe = p.allocate(5, "f32")           # other dtype -> its own parent
	assert (pe, oe) == (2, 0) and p.size() == 128 * 2 + 16 * 2 + 8 * 4
	assert not p.free(12345)                    # foreign blocks are ignored
	for blk in (c, d, e):
		assert p.free(blk)
	assert p.free_segments() == [[(0, 128)], [(0, 16)], [(0, 8)]]
	p.reserve(1000, "f32")                      # ceil(1000/4) = 250 -> 256 elements
	assert p.size() == 128 * 2 + 16 * 2 + 8 * 4 + 256 * 4
	f, pf, of = p.allocate(0, "f32")           # a request of 0 takes 1 element, first fit in parent 2
	assert (pf, of) == (2, 0)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_pinned_pool_matches_policy_model(seed):
	from oracle.pinned_pool import PoolModel

	rng = random.Random(seed)
	p, m = _pool(), PoolModel()
	live = []
	sizes = {"bf16": 2, "f32": 4}
	for step in range(400):
		if live and rng.random() < 0.45:
			addr, pi, off, n, esz = live.pop(rng.randrange(len(live)))
			assert p.free(addr) and m.free(pi, off)
		else:
			dt = rng.choice(["bf16", "bf16", "f32"])
			n = rng.choice([1, 3, 17, 64, 100, 1000, 4096, rng.randrange(1, 5000)])
			addr, pi, off = p.allocate(n, dt)
			assert (pi, off) == m.allocate(n, dt), f"step {step}"
			live.append((addr, pi, off, n, sizes[dt]))
		assert p.free_segments() == [pp["free"] for pp in m.parents]
		# live blocks never overlap (byte ranges)
		spans = sorted((a, a + n * e) for a, _, _, n, e in live)
		assert all(spans[i][1] <= spans[i + 1][0] for i in range(len(spans) - 1))
	assert p.size() == m.size_bytes(sizes)
	for addr, pi, off, n, esz in live:
		assert p.free(addr)
	assert all(len(s) == 1 and s[0][0] == 0 for s in p.free_segments())
	assert all((s[0][1] & (s[0][1] - 1)) == 0 for s in p.free_segments()), "parent sizes are powers of two"
