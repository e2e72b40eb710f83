"""Stage executors with the slot semantics of the reference's PipelineBlock.

``Variable`` restates elf/execution/block.py:18-131 (three per-micro-batch slot lists with
set-once / pop-once rules).  ``HipStageBlock`` is the PipelineBlock duck type (block.py:134-694)
for a stage made of transformer blocks on an MI355X: every compute op is one call into
libelf_stage.so; torch only owns the boundary tensors, the weights and the gradient buffers.
There is no other execution path in this class: without the library, or for a module it does not
recognise, construction raises.
"""

import ctypes
import logging

import torch

from .. import _lib
from ..models import EndStage, LlamaBlock, TransformerBlock
from ..scheduling import OpOptions
from ..utils import Timer

logger = logging.getLogger("block")

__all__ = ["Variable", "StageBlockBase", "HipStageBlock", "StageConfig", "MemStats"]


class Variable:
	"""One input or output of a block: data received and waiting (``to_process``: (work, tensor)),
	data kept for the backward (``saved``) and data ready to leave (``to_send``), per micro-batch.
	A slot can be set once and is emptied when read."""

	def __init__(self, name, peer, group=None):
		self.name, self.peer, self.group = name, peer, group
		self.metadata = None
		self.was_metadata_sent = False
		self.to_process, self.saved, self.to_send = [], [], []

	def get(self, queue, mb_id, delete=True):
		if len(queue) <= mb_id:
			raise Exception(f"Variable {self.name} - Data queue shorter than mb_id {mb_id}")
		data = queue[mb_id]
		if data is None:
			raise Exception(f"Variable {self.name} - Trying to pop data at mb_id {mb_id}, but it's empty")
		if delete:
			queue[mb_id] = None
		return data

	def set(self, queue, mb_id, value):
		if len(queue) <= mb_id:
			queue.extend([None] * (mb_id + 1 - len(queue)))
		if queue[mb_id] is not None:
			raise Exception(f"Variable {self.name} - Trying to set data at mb_id {mb_id}, but it's already set")
		queue[mb_id] = value

	def wait_and_pop(self, mb_id):
		work, tensor = self.get(self.to_process, mb_id)
		if work is not None:
			work.wait()
		return tensor.detach()

	def clear(self):
		self.to_process.clear()
		self.saved.clear()
		self.to_send.clear()

	def _state(self):
		n = [sum(x is not None for x in q) for q in (self.to_process, self.saved, self.to_send)]
		return f"{self} - to process: {n[0]}, saved: {n[1]}, to send: {n[2]}"

	def __str__(self):
		return f"Variable(name={self.name},peer={self.peer},metadata={self.metadata})"

	__repr__ = __str__


class StageConfig(ctypes.Structure):
	"""elf_stage_cfg of include/elf_stage.h."""

	_fields_ = [
		("arch", ctypes.c_int), ("n_blocks", ctypes.c_int), ("d_model", ctypes.c_int), ("n_heads", ctypes.c_int),
		("n_kv_heads", ctypes.c_int), ("head_dim", ctypes.c_int), ("ffn", ctypes.c_int), ("seq", ctypes.c_int),
		("mb", ctypes.c_int), ("causal", ctypes.c_int), ("eps", ctypes.c_float), ("rope_theta", ctypes.c_double),
	]


class MemStats(ctypes.Structure):
	"""elf_mem_stats of include/elf_stage.h."""

	_fields_ = [(n, ctypes.c_int64) for n in ("live_bytes", "peak_bytes", "reserved_bytes", "pinned_bytes", "d2h_bytes", "h2d_bytes", "workspace_bytes")]


_P = ctypes.c_void_p
_I = ctypes.c_int
for _name, _ret, _args in [
	("elf_stage_create", _I, [ctypes.POINTER(StageConfig), ctypes.POINTER(_P)]),
	("elf_stage_destroy", None, [_P]),
	("elf_stage_bind_param", _I, [_P, _I, _I, _P, _P]),
	("elf_stage_set_ends", _I, [_P, _I, _I, _I, _I]),
	("elf_stage_set_mb_samples", _I, [_P, _I, _I]),
	("elf_stage_set_lean_stash", _I, [_P, _I]),
	("elf_stage_forward", _I, [_P, _I, _P, _P, ctypes.c_uint32, _P]),
	("elf_stage_backward_inputs", _I, [_P, _I, _P, _P, _P, ctypes.c_uint32, _P]),
	("elf_stage_backward_params", _I, [_P, _I, _P]),
	("elf_stage_bind_grad_bf16", _I, [_P, _I, _I, _P]),
	("elf_stage_backward_params_scaled", _I, [_P, _I, ctypes.c_float, _P]),
	("elf_stage_recompute_forward", _I, [_P, _I, _P, _I, _P]),
	("elf_stage_recompute_backward_inputs", _I, [_P, _I, _P, _P]),
	("elf_stage_offload", _I, [_P, _I, _P]),
	("elf_stage_prefetch", _I, [_P, _I, _P]),
	("elf_stage_release", _I, [_P, _I]),
	("elf_stage_reserve_pinned", _I, [_P, ctypes.c_int64]),
	("elf_stage_clear", _I, [_P]),
	("elf_stage_mem_stats", _I, [_P, ctypes.POINTER(MemStats)]),
	("elf_stage_reset_peak", _I, [_P]),
]:
	_lib.register(_name, _ret, _args)

ARCH_GPT, ARCH_LLAMA = 0, 1
FWD_REMAT_ROOT, FWD_REMAT_ATTN, FWD_OFFLOAD, FWD_REMAT_NORM = 1, 2, 4, 8
BWD_RECOMPUTE_ACTIVATIONS, BWD_RECOMPUTE_GRADIENTS = 1, 2
# parameter ids of elf_stage_bind_param
P_NORM1_G, P_NORM1_B, P_WQKV, P_WO, P_NORM2_G, P_NORM2_B, P_W1, P_W2 = range(8)
P_EMBED, P_FNORM_G, P_FNORM_B, P_HEAD = 8, 9, 10, 11  # stage-level, bound with block = -1


def _stream():
	return torch.cuda.current_stream().cuda_stream


class StageBlockBase:
	"""What every stage executor of this build shares: identity, the ``Variable`` slots of the stage's
	signature, and the transfer ops (on one GPU a peer is either in this process or stands for another
	rank and is fed from local buffers, ``set_boundary``).  Sub-classes add the compute ops of the
	PipelineBlock duck type (elf/execution/block.py:134-694)."""

	def _init_common(self, model, id_, placement, signature, pp_group, dp_group, recv_pgs, send_pgs):
		self.id = id_
		self.placement = placement
		self.rank = placement[id_]
		self.is_first = id_ == 0
		self.is_last = id_ == len(placement) - 1
		self.signature = signature
		self.pp_group, self.dp_group = pp_group, dp_group
		self.recv_pgs, self.send_pgs = recv_pgs, send_pgs
		self.model = model.cuda()
		self.device = torch.cuda.current_device()
		self.input_variables = [Variable(n, s, pp_group) for n, s in zip(signature.inputs, signature.sources)]
		self.output_variables = [[Variable(n, d, pp_group) for d in dsts] for n, dsts in zip(signature.outputs, signature.targets)]
		self.compute_time = []
		self.send_ops = []

	def __str__(self):
		return f"Rank {self.rank} - Layer {self.id}"

	def _timed(self, name):
		t = Timer(name=name)
		self.compute_time.append(t)
		return t

	# ------------------------------------------------------------------ transfers (single GPU: peers are local or absent)
	def set_boundary(self, inputs=None, grads=None, keep_sent=False):
		"""Stand-ins for the stage's remote peers: ``inputs(mb)`` / ``grads(mb)`` (callables or
		sequences of tensors) supply what RECV_FORWARD / RECV_BACKWARD would receive from another
		rank; what SEND_FORWARD / SEND_BACKWARD would ship is dropped, or collected in
		``sent_forward`` / ``sent_backward`` when ``keep_sent`` is set."""
		self._feed_x = (lambda mb: inputs[mb]) if inputs is not None and not callable(inputs) else inputs
		self._feed_dy = (lambda mb: grads[mb]) if grads is not None and not callable(grads) else grads
		self._keep_sent = keep_sent
		self.sent_forward, self.sent_backward = {}, {}

	def _remote(self, peer):
		return peer is not None and self.placement[peer] != self.rank and peer not in getattr(self, "local_ids", ())

	def _need_feed(self, feed, what):
		if feed is None:
			raise NotImplementedError(f"{self}: {what} from another rank needs set_boundary(): this build feeds stage boundaries from local buffers")
		return feed

	def _sends_input_grads(self):
		return True

	def send_forward(self, mb_id, **options):
		dst = options.get("dst")
		if self._remote(dst):
			for targets in self.output_variables:
				for target in targets:
					if target.peer == dst:
						y = target.get(target.to_send, mb_id)
						if getattr(self, "_keep_sent", False):
							self.sent_forward[mb_id] = y

	def send_backward(self, mb_id, **options):
		dst = options.get("dst")
		if self._remote(dst) and self._sends_input_grads():
			for var in self.input_variables:
				if var.peer == dst:
					dx = var.get(var.to_send, mb_id)
					if getattr(self, "_keep_sent", False):
						self.sent_backward[mb_id] = dx

	def recv_forward(self, mb_id, mb_size, **options):
		src = options.get("src")
		if self._remote(src):
			for var in self.input_variables:
				if var.peer == src:
					x = self._need_feed(getattr(self, "_feed_x", None), "recv_forward")(mb_id)
					var.set(var.to_process, mb_id, (None, x))

	def recv_backward(self, mb_id, mb_size, **options):
		src = options.get("src")
		if self._remote(src):
			for targets in self.output_variables:
				for target in targets:
					if target.peer == src:
						dy = self._need_feed(getattr(self, "_feed_dy", None), "recv_backward")(mb_id)
						target.set(target.to_process, mb_id, (None, dy))

	def _wait_for_send_ops(self):
		self.send_ops.clear()

	def all_reduce_param_grads(self, **options):
		if self.dp_group is None:
			return
		import torch.distributed as dist

		for g in self._grad_buffers():
			dist.all_reduce(g, group=self.dp_group, op=dist.ReduceOp.AVG, async_op=True)


class HipStageBlock(StageBlockBase):
	"""One pipeline stage (a chain of TransformerBlock or LlamaBlock modules) executed by
	libelf_stage.so.

	The module's linear weights are re-homed into fused bf16 buffers (q|k|v rows, gate|up rows) of
	which the original ``nn.Parameter``s become views, so optimizers keep working on the module.
	Weight gradients accumulate in fp32 (``param.main_grad`` views of fused fp32 buffers) across
	the W passes of a step; ``scale_grads`` divides by the batch size and writes the bf16
	``param.grad`` the reference exposes.

	``lean_stash`` (False / 0, True / 1, 2): at level 1 forwards keep neither the norm outputs nor the FFN
	activation and B forms them again (a third less held between F and B, same results); level 2 also leaves
	out the QKV projection and the attention residual, which B forms again with two GEMMs (a quarter less
	again, about 5 % of a block's time).  ``Pipeline`` picks the level under a memory budget
	(``set_lean_stash``: between steps only).
	"""

	def __init__(self, model, id_, placement, signature, pp_group=None, dp_group=None, recv_pgs=None, send_pgs=None, *, mb_size, seq_len=None, lean_stash=False):
		if not torch.cuda.is_available():
			raise _lib.ElfStageError("HipStageBlock needs an MI355X: there is no CPU path for the stage kernels")
		self.lib = _lib.load()
		self._handle = None
		self._init_common(model, id_, placement, signature, pp_group, dp_group, recv_pgs, send_pgs)
		if len(self.input_variables) != 1 or len(self.output_variables) != 1:
			raise _lib.ElfStageError("HipStageBlock: a chain of transformer blocks has one input and one output (AutogradStageBlock runs stages with other signatures)")
		self._samples = {}  # mb -> sequences in it, where fewer than mb_size
		self._kept = {}  # mb -> external tensors the library still points at (x until B/recompute, dy until W)
		self._remat_cache = {}  # id(strategy) -> (strategy, forward flags)
		self.lean_stash = int(lean_stash)
		self._build(mb_size, seq_len)

	def set_lean_stash(self, level):
		"""What the forwards issued from now on keep (0, 1 or 2, see the class docstring).  Between steps only: a
		micro-batch's B reads the stash its own F left."""
		_lib.check(self.lib.elf_stage_set_lean_stash(self._handle, int(level)), "elf_stage_set_lean_stash")
		self.lean_stash = int(level)

	# ------------------------------------------------------------------ set-up
	def _build(self, mb_size, seq_len):
		core = self.model.blocks if isinstance(self.model, EndStage) else self.model
		self.ends = self.model if isinstance(self.model, EndStage) else None
		blocks = list(core.children()) if not isinstance(core, (TransformerBlock, LlamaBlock)) else [core]
		if not blocks or not all(isinstance(b, (TransformerBlock, LlamaBlock)) for b in blocks) or len({type(b) for b in blocks}) != 1:
			raise _lib.ElfStageError("HipStageBlock: the stage must be a chain of TransformerBlock or of LlamaBlock modules")
		b0 = blocks[0]
		llama = isinstance(b0, LlamaBlock)
		seq = seq_len or getattr(core, "seq_len", None)
		if seq is None:
			raise _lib.ElfStageError("HipStageBlock: seq_len is required (StageModule carries it)")
		att = b0.attn
		cfg = StageConfig(
			ARCH_LLAMA if llama else ARCH_GPT, len(blocks), b0.dim, att.num_heads, att.num_kv_heads, att.head_dim, b0.ffn_dim,
			seq, mb_size, int(b0.causal), float(b0.eps), float(b0.rope_theta) if llama else 0.0,
		)
		self.cfg = cfg
		self.blocks = blocks
		dev = torch.device("cuda", self.device)
		self._fused_w, self._fused_g, self._fused_bf16_grad = [], [], []  # the fused buffers (kept alive here)
		self._w_scaled = []  # indices of the fused buffers of linear layers: what a W with the folded gradient scale covers
		self._folded_scale = None  # 1 / batch size that the step's last W applied, until scale_grads has run
		self._param_loc = {}  # parameter -> (fused buffer index, first row, rows)
		self.main_grads = {}  # parameter -> fp32 accumulator view
		handle = ctypes.c_void_p()
		_lib.check(self.lib.elf_stage_create(ctypes.byref(cfg), ctypes.byref(handle)), "elf_stage_create")
		self._handle = handle
		if self.lean_stash:
			_lib.check(self.lib.elf_stage_set_lean_stash(self._handle, self.lean_stash), "elf_stage_set_lean_stash")

		def fuse(params, pad_rows=0):
			"""Move `params` (row blocks of one matrix) into one bf16 buffer + one fp32 grad buffer
			(`pad_rows` extra zero rows at the end)."""
			rows = sum(p.shape[0] for p in params) + pad_rows
			w = torch.zeros((rows,) + tuple(params[0].shape[1:]), dtype=torch.bfloat16, device=dev)
			g = torch.zeros(w.shape, dtype=torch.float32, device=dev)
			r = 0
			for p in params:
				n = p.shape[0]
				w[r : r + n].copy_(p.data)
				p.data = w[r : r + n]
				p.main_grad = g[r : r + n]
				self.main_grads[p] = p.main_grad
				self._param_loc[p] = (len(self._fused_w), r, n)
				r += n
			self._fused_w.append(w)
			self._fused_g.append(g)
			self._fused_bf16_grad.append(None)
			return w, g

		def bind(block, pid, w, g):
			_lib.check(self.lib.elf_stage_bind_param(self._handle, block, pid, w.data_ptr(), g.data_ptr()), "elf_stage_bind_param")
			if pid in (P_WQKV, P_WO, P_W1, P_W2, P_HEAD):
				# linear layers: the bf16 gradient the step's last W writes together with the scaled accumulator
				i = len(self._fused_w) - 1
				self._fused_bf16_grad[i] = torch.empty_like(w)
				self._w_scaled.append(i)
				_lib.check(self.lib.elf_stage_bind_grad_bf16(self._handle, block, pid, self._fused_bf16_grad[i].data_ptr()), "elf_stage_bind_grad_bf16")

		for i, b in enumerate(blocks):
			m = b.mlp
			groups = {
				P_NORM1_G: [b.norm1.weight], P_NORM2_G: [b.norm2.weight],
				P_WQKV: [att_i.weight for att_i in (b.attn.q_proj, b.attn.k_proj, b.attn.v_proj)], P_WO: [b.proj.weight],
				P_W1: [m.gate_proj.weight, m.up_proj.weight] if llama else [m.fc1.weight],
				P_W2: [m.down_proj.weight if llama else m.fc2.weight],
			}
			if not llama:
				groups[P_NORM1_B] = [b.norm1.bias]
				groups[P_NORM2_B] = [b.norm2.bias]
			for pid, params in groups.items():
				if any(p.dtype != torch.bfloat16 for p in params):
					raise _lib.ElfStageError("HipStageBlock: parameters must be bf16")
				w, g = fuse(params)
				bind(i, pid, w, g)
		self.T = mb_size * seq
		self.d = b0.dim
		self.mb_size, self.seq = mb_size, seq
		# first / last stage of a pipeline: token embedding, (final norm,) output head
		self.vocab_in = self.vocab_out = self.vld = 0
		if self.ends is not None:
			e = self.ends
			stage_level = {}
			if e.embed is not None:
				self.vocab_in = e.embed.num_embeddings
				stage_level[P_EMBED] = ([e.embed.weight], 0)
			if e.head is not None:
				self.vocab_out = e.head.out_features
				self.vld = -(-self.vocab_out // 64) * 64
				stage_level[P_HEAD] = ([e.head.weight], self.vld - self.vocab_out)
			if e.norm_f is not None:
				stage_level[P_FNORM_G] = ([e.norm_f.weight], 0)
				if not llama:
					stage_level[P_FNORM_B] = ([e.norm_f.bias], 0)
			_lib.check(self.lib.elf_stage_set_ends(self._handle, self.vocab_in, self.vocab_out, self.vld, int(e.norm_f is not None)), "elf_stage_set_ends")
			for pid, (params, pad) in stage_level.items():
				if any(p.dtype != torch.bfloat16 for p in params):
					raise _lib.ElfStageError("HipStageBlock: parameters must be bf16")
				w, g = fuse(params, pad)
				bind(-1, pid, w, g)

	def __del__(self):
		try:
			if self._handle:
				self.lib.elf_stage_destroy(self._handle)
				self._handle = None
		except Exception:
			pass

	def _rows(self, mb_id):
		"""Tokens in micro-batch ``mb_id`` (fewer than ``T`` for a short last micro-batch)."""
		return self._samples.get(mb_id, self.mb_size) * self.seq

	def _set_samples(self, mb_id, t, per_sample):
		"""Tell the library how many sequences the incoming micro-batch holds (block.py:210-263 takes
		whatever batch arrives; here the stage was sized for ``mb_size`` and accepts 1..mb_size)."""
		n, rem = divmod(t.numel(), per_sample)
		if rem or not 1 <= n <= self.mb_size:
			raise _lib.ElfStageError(f"{self}: stage input of {tuple(t.shape)} is not 1..{self.mb_size} sequences of {self.seq} tokens")
		if n != self._samples.get(mb_id, self.mb_size):
			_lib.check(self.lib.elf_stage_set_mb_samples(self._handle, mb_id, n), "elf_stage_set_mb_samples")
			if n == self.mb_size:
				self._samples.pop(mb_id, None)
			else:
				self._samples[mb_id] = n

	def _check_io(self, t, what, mb_id):
		rows = self._rows(mb_id)
		if t.dtype != torch.bfloat16 or not t.is_cuda or t.numel() != rows * self.d:
			raise _lib.ElfStageError(f"{self}: {what} must be a bf16 GPU tensor of {rows}x{self.d} elements, got {tuple(t.shape)} {t.dtype} {t.device}")
		return t.contiguous()

	def _check_ids(self, t, mb_id):
		rows = self._rows(mb_id)
		if t.dtype != torch.int64 or not t.is_cuda or t.numel() != rows:
			raise _lib.ElfStageError(f"{self}: the input of a first stage must be an int64 GPU tensor of {rows} token ids, got {tuple(t.shape)} {t.dtype} {t.device}")
		return t.contiguous()

	def _new_output(self, x, mb_id):
		"""(buffer the library writes, tensor handed on).  Last stage: logits [rows, vld] with the
		padding columns hidden from the caller; otherwise activations shaped like the input."""
		n = self._samples.get(mb_id, self.mb_size)
		if self.vocab_out:
			buf = torch.empty(n * self.seq, self.vld, dtype=torch.bfloat16, device=x.device)
			return buf, buf.view(n, self.seq, self.vld)[..., : self.vocab_out]
		if self.vocab_in:
			buf = torch.empty(n, self.seq, self.d, dtype=torch.bfloat16, device=x.device)
			return buf, buf
		buf = torch.empty_like(x)
		return buf, buf

	def _check_dy(self, dy, mb_id):
		"""Gradient of the stage output in the layout the library reads."""
		if not self.vocab_out:
			return self._check_io(dy, "output gradient", mb_id)
		rows = self._rows(mb_id)
		if dy.dtype != torch.bfloat16 or not dy.is_cuda or dy.numel() != rows * self.vocab_out:
			raise _lib.ElfStageError(f"{self}: the gradient of the logits must be a bf16 GPU tensor of {rows}x{self.vocab_out} elements, got {tuple(dy.shape)} {dy.dtype} {dy.device}")
		if self.vld == self.vocab_out:
			return dy.contiguous()
		if self._rows_padded(dy, rows):
			# rows already sit vld apart (the layout elf_amd.losses writes): read in place, with the
			# columns past the vocabulary cleared so they add nothing to dX and dW
			buf = torch.as_strided(dy, (rows, self.vld), (self.vld, 1))
			buf[:, self.vocab_out :].zero_()
			return buf
		pad = torch.zeros(rows, self.vld, dtype=torch.bfloat16, device=dy.device)
		pad[:, : self.vocab_out] = dy.reshape(rows, self.vocab_out)
		return pad

	def _rows_padded(self, dy, rows):
		"""Whether ``dy`` is a [..., vocab_out] view whose rows are exactly ``vld`` elements apart inside
		one allocation that holds all ``rows * vld`` of them."""
		if dy.dim() < 2 or dy.stride(-1) != 1 or dy.stride(-2) != self.vld or dy.data_ptr() % 16:
			return False
		expect = self.vld
		for size, stride in zip(reversed(dy.shape[:-1]), reversed(dy.stride()[:-1])):
			if size != 1 and stride != expect:
				return False
			expect *= size
		room = dy.untyped_storage().nbytes() // dy.element_size() - dy.storage_offset()
		return room >= rows * self.vld

	def _remat_flags(self, strategy):
		"""Forward flags for a ``remat_strategy`` (elf/execution/remat.py:26-74: every module the strategy
		selects runs under ``checkpoint``).  What this executor can express: the stage root (whole-stage
		checkpoint), all attention cores, all norm modules; an activation module (``nn.GELU``) may be
		selected too and changes nothing, because the only tensor it would keep is its own input, which the
		stash holds as the FFN pre-activation either way; ``nn.Dropout`` modules do not occur in these
		blocks.  A strategy that selects nothing runs a plain forward, as in the reference.  Anything else
		(single blocks, linears, some but not all modules of a kind) raises: a remat decision is never
		dropped silently."""
		if strategy is None:
			return 0
		key = id(strategy)
		cached = self._remat_cache.get(key)
		if cached is not None and cached[0] is strategy:
			return cached[1]
		named = list(self.model.named_modules())
		selected = [(n, m) for n, m in named if strategy(n, m)]
		if any(n == "" for n, _ in selected):
			flags = FWD_REMAT_ROOT
		else:
			norms, cores, acts = set(), set(), set()
			for b in self.blocks:
				norms.update((id(b.norm1), id(b.norm2)))
				cores.add(id(b.attn.attn))
				if hasattr(b.mlp, "activation"):
					acts.add(id(b.mlp.activation))
			if self.ends is not None and self.ends.norm_f is not None:
				norms.add(id(self.ends.norm_f))
			chosen = {id(m) for _, m in selected}
			flags = 0
			for group, flag in ((norms, FWD_REMAT_NORM), (cores, FWD_REMAT_ATTN), (acts, 0)):
				hit = chosen & group
				if hit and hit != group:
					raise _lib.ElfStageError(f"{self}: remat_strategy selects some but not all modules of one kind; this executor checkpoints a kind of module for the whole stage")
				if hit:
					flags |= flag
			other = [n for n, m in selected if id(m) not in norms | cores | acts]
			if other:
				raise _lib.ElfStageError(f"{self}: remat_strategy selects {other[:4]}; this executor can checkpoint the stage root, the attention cores and the norm modules")
		self._remat_cache[key] = (strategy, flags)
		return flags

	# ------------------------------------------------------------------ compute ops
	def forward(self, mb_id, **options):
		"""F.  Options: ``remat_strategy`` (see ``_remat_flags``) and ``activation_offload`` (handled by
		the offloader the engine wraps around this call)."""
		var = self.input_variables[0]
		x = var.wait_and_pop(mb_id)
		self._set_samples(mb_id, x, self.seq if self.vocab_in else self.seq * self.d)
		x = self._check_ids(x, mb_id) if self.vocab_in else self._check_io(x, "stage input", mb_id)
		flags = self._remat_flags(options.get(OpOptions.REMAT_STRATEGY))
		ybuf, y = self._new_output(x, mb_id)
		with self._timed(f"forward({self.id}:{mb_id})"):
			_lib.check(self.lib.elf_stage_forward(self._handle, mb_id, x.data_ptr(), ybuf.data_ptr(), flags, _stream()), "elf_stage_forward")
		self._kept.setdefault(mb_id, {})["x"] = x
		for dst in self.output_variables[0]:
			dst.set(dst.to_send, mb_id, y)
		var.set(var.saved, mb_id, x)
		out0 = self.output_variables[0][0]
		out0.set(out0.saved, mb_id, y)
		if self.is_last:
			return [out0.get(out0.to_send, mb_id)]

	def backward_inputs(self, mb_id, **options):
		"""B.  Options ``recompute_activations`` / ``recompute_gradients`` drop the W stash halves."""
		var = self.input_variables[0]
		x = var.get(var.saved, mb_id)
		outs = self.output_variables[0]
		outs[0].get(outs[0].saved, mb_id)
		dy = outs[0].wait_and_pop(mb_id)
		for dst in outs[1:]:
			dy = dy + dst.wait_and_pop(mb_id)
		dy = self._check_dy(dy, mb_id)
		ra = bool(options.get(OpOptions.RECOMPUTE_ACTIVATIONS, False))
		rg = bool(options.get(OpOptions.RECOMPUTE_GRADIENTS, False))
		flags = (BWD_RECOMPUTE_ACTIVATIONS if ra else 0) | (BWD_RECOMPUTE_GRADIENTS if rg else 0)
		dx = None if self.vocab_in else torch.empty_like(x)  # token ids have no gradient
		with self._timed(f"backward_inputs({self.id}:{mb_id})"):
			_lib.check(self.lib.elf_stage_backward_inputs(self._handle, mb_id, x.data_ptr(), dy.data_ptr(), dx.data_ptr() if dx is not None else None, flags, _stream()), "elf_stage_backward_inputs")
		kept = self._kept.setdefault(mb_id, {})
		kept["dy"] = dy  # the last block's dY of the W stash is this tensor
		if not ra:
			kept.pop("x", None)
		if dx is not None:
			var.set(var.to_send, mb_id, dx)
		if ra:
			var.set(var.saved, mb_id, x)
		if rg:
			outs[0].set(outs[0].to_process, mb_id, dy)

	folds_grad_scale = True  # Engine may pass ``final_scale`` to the step's last backward_params

	def backward_params(self, mb_id, **options):
		"""W: fp32 dW += dY^T X for every linear layer of the stage.  ``final_scale`` (set by the Engine on the step's
		last W when a gradient scale follows it): the linear layers' accumulators leave this pass multiplied by it,
		with their bf16 copies written; ``scale_grads`` then only has the small rest to do."""
		scale = options.get("final_scale")
		with self._timed(f"backward_params({self.id}:{mb_id})"):
			if scale:
				_lib.check(self.lib.elf_stage_backward_params_scaled(self._handle, mb_id, float(scale), _stream()), "elf_stage_backward_params_scaled")
				self._folded_scale = ctypes.c_float(float(scale)).value  # as the library received it
			else:
				_lib.check(self.lib.elf_stage_backward_params(self._handle, mb_id, _stream()), "elf_stage_backward_params")
		self._kept.pop(mb_id, None)

	def recompute_forward(self, mb_id, **options):
		var = self.input_variables[0]
		x = var.get(var.saved, mb_id)
		save = bool(options.get(OpOptions.SAVE, False))
		with self._timed(f"recompute_forward({self.id}:{mb_id})"):
			_lib.check(self.lib.elf_stage_recompute_forward(self._handle, mb_id, x.data_ptr(), int(save), _stream()), "elf_stage_recompute_forward")
		if save:
			var.set(var.saved, mb_id, x)
			out0 = self.output_variables[0][0]
			out0.set(out0.saved, mb_id, x)  # placeholder: the graph lives inside the library

	def recompute_backward_inputs(self, mb_id, **options):
		var = self.input_variables[0]
		var.get(var.saved, mb_id)
		out0 = self.output_variables[0][0]
		out0.get(out0.saved, mb_id)
		dy = out0.get(out0.to_process, mb_id)
		with self._timed(f"recompute_backward_inputs({self.id}:{mb_id})"):
			_lib.check(self.lib.elf_stage_recompute_backward_inputs(self._handle, mb_id, dy.data_ptr(), _stream()), "elf_stage_recompute_backward_inputs")
		self._kept.setdefault(mb_id, {})["dy"] = dy

	# ------------------------------------------------------------------ gradients
	def scale_grads(self, batch_size):
		"""main_grad /= batch_size, and param.grad = bf16(main_grad) (block.py:518-527)."""
		inv = 1.0 / float(batch_size)
		done = ()
		if self._folded_scale is not None:
			# the step's last W has scaled the linear layers already (and written their bf16 copies)
			if self._folded_scale != ctypes.c_float(inv).value:
				raise _lib.ElfStageError(f"{self}: the last W folded a gradient scale of {self._folded_scale}, scale_grads is asked for {inv}")
			done = self._w_scaled
			self._folded_scale = None
		for i, (w, g) in enumerate(zip(self._fused_w, self._fused_g)):
			if i in done:
				continue
			if self._fused_bf16_grad[i] is None:
				self._fused_bf16_grad[i] = torch.empty_like(w)
			_lib.check(self.lib.elf_scale_grads(g.data_ptr(), self._fused_bf16_grad[i].data_ptr(), g.numel(), inv, _stream()), "elf_scale_grads")
		for p, (i, r, n) in self._param_loc.items():
			p.grad = self._fused_bf16_grad[i][r : r + n]

	def zero_grad(self):
		self._folded_scale = None
		for g in self._fused_g:
			g.zero_()
		for p in self.main_grads:
			p.grad = None

	def _grad_buffers(self):
		return self._fused_g

	def _sends_input_grads(self):
		return not self.vocab_in  # token ids have no gradient to send

	# ------------------------------------------------------------------ offload hooks used by StageOffloader
	def offload(self, mb_id):
		_lib.check(self.lib.elf_stage_offload(self._handle, mb_id, _stream()), "elf_stage_offload")

	def prefetch(self, mb_id):
		_lib.check(self.lib.elf_stage_prefetch(self._handle, mb_id, _stream()), "elf_stage_prefetch")

	def release(self, mb_id):
		_lib.check(self.lib.elf_stage_release(self._handle, mb_id), "elf_stage_release")

	def reserve_pinned(self, nbytes):
		"""Grow the pinned-host arena of activation offload by ``nbytes`` ahead of the first step."""
		_lib.check(self.lib.elf_stage_reserve_pinned(self._handle, int(nbytes)), "elf_stage_reserve_pinned")

	def clear(self):
		"""Drop every micro-batch state held by the library and the tensors pinned for it."""
		_lib.check(self.lib.elf_stage_clear(self._handle), "elf_stage_clear")
		self._kept.clear()
		self._samples.clear()

	def end_step(self):
		"""After a step whose every micro-batch went through W the library holds nothing: only the
		references kept for it are dropped, without the device synchronisation of ``clear``.  A step
		that left state behind (a forward-only schedule) is cleared in full."""
		if self.mem_stats()["live_bytes"] == 0 and not any("x" in k for k in self._kept.values()):
			self._kept.clear()
		else:
			self.clear()

	def mem_stats(self):
		st = MemStats()
		_lib.check(self.lib.elf_stage_mem_stats(self._handle, ctypes.byref(st)), "elf_stage_mem_stats")
		return {n: getattr(st, n) for n, _ in MemStats._fields_}

	def reset_peak(self):
		_lib.check(self.lib.elf_stage_reset_peak(self._handle), "elf_stage_reset_peak")
