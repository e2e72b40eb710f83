"""ctypes binding of libelf_stage.so (the C ABI declared in include/elf_stage.h).

The library is built in-tree by ``__graft_entry__.build()`` (or ``make -C elf_amd/csrc``).
There is no fallback: if the shared object is missing, loading raises.
"""

import ctypes
import os
from ctypes import c_int, c_int64, c_float, c_double, c_void_p, c_char_p, POINTER

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libelf_stage.so")

_lib = None

# name -> (restype, argtypes); kept in one table so that tests can check the exported symbols
# against the header.
_P = c_void_p
_SIGNATURES = {
	"elf_last_error": (c_char_p, []),
	"elf_abi_version": (c_int, []),
	"elf_gemm_bf16": (c_int, [c_int, c_int, c_int, c_int, c_int, _P, c_int64, _P, c_int64, _P, c_int64, c_int, _P, c_int64, c_int, c_int, _P]),
	"elf_norm_fwd": (c_int, [c_int, _P, _P, _P, _P, _P, c_int, c_int, c_float, _P]),
	"elf_norm_bwd_workspace_floats": (c_int64, [c_int, c_int]),
	"elf_norm_bwd": (c_int, [c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, _P]),
	"elf_gemm_rope_bf16": (c_int, [c_int, c_int, c_int, _P, c_int64, _P, c_int64, _P, c_int64, _P, c_int, c_int, c_int, _P]),
	"elf_colsum_workspace_floats": (c_int64, [c_int64, c_int]),
	"elf_colsum_bf16": (c_int, [_P, c_int64, _P, c_int64, c_int, _P, _P]),
	"elf_norm_bwd_noalloc": (c_int, [c_int, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, _P]),
	"elf_gelu_fwd": (c_int, [_P, _P, c_int64, _P]),
	"elf_gelu_bwd": (c_int, [_P, _P, _P, c_int64, _P]),
	"elf_gemm_act_bf16": (c_int, [c_int, c_int, c_int, c_int, _P, c_int64, _P, c_int64, _P, c_int64, _P, c_int64, _P]),
	"elf_gemm_swiglu_bwd_bf16": (c_int, [c_int, c_int, c_int, _P, c_int64, _P, c_int64, _P, c_int64, _P, c_int64, _P, _P]),
	"elf_swiglu_fwd": (c_int, [_P, _P, c_int64, c_int, _P]),
	"elf_swiglu_bwd": (c_int, [_P, _P, _P, c_int64, c_int, _P]),
	"elf_rope_table": (c_int, [_P, c_int, c_int, c_double, _P]),
	"elf_rope_apply": (c_int, [_P, _P, c_int64, c_int, c_int, c_int, c_int, c_int, _P]),
	"elf_scale_grads": (c_int, [_P, _P, c_int64, c_float, _P]),
	"elf_add_bf16": (c_int, [_P, _P, _P, c_int64, _P]),
	"elf_embedding_fwd": (c_int, [_P, _P, _P, c_int64, c_int, c_int, _P]),
	"elf_embedding_bwd": (c_int, [_P, _P, _P, c_int64, c_int, c_int, _P]),
	"elf_cross_entropy": (c_int, [_P, c_int64, _P, c_int64, c_int64, c_int64, c_float, _P, _P, _P, c_int64, _P]),
	"elf_cross_entropy_reduce": (c_int, [_P, _P, c_int64, c_int64, _P, _P]),
	"elf_attn_fwd": (c_int, [_P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_float, _P]),
	"elf_attn_bwd_workspace_bytes": (c_int64, [c_int, c_int, c_int, c_int, c_int]),
	"elf_gemm_turn_giveups": (c_int, [POINTER(ctypes.c_uint64)]),
	"elf_gemm_dw_group": (c_int, [c_int, _P, c_int, c_float, _P]),
	"elf_hbm_probe": (c_int, [c_int, _P, _P, c_int64, _P]),
	"elf_prof_enable": (None, [c_int]),
	"elf_prof_collect": (c_int, [c_int, POINTER(c_double), POINTER(c_double)]),
	"elf_prof_launches": (c_int64, [c_int, POINTER(c_double)]),
	"elf_attn_bwd": (c_int, [_P] * 10 + [c_int64] * 8 + [c_int] * 6 + [c_float, _P]),
	"elf_attn_bwd_rope": (c_int, [_P] * 10 + [c_int64] * 8 + [c_int] * 6 + [c_float, _P, _P]),
}


class ElfStageError(RuntimeError):
	"""A C-ABI call returned a negative status."""


def exported_symbols():
	return sorted(_SIGNATURES)


def register(name, restype, argtypes):
	"""Add a signature (used by modules that bind further entry points)."""
	_SIGNATURES[name] = (restype, argtypes)
	if _lib is not None:
		fn = getattr(_lib, name)
		fn.restype, fn.argtypes = restype, argtypes


def load():
	"""Load the shared object (once) and type every entry point. Raises if it is not built."""
	global _lib
	if _lib is not None:
		return _lib
	if not os.path.exists(LIB_PATH):
		raise ElfStageError(
			f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
			"or `make -C elf_amd/csrc`. There is no non-HIP fallback."
		)
	lib = ctypes.CDLL(LIB_PATH)
	for name, (restype, argtypes) in _SIGNATURES.items():
		fn = getattr(lib, name)
		fn.restype, fn.argtypes = restype, argtypes
	_lib = lib
	return lib


def check(rc, what=""):
	if rc != 0:
		msg = load().elf_last_error().decode()
		raise ElfStageError(f"{what} failed (rc={rc}): {msg}")
