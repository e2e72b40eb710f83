"""``elf``: the reference package name (elf/__init__.py:1-13 of topal-team/elf exports ``Pipeline``,
``PipelineConfig`` and the registries), provided by this build so that ``from elf import Pipeline``
keeps working.  Everything lives in ``elf_amd``; the sub-module names of the reference that this path
covers (``elf.scheduling``, ``elf.execution``, ``elf.registry``, ``elf.utils``, ``elf.partitioners``,
``elf.pipeline``, ``elf.zb_utils``) resolve to the ``elf_amd`` modules of the same names."""

import importlib
import sys

import elf_amd
from elf_amd import *  # noqa: F401,F403
from elf_amd import __all__ as _names

__all__ = list(_names)

for _sub in ("scheduling", "execution", "registry", "utils", "partitioners", "pipeline", "zb_utils", "benchmark_utils", "models", "losses"):
	_mod = importlib.import_module(f"elf_amd.{_sub}")
	sys.modules[f"elf.{_sub}"] = _mod
	globals()[_sub] = _mod

from elf_amd.zb_utils import replace_layer_with_layer_dw, replace_linear_with_linear_dw  # noqa: E402,F401

__all__ += ["replace_layer_with_layer_dw", "replace_linear_with_linear_dw"]
