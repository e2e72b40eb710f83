"""elf_amd: MI355X-native execution path of one ELF pipeline stage (see include/elf_stage.h).

Top-level names follow the reference package (elf/__init__.py): ``Pipeline``, ``PipelineConfig``,
``Placement``, ``sequential_signatures``.  They are resolved on first use, so that importing the
package (e.g. for the schedulers alone) does not load the HIP library.
"""

__all__ = ["Pipeline", "PipelineConfig", "Placement", "sequential_signatures"]


def __getattr__(name):
	if name in ("Pipeline", "PipelineConfig"):
		from . import pipeline

		return getattr(pipeline, name)
	if name == "Placement":
		from .utils import Placement

		return Placement
	if name == "sequential_signatures":
		from .partitioners.utils import sequential_signatures

		return sequential_signatures
	raise AttributeError(f"module 'elf_amd' has no attribute {name!r}")
