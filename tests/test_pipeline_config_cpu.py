"""``PipelineConfig`` against the values the reference's own tests hold
(tests/unit/test_pipeline_config.py:7-59: defaults, explicit fields, ``to_kwargs``, partial overrides)."""

import dataclasses

import pytest

from elf_amd.pipeline import PipelineConfig

REFERENCE_DEFAULTS = {"tracer": "default", "partitioner": "constrained", "scheduler": "auto", "placement": "auto", "pp": None, "dp": 1, "worker": 0}


def test_defaults_are_the_reference_defaults():
	cfg = PipelineConfig()
	for name, want in REFERENCE_DEFAULTS.items():
		assert getattr(cfg, name) == want, name


def test_every_field_can_be_set():
	given = {"tracer": "fx", "partitioner": "metis", "scheduler": "afab", "placement": "manual", "pp": 4, "dp": 2, "worker": 1}
	cfg = PipelineConfig(**given)
	assert {k: getattr(cfg, k) for k in given} == given


def test_to_kwargs_lists_every_field():
	kwargs = PipelineConfig(pp=4, dp=2).to_kwargs()
	assert set(REFERENCE_DEFAULTS) <= set(kwargs)
	assert kwargs["pp"] == 4 and kwargs["dp"] == 2 and kwargs["tracer"] == "default"
	# fields left at None are dropped (elf/pipeline.py:92-94)
	cfg = PipelineConfig(pp=4, dp=2)
	assert set(kwargs) == {f.name for f in dataclasses.fields(PipelineConfig) if getattr(cfg, f.name) is not None}
	assert "pp" not in PipelineConfig().to_kwargs()


@pytest.mark.parametrize("override", [{"scheduler": "zbh2", "dp": 4}, {"memory_budget": 48000.0}, {"partitioner": False}])
def test_partial_overrides_keep_the_other_defaults(override):
	cfg = PipelineConfig(**override)
	for name, want in {**REFERENCE_DEFAULTS, **override}.items():
		assert getattr(cfg, name) == want, name


def test_reference_package_name_resolves_to_this_build():
	"""``from elf import Pipeline`` (the reference's top-level names, elf/__init__.py:1-13) and its
	sub-module paths reach the elf_amd modules, not copies of them."""
	import elf
	import elf.scheduling
	import elf_amd.scheduling
	from elf import Pipeline, PipelineConfig, Placement, replace_layer_with_layer_dw, sequential_signatures
	from elf.registry import SCHEDULERS
	from elf.zb_utils import LinearDW

	import elf_amd.pipeline
	import elf_amd.registry
	import elf_amd.zb_utils

	assert Pipeline is elf_amd.pipeline.Pipeline and PipelineConfig is elf_amd.pipeline.PipelineConfig
	assert elf.scheduling is elf_amd.scheduling and SCHEDULERS is elf_amd.registry.SCHEDULERS and LinearDW is elf_amd.zb_utils.LinearDW
	assert Placement([0, 1]).get_ids(1) == [1] and len(sequential_signatures([0, 1])) == 2 and callable(replace_layer_with_layer_dw)
	assert set(elf.__all__) >= {"Pipeline", "PipelineConfig", "Placement", "sequential_signatures", "replace_layer_with_layer_dw"}
