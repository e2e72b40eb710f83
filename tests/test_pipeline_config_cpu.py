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
