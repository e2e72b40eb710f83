"""The boundary-tensor header (reference elf/utils.py:150-220): known headers, round trips, and the
reference's quirks (a zero ends the shape; 15 dimensions at most)."""

import pytest
import torch

from elf_amd.utils import WIRE_DTYPES, TensorMetadata


def test_dtype_codes_follow_the_reference_table():
	# elf/utils.py:19-31: fp16, bf16, fp32, fp64, int16, int32, int64, complex32/64/128, bool
	assert WIRE_DTYPES.index(torch.float16) == 0
	assert WIRE_DTYPES.index(torch.bfloat16) == 1
	assert WIRE_DTYPES.index(torch.float32) == 2
	assert WIRE_DTYPES.index(torch.int64) == 6
	assert WIRE_DTYPES.index(torch.bool) == 10
	assert len(WIRE_DTYPES) == 11


def test_known_header_of_a_stage_boundary():
	# one sample of a Llama-3-8B boundary: [seq 4096, d_model 4096] bf16
	sample = torch.empty(2, 4096, 4096, dtype=torch.bfloat16, device="meta")[0]
	h = TensorMetadata(sample).to_tensor().cpu()
	assert h.dtype == torch.float32 and h.shape == (TensorMetadata.MAX_SIZE,)
	assert h.tolist() == [1.0, 4096.0, 4096.0] + [0.0] * 13


@pytest.mark.filterwarnings("ignore:ComplexHalf")
@pytest.mark.parametrize("dtype", WIRE_DTYPES)
@pytest.mark.parametrize("shape", [(), (7,), (128, 768), (3, 5, 2, 9), (2, 1) * 7 + (3,)])  # the last one: 15 dimensions
def test_round_trip(dtype, shape):
	meta = TensorMetadata(torch.empty(shape, dtype=dtype, device="meta"))
	back = TensorMetadata.from_tensor(meta.to_tensor().cpu())
	assert back.dtype == dtype and back.shape == list(shape)
	buf = back.get_buffer(4)
	assert buf.shape == (4, *shape) and buf.dtype == dtype


def test_token_ids_header():
	# first stage input: int64 ids, one sample = [seq]
	meta = TensorMetadata.from_tensor(torch.tensor([6.0, 1024.0] + [0.0] * 14))
	assert meta.dtype == torch.int64 and meta.shape == [1024]
	assert meta.get_buffer(8).shape == (8, 1024)


def test_a_zero_extent_ends_the_shape():
	meta = TensorMetadata(torch.empty(4, 0, 3, device="meta"))
	assert TensorMetadata.from_tensor(meta.to_tensor().cpu()).shape == [4]


def test_too_many_dimensions():
	with pytest.raises(IndexError):
		TensorMetadata(torch.empty((1,) * 16, device="meta")).to_tensor()
	with pytest.raises(AssertionError):
		TensorMetadata.from_tensor(torch.zeros(2, 16))
