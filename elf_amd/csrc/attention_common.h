// Flash-style attention forward / backward on bf16 MFMA for gfx950, for the packed
// projection layout a stage keeps in HBM:  q/k/v are column slices of one [T, ld] buffer
// (T = batch * S tokens; head h of q occupies columns [h*D, (h+1)*D)), so no head transpose
// ever goes through memory.  Supports grouped-query attention (Hq a multiple of Hkv) and an
// optional causal mask.  Softmax statistics are fp32; probabilities are rounded to bf16 only
// as MFMA operands.
//
// Replaces F.scaled_dot_product_attention / softmax(QK^T * scale) V and its autograd backward
// in the reference model zoo (benchmarks/models/simple.py:362-367, 379-386, 412-434).
//
// Forward: one workgroup = 128 queries of one (batch, head); each of its 4 waves owns 32
// queries and computes S^T = K Q^T so that a query is a column of the MFMA accumulator: the
// running max / sum of a query then live in one lane pair, and P^T is already laid out as
// the B operand of O^T = V^T P^T.  K and V tiles (64 keys) are staged in LDS, V is read with
// the LDS transpose read.
//
// Backward: one workgroup pass = 128 keys of one (batch, kv head); each wave owns 32 keys and
// keeps their dK^T / dV^T accumulators in registers while the workgroup walks over the
// query tiles (32 queries at a time) of every query head in the group; dS^T goes through LDS,
// each wave multiplies it with its slice of K one tile later and stores its part of the key
// tile's partial dQ; a second kernel adds the partials of all key tiles in a fixed order.
#pragma once
#include "common.h"
#include "kernels.h"
#include "lds_dma.h"

namespace elf {

namespace attn {

constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ bf16x8 pack8(const float* v) {
	bf16x8 r;
#pragma unroll
	for (int i = 0; i < 8; i++) r[i] = (bf16_t)v[i];
	return r;
}

struct AttnArgs {
	const bf16_t* q;
	const bf16_t* k;
	const bf16_t* v;
	bf16_t* o;
	float* lse;  // [B, Hq, S], natural-log units
	int64_t ldq, ldk, ldv, ldo;
	int B, S, Hq, Hkv;
	float scale;
};

}  // namespace attn
}  // namespace elf
