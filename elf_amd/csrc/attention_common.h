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
// Backward: one workgroup = 128 keys of one (batch, kv head); each wave owns 32 keys and
// keeps their dK^T / dV^T accumulators in registers while the workgroup walks over the
// query tiles (32 queries at a time) of every query head in the group; dQ is reduced across
// the four waves through an LDS copy of dS and added to an fp32 buffer with atomics.
#pragma once
#include "common.h"
#include "kernels.h"
#include "lds_dma.h"

namespace elf {

namespace attn {

constexpr float LOG2E = 1.4426950408889634f;

template <int D>
struct AttnSmem {
	static constexpr int LDR = D + 8;   // row stride (elements) of tiles read along d
	static constexpr int LDT = D + 16;  // row stride of tiles read with the transpose read
};

// Cooperative copy of a ROWS x D bf16 tile (global row stride ld) into LDS with row stride LDS_LD.
template <int ROWS, int D, int LDS_LD, int NT>
__device__ __forceinline__ void copy_tile_g2r(const bf16_t* __restrict__ g, int64_t ld, int tid, u32x4 (&regs)[ROWS * D / 8 / NT]) {
	constexpr int CPR = D / 8;
	constexpr int RPP = NT / CPR;
	const int c = tid % CPR, r = tid / CPR;
#pragma unroll
	for (int i = 0; i < ROWS * D / 8 / NT; i++)
		regs[i] = *reinterpret_cast<const u32x4*>(g + (int64_t)(r + i * RPP) * ld + c * 8);
}
template <int ROWS, int D, int LDS_LD, int NT>
__device__ __forceinline__ void copy_tile_r2s(bf16_t* s, int tid, const u32x4 (&regs)[ROWS * D / 8 / NT]) {
	constexpr int CPR = D / 8;
	constexpr int RPP = NT / CPR;
	const int c = tid % CPR, r = tid / CPR;
#pragma unroll
	for (int i = 0; i < ROWS * D / 8 / NT; i++)
		*reinterpret_cast<u32x4*>(s + (r + i * RPP) * LDS_LD + c * 8) = regs[i];
}

// MFMA operand (rows row0..row0+31 of an LDS tile, 8 consecutive columns starting at
// col0 + 8*(lane/32)): plain 16-byte read.
template <int LD>
__device__ __forceinline__ bf16x8 frag_rows(const bf16_t* s, int row0, int col0, int lane) {
	return *reinterpret_cast<const bf16x8*>(s + (row0 + (lane & 31)) * LD + col0 + 8 * (lane >> 5));
}
// MFMA operand for a tile stored [k][m]: lane gets column m0 + lane%32 at the 8 rows
// {kA..kA+3, kB..kB+3} where kA = k0 + 4*(lane/32), kB = kA + 8.  This is the row order in
// which a 32x32 accumulator holds its rows (register r <-> row (r/4)*8 + 4*(lane/32) + r%4), so
// an accumulator tile converted to bf16 is directly the matching B operand.
template <int LD>
__device__ __forceinline__ bf16x8 frag_cols_acc_order(const bf16_t* s, int k0, int m0, int lane) {
	const int j = lane & 15;
	const bf16_t* p0 = s + (k0 + 4 * (lane >> 5) + (j >> 2)) * LD + m0 + 16 * ((lane & 31) >> 4) + 4 * (j & 3);
	s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p0));
	s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p0 + 8 * LD));
	return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}
// Same, but with the natural k order {k0 + 8*(lane/32) .. +7}.
template <int LD>
__device__ __forceinline__ bf16x8 frag_cols(const bf16_t* s, int k0, int m0, int lane) {
	const int j = lane & 15;
	const bf16_t* p0 = s + (k0 + 8 * (lane >> 5) + (j >> 2)) * LD + m0 + 16 * ((lane & 31) >> 4) + 4 * (j & 3);
	s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p0));
	s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p0 + 4 * LD));
	return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

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
