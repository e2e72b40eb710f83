// Attention backward kernels (see attention_common.h for the layout conventions).
#include "attention_common.h"
#include <type_traits>

namespace elf {
namespace attn {

// ------------------------------------------------------------------------------------------
// delta[b,h,s] = sum_d dO * O and nlse2[b,h,s] = -lse * log2(e).  D/8 lanes share one (token, head)
// row, 16 bytes each, so a wave covers 4 (D = 128) or 8 (D = 64) rows per step.
__global__ __launch_bounds__(256) void attn_delta_kernel(const bf16_t* __restrict__ dO, const bf16_t* __restrict__ O,
                                                         const float* __restrict__ lse, float* __restrict__ delta,
                                                         float* __restrict__ nlse2, int64_t ldd, int64_t ldo, int B, int S,
                                                         int Hq, int D) {
	const int lpr = D / 8;  // lanes per row: 8 or 16
	const int rows_per_block = 256 / lpr;
	const int sub = threadIdx.x % lpr;
	const int64_t n = (int64_t)B * S * Hq;
	for (int64_t idx = (int64_t)blockIdx.x * rows_per_block + threadIdx.x / lpr; idx < n; idx += (int64_t)gridDim.x * rows_per_block) {
		const int h = (int)(idx % Hq);
		const int64_t tok = idx / Hq;
		const bf16x8 x = *reinterpret_cast<const bf16x8*>(dO + tok * ldd + h * D + sub * 8);
		const bf16x8 y = *reinterpret_cast<const bf16x8*>(O + tok * ldo + h * D + sub * 8);
		float s = 0.f;
#pragma unroll
		for (int j = 0; j < 8; j++) s += (float)x[j] * (float)y[j];
		for (int o = lpr >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
		if (sub == 0) {
			const int64_t b = tok / S, sp = tok % S;
			delta[(b * Hq + h) * S + sp] = s;
			nlse2[(b * Hq + h) * S + sp] = -lse[(b * Hq + h) * S + sp] * LOG2E;
		}
	}
}

struct AttnBwdArgs {
	const bf16_t* q;
	const bf16_t* k;
	const bf16_t* v;
	const bf16_t* dO;
	const float* nlse2;  // -lse * log2(e)
	const float* delta;
	bf16_t* dq_part;  // per key tile partial dQ, see part_row0()
	bf16_t* dk;
	bf16_t* dv;
	int64_t ldq, ldk, ldv, lddo, lddk, lddv;
	int B, S, Hq, Hkv;
	float scale;
	// non-null: the q and k heads carry a rotary embedding whose backward (the inverse rotation) is applied to
	// dQ and dK before they are stored; (cos, sin) table [S, D / 2] of rope_table()
	const float2* rope_cs;
};

// dQ partials.  Every 128-key tile contributes a [queries, Hq*D] partial dQ; the partials are written
// with plain stores, each by exactly one workgroup, rounded to bf16 (like the P and dS operands of the
// products they come from), and summed in fp32 in a fixed order by dq_reduce_kernel: no atomics, no
// zero fill, and a result that does not depend on the order in which workgroups run.  (Adding the
// tiles into one fp32 buffer with atomics costs a read-modify-write of a line that is never cache
// resident per 32 lanes: 0.3 T lanes/s chip-wide, 0.68 of 1.81 ms at the Llama-3-8B shape.)
// Layout per batch element: the slices of the key tiles one after the other; with a causal mask
// slice kt only holds the queries q >= 128 kt, so it starts at row kt S - 128 kt (kt - 1) / 2 and
// its row index is q - 128 kt.
__host__ __device__ __forceinline__ int64_t part_row0(int kt, int S, bool causal) {
	return causal ? (int64_t)kt * S - 64 * (int64_t)kt * (kt - 1) : (int64_t)kt * S;
}
__host__ __device__ __forceinline__ int64_t part_rows(int S, bool causal) { return part_row0(S / 128, S, causal); }

// Tiles fetched straight into LDS (lds_dma.h) are unpadded; the 16-byte chunk index of a row is
// XOR-swizzled with a function of the row chosen so that both access patterns are conflict
// free: row-wise fragment reads (16 consecutive rows, same chunk) and transpose reads (a
// half-wave takes 64 contiguous bytes from each of 4 consecutive rows).
template <int D>
struct BwdTile {
	static constexpr int ROW_BYTES = D * 2;
	static constexpr int CPR = D / 8;             // 16-byte chunks per row
	static constexpr int RPI = 1024 / ROW_BYTES;  // rows per DMA wave instruction
	__device__ static __forceinline__ int swz(int row) {
		// D = 128 (16 chunks per row, a row spans all banks): bits [3:2] from row % 4 put four consecutive
		// rows into four different 64-byte bank groups, bits [1:0] from row / 4 make 16 consecutive rows
		// distinct.  D = 64 (8 chunks, two rows span all banks): the same for row pairs, bit-reversed.
		return D == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | (((row >> 2) & 1) << 1) | ((row >> 3) & 1));
	}
	// row-wise operand: rows row0 + lane%32, 8 consecutive columns from 16*ks + 8*(lane/32)
	__device__ static __forceinline__ bf16x8 rows(const unsigned char* t, int row0, int ks, int lane) {
		const int r = row0 + (lane & 31);
		return *reinterpret_cast<const bf16x8*>(t + r * ROW_BYTES + (((2 * ks + (lane >> 5)) ^ swz(r)) << 4));
	}
	// transposed operand: column m0 + lane%32 at the rows {kA..kA+3, kA+second..+3}, kA = k0 + 4*(lane/32)
	// (second = 8: accumulator row order) or kA = k0 + 8*(lane/32) (second = 4: natural order)
	template <bool ACC_ORDER>
	__device__ static __forceinline__ bf16x8 cols(const unsigned char* t, int k0, int m0, int lane) {
		const int j = lane & 15;
		const int kk = k0 + (ACC_ORDER ? 4 : 8) * (lane >> 5) + (j >> 2);
		const int k2 = kk + (ACC_ORDER ? 8 : 4);
		const int c = (m0 + 16 * ((lane & 31) >> 4) + 4 * (j & 3)) >> 3;
		const unsigned char* p0 = t + kk * ROW_BYTES + ((c ^ swz(kk)) << 4) + (j & 1) * 8;
		const unsigned char* p1 = t + k2 * ROW_BYTES + ((c ^ swz(k2)) << 4) + (j & 1) * 8;
		s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p0));
		s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p1));
		return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
	}
};

// 4 bytes per lane from a per-lane global address to LDS at lds_byte_addr + lane * 4.
__device__ __forceinline__ void dma4(const void* lane_addr, uint32_t lds_byte_addr) {
	asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_byte_addr), "v"(lane_addr) : "memory", "m0");
}

// dS^T tile in LDS: [key][q] bf16 with 64-byte rows (32 queries); the 16-byte chunk index is
// XOR-swizzled with (key >> 2) & 3 so that the 8-byte accumulator writes of 32 consecutive keys
// and the transpose reads of 4 consecutive keys both spread over all banks.
__device__ __forceinline__ int ds_t_offset(int key, int q) {  // q a multiple of 4
	return key * 64 + (((q >> 3) ^ ((key >> 2) & 3)) << 4) + ((q >> 2) & 1) * 8;
}
// A operand from the dS^T tile: row q = lane%32, keys k0 + 8*(lane/32) .. +7
__device__ __forceinline__ bf16x8 ds_t_frag(const unsigned char* t, int k0, int lane) {
	const int j = lane & 15;
	const int kk = k0 + 8 * (lane >> 5) + (j >> 2);
	const int q = 16 * ((lane & 31) >> 4) + 4 * (j & 3);
	s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(t + ds_t_offset(kk, q)));
	s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(t + ds_t_offset(kk + 4, q)));
	return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// dK^T / dV^T accumulators of one wave -> memory: register r of tile dt <-> d = dt*32 + (r/4)*8 + 4g + r%4, lane <-> key.
// With a rotary embedding on the k heads, dK (scaled and rounded to bf16, as a separate RoPE pass over the stored
// gradient would read it) is rotated back first; the partner of column d is d + D/2, same register of tile dt + DT/2.
template <int D>
__device__ __forceinline__ void store_dk_dv(const f32x16 (&acc_dk)[D / 32], const f32x16 (&acc_dv)[D / 32], bf16_t* dkp, bf16_t* dvp, float scale, int g,
                                            const float2* cs_row) {
	constexpr int DT = D / 32;
#pragma unroll
	for (int dt = 0; dt < DT; dt++) {
#pragma unroll
		for (int r4 = 0; r4 < 4; r4++) {
			bf16x4 v4;
#pragma unroll
			for (int u = 0; u < 4; u++) v4[u] = (bf16_t)acc_dv[dt][r4 * 4 + u];
			*reinterpret_cast<bf16x4*>(dvp + dt * 32 + r4 * 8 + 4 * g) = v4;
		}
	}
	if (cs_row == nullptr) {
#pragma unroll
		for (int dt = 0; dt < DT; dt++) {
#pragma unroll
			for (int r4 = 0; r4 < 4; r4++) {
				bf16x4 k4;
#pragma unroll
				for (int u = 0; u < 4; u++) k4[u] = (bf16_t)(acc_dk[dt][r4 * 4 + u] * scale);
				*reinterpret_cast<bf16x4*>(dkp + dt * 32 + r4 * 8 + 4 * g) = k4;
			}
		}
		return;
	}
#pragma unroll
	for (int dt = 0; dt < DT / 2; dt++) {
#pragma unroll
		for (int r4 = 0; r4 < 4; r4++) {
			const int i = dt * 32 + r4 * 8 + 4 * g;
			const f32x4 t0 = *reinterpret_cast<const f32x4*>(cs_row + i), t1 = *reinterpret_cast<const f32x4*>(cs_row + i + 2);
			bf16x4 lo4, hi4;
#pragma unroll
			for (int u = 0; u < 4; u++) {
				const float lo = (float)(bf16_t)(acc_dk[dt][r4 * 4 + u] * scale), hi = (float)(bf16_t)(acc_dk[dt + DT / 2][r4 * 4 + u] * scale);
				const float c = (u < 2 ? t0 : t1)[(u & 1) * 2], sn = (u < 2 ? t0 : t1)[(u & 1) * 2 + 1];
				float rl, rh;
				rope_rot(lo, hi, c, -sn, rl, rh);
				lo4[u] = (bf16_t)rl;
				hi4[u] = (bf16_t)rh;
			}
			*reinterpret_cast<bf16x4*>(dkp + i) = lo4;
			*reinterpret_cast<bf16x4*>(dkp + i + D / 2) = hi4;
		}
	}
}

// One workgroup pass = 128 keys of one (batch, kv head); wave w owns keys [32w, 32w+32) and
// keeps their K / V rows (MFMA B operands) and dK^T / dV^T accumulators in registers while the
// workgroup walks over the 32-query tiles of every query head of the group.  Q and dO tiles
// arrive by direct-to-LDS loads one tile ahead.  Per tile and wave:
//   S = Q K^T, dP = dO V^T  (A operands: LDS rows)      P = exp2(S*sc - lse), dS = P (dP - delta)
//   dV^T += dO^T P, dK^T += Q^T dS  (A operands: LDS transpose reads; B: P / dS from registers)
// dS^T goes to LDS; after the next workgroup barrier each wave multiplies the whole 32x128 dS
// by its slice of K (held in registers as B operands) to get its slice of the dQ tile.  That
// product runs one tile behind, so a tile costs one barrier; the slice goes to this key tile's
// partial dQ buffer (bf16).  The softmax scale of dK and dQ is applied by the epilogue / the
// reduction kernel.  With a causal mask key tile kt meets 1 - kt/nkt of the query tiles, so
// a workgroup takes the tiles kt and nkt-1-kt one after the other: every workgroup then does
// the same amount of work.
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256, D == 64 ? 2 : 1) void attn_bwd_kernel(AttnBwdArgs a) {
	using TL = BwdTile<D>;
	constexpr int BKV = 128, BQ = 32;
	constexpr int NF = D / 16;  // fragments per operand tile
	constexpr int DT = D / 32;
	constexpr int NQ = BKV / 16;  // fragments of the dQ product (all 128 keys); waves 0..DT-1 own one 32-column slice each
	constexpr int K_BYTES = BKV * TL::ROW_BYTES, Q_BYTES = BQ * TL::ROW_BYTES;
	constexpr int STAGE = 2 * Q_BYTES + 256;  // Q tile, dO tile, 32 nlse2 + 32 delta floats
	constexpr int DS_BYTES = BKV * BQ * 2;
	constexpr int Q_LOADS = 8 / TL::RPI;  // DMA instructions per wave and tile (8 rows per wave)
	extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
	unsigned char* const sKt = smem_raw;            // K tile, [key][d]
	unsigned char* const sStage = sKt + K_BYTES;    // 2 x {Q [q][d], dO [q][d], nlse2, delta}
	unsigned char* const sdS = sStage + 2 * STAGE;  // 2 x dS^T [key][q]

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int g = lane >> 5, kl = lane & 31;
	const int nkt = a.S / BKV;
	const int npair = CAUSAL ? (nkt + 1) / 2 : nkt;
	int pair = blockIdx.x % npair;
	int bh = blockIdx.x / npair;
	{
		// all key-tile workgroups of a (batch, kv head) group on one XCD (workgroup w runs on XCD w % 8)
		const int ngroups = (int)(gridDim.x / npair);
		if (ngroups % 8 == 0) {
			const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
			bh = xcd + 8 * (slot / npair);
			pair = slot % npair;
		}
	}
	const int hk = bh % a.Hkv, b = bh / a.Hkv;
	const int G = a.Hq / a.Hkv;
	const int64_t tok0 = (int64_t)b * a.S;
	const int64_t HqD = (int64_t)a.Hq * D;
	const float sc = a.scale * LOG2E;
	const bool dq_wave = DT == 4 || wave < DT;  // head_dim 64: two slices, waves 2 and 3 have no dQ share
	const int dq_dt = wave % DT;
	const int key_l = wave * 32 + kl;                        // this lane's key within the tile
	const int nqt_all = a.S / BQ;
	const int dq_lane = kl * (int)HqD + dq_dt * 32 + 4 * g;  // lane part of a dQ tile address (elements): query kl, first of 4 columns

	// DMA plan for one (Q, dO) tile pair: wave w moves rows [w*8, w*8+8) of each
	uint32_t qoff[Q_LOADS], dooff[Q_LOADS];
#pragma unroll
	for (int i = 0; i < Q_LOADS; i++) {
		const int row = wave * 8 + i * TL::RPI + lane / TL::CPR, slot = lane % TL::CPR;
		qoff[i] = (uint32_t)((row * a.ldq + ((slot ^ TL::swz(row)) << 3)) * 2);
		dooff[i] = (uint32_t)((row * a.lddo + ((slot ^ TL::swz(row)) << 3)) * 2);
	}
	auto zero_ds = [&](unsigned char* t) {
#pragma unroll
		for (int i = 0; i < 4; i++) *reinterpret_cast<u32x2*>(t + ds_t_offset(key_l, 8 * i + 4 * g)) = u32x2{0u, 0u};
	};
	// registers [r_lo, r_hi) of a dQ^T accumulator tile -> the partial buffer.  The dQ product is computed
	// transposed (rows d, columns q) so that a lane holds 4 consecutive columns of one query's row:
	// four 8-byte stores per tile and lane (2-byte stores, one per register, cost 500 cycles more per tile)
	auto dq_out = [&](bf16_t* tile, const f32x16& v, int r_lo, int r_hi) {
		if (!dq_wave) return;
#pragma unroll
		for (int j = 0; j < 4; j++)
			if (4 * j >= r_lo && 4 * j < r_hi) {
				bf16x4 o;
#pragma unroll
				for (int t = 0; t < 4; t++) o[t] = (bf16_t)v[4 * j + t];
				*reinterpret_cast<bf16x4*>(tile + dq_lane + 8 * j) = o;
			}
	};

	const int n_pass = (CAUSAL && nkt - 1 - pair != pair) ? 2 : 1;
#pragma unroll 1
	for (int pass = 0; pass < n_pass; pass++) {
		const int kt_idx = pass == 0 ? pair : nkt - 1 - pair;
		const int key0 = kt_idx * BKV;       // first key of the pass
		const int wkey0 = key0 + wave * 32;  // first key of this wave
		if (pass > 0) __syncthreads();       // every wave is done with the LDS of the previous pass

		// K tile -> LDS; this wave moves rows [wave*32, wave*32+32)
		{
			const bf16_t* kb = a.k + (tok0 + key0) * a.ldk + hk * D;
#pragma unroll
			for (int i = 0; i < 32 / TL::RPI; i++) {
				const int row = wave * 32 + i * TL::RPI + lane / TL::CPR, slot = lane % TL::CPR;
				dma16(kb, (uint32_t)((row * a.ldk + ((slot ^ TL::swz(row)) << 3)) * 2),
				      __builtin_amdgcn_readfirstlane(lds_addr(sKt) + (wave * 32 + i * TL::RPI) * TL::ROW_BYTES));
			}
		}
		// own K and V rows as B operands (n = key, 8 consecutive d) in registers
		bf16x8 kf[NF], vf[NF];
		{
			const bf16_t* kp = a.k + (tok0 + wkey0 + kl) * a.ldk + hk * D + 8 * g;
			const bf16_t* vp = a.v + (tok0 + wkey0 + kl) * a.ldv + hk * D + 8 * g;
#pragma unroll
			for (int ks = 0; ks < NF; ks++) {
				kf[ks] = *reinterpret_cast<const bf16x8*>(kp + ks * 16);
				vf[ks] = *reinterpret_cast<const bf16x8*>(vp + ks * 16);
				// the pass-long B operands live in the accumulator half of the register file (the matrix
				// pipe reads them there directly): pinning them at their definition keeps the allocator from
				// copying them into the vector half before every product
				asm volatile("" : "+a"(kf[ks]), "+a"(vf[ks]));
			}
		}
		f32x16 acc_dk[DT], acc_dv[DT];
#pragma unroll
		for (int i = 0; i < DT; i++)
#pragma unroll
			for (int r = 0; r < 16; r++) acc_dk[i][r] = acc_dv[i][r] = 0.f;

		// Walk over (query head in group, query tile); causal: only tiles that reach key0.
		const int qt_first = CAUSAL ? key0 / BQ : 0;
		const int n_iter = G * (nqt_all - qt_first);

		// tile whose loads are issued next: running pointers, recomputed when the walk moves to the next head
		int ld_h = hk * G, ld_qt = qt_first;
		const bf16_t* ld_q;
		const bf16_t* ld_do;
		const float* ld_stat;  // lanes 0..31: nlse2 of the tile's queries, lanes 32..63: delta
		auto seek = [&]() {
			const int64_t row = tok0 + ld_qt * BQ;
			ld_q = a.q + row * a.ldq + ld_h * D;
			ld_do = a.dO + row * a.lddo + ld_h * D;
			ld_stat = (lane < 32 ? a.nlse2 : a.delta) + ((int64_t)b * a.Hq + ld_h) * a.S + ld_qt * BQ + (lane & 31);
		};
		seek();
		const uint32_t lds_stage = lds_addr(sStage) + wave * 8 * TL::ROW_BYTES;
		auto issue = [&](int stage) {
			const uint32_t st = lds_stage + (uint32_t)stage * STAGE;
#pragma unroll
			for (int i = 0; i < Q_LOADS; i++) {
				dma16(ld_q, qoff[i], __builtin_amdgcn_readfirstlane(st + i * TL::RPI * TL::ROW_BYTES));
				dma16(ld_do, dooff[i], __builtin_amdgcn_readfirstlane(st + Q_BYTES + i * TL::RPI * TL::ROW_BYTES));
			}
			if (wave == 0) dma4(ld_stat, __builtin_amdgcn_readfirstlane(st + 2 * Q_BYTES));
			if (++ld_qt == nqt_all) {
				ld_qt = qt_first;
				ld_h++;
				seek();
			} else {
				ld_q += BQ * a.ldq;
				ld_do += BQ * a.lddo;
				ld_stat += BQ;
			}
		};

		issue(0);
		zero_ds(sdS + DS_BYTES);  // the "previous tile" of the first iteration
		wait_vmcnt<0>();
		__syncthreads();
		// this wave's slice of K^T as A operands of the dQ^T product (rows d, k = key)
		bf16x8 ktf[NQ];
#pragma unroll
		for (int i = 0; i < NQ; i++) ktf[i] = TL::template cols<false>(sKt, i * 16, dq_dt * 32, lane);

		// position of the current tile; dq_prev_tile = where the dQ tile of iteration it-1 goes
		int cur_h = hk * G, cur_qt = qt_first;
		// rows of this key tile's slice: first query of the slice = key0 (causal) or 0
		bf16_t* const part = a.dq_part + ((int64_t)b * part_rows(a.S, CAUSAL) + part_row0(kt_idx, a.S, CAUSAL) - qt_first * BQ) * HqD;
		bf16_t* dq_prev_tile = part + (int64_t)(qt_first * BQ) * HqD + cur_h * D;

		for (int it = 0; it < n_iter; it++) {
			if (it + 1 < n_iter) issue((it + 1) & 1);
			const unsigned char* sQ = sStage + (it & 1) * STAGE;
			const unsigned char* sdO = sQ + Q_BYTES;
			const float* sLse = reinterpret_cast<const float*>(sdO + Q_BYTES);
			const unsigned char* sdS_prev = sdS + ((it + 1) & 1) * DS_BYTES;
			unsigned char* sdS_cur = sdS + (it & 1) * DS_BYTES;
			const int q0 = cur_qt * BQ;

			bf16x8 bA[NF], bC[NF];
			f32x16 dq, s, dp;
#pragma unroll
			for (int r = 0; r < 16; r++) dq[r] = s[r] = dp[r] = 0.f;
			if constexpr (DT == 4) {
#pragma unroll
				for (int i = 0; i < NF; i++) bC[i] = ds_t_frag(sdS_prev, i * 16, lane);
#pragma unroll
				for (int i = 0; i < NF; i++) bA[i] = TL::rows(sQ, 0, i, lane);
				__builtin_amdgcn_sched_barrier(0);
				// dQ product of the previous tile, interleaved with S of this one
#pragma unroll
				for (int i = 0; i < NF; i++) {
					dq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktf[i], bC[i], dq, 0, 0, 0);
					s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bA[i], kf[i], s, 0, 0, 0);
				}
			} else {
#pragma unroll
				for (int i = 0; i < NF; i++) bA[i] = TL::rows(sQ, 0, i, lane);
				if (dq_wave) {
					bf16x8 bD[NQ];
#pragma unroll
					for (int i = 0; i < NQ; i++) bD[i] = ds_t_frag(sdS_prev, i * 16, lane);
#pragma unroll
					for (int i = 0; i < NQ; i++) dq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktf[i], bD[i], dq, 0, 0, 0);
				}
#pragma unroll
				for (int i = 0; i < NF; i++) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bA[i], kf[i], s, 0, 0, 0);
			}
			__builtin_amdgcn_sched_barrier(0);
#pragma unroll
			for (int i = 0; i < NF; i++) bC[i] = TL::rows(sdO, 0, i, lane);
			dq_out(dq_prev_tile, dq, 0, 4);
			__builtin_amdgcn_sched_barrier(0);
			// dP = dO V^T on the matrix pipe while the vector pipe turns S into P
#pragma unroll
			for (int i = 0; i < NF; i++) dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bC[i], vf[i], dp, 0, 0, 0);
			// dO^T fragments: rows d, k = queries in accumulator order
#pragma unroll
			for (int i = 0; i < NF; i++) bA[i] = TL::template cols<true>(sdO, (i / DT) * 16, (i % DT) * 32, lane);
			// causal mask: key > query  <=>  row index of the accumulator register < key - q0
			// (never true for a tile that lies wholly after the wave's keys; a wave whose keys lie
			// wholly after the tile gets P = 0 everywhere)
			const int kq = wkey0 + kl - q0 - 4 * g;
			float p[16];
			auto softmax = [&](auto masked) {
#pragma unroll
				for (int r4 = 0; r4 < 4; r4++) {
					const f32x4 l4 = *reinterpret_cast<const f32x4*>(sLse + r4 * 8 + 4 * g);
#pragma unroll
					for (int t = 0; t < 4; t++) {
						float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r4 * 4 + t], sc, l4[t]));
						if (decltype(masked)::value && r4 * 8 + t < kq) pr = 0.f;
						p[r4 * 4 + t] = pr;
					}
				}
			};
			// only the tiles on the diagonal (the wave's last key lies after the tile's first query) need the mask
			if (CAUSAL && wkey0 + 31 > q0) softmax(std::true_type{});
			else softmax(std::false_type{});
			const bf16x8 pf[2] = {pack8(p), pack8(p + 8)};
			dq_out(dq_prev_tile, dq, 4, 8);
			__builtin_amdgcn_sched_barrier(0);
			// dV^T[d][key] += dO^T[d][q] P[q][key] while the vector pipe forms dS = P (dP - delta)
#pragma unroll
			for (int i = 0; i < NF; i++) bC[i] = TL::template cols<true>(sQ, (i / DT) * 16, (i % DT) * 32, lane);
#pragma unroll
			for (int i = 0; i < NF; i++)
				acc_dv[i % DT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bA[i], pf[i / DT], acc_dv[i % DT], 0, 0, 0);
			float ds[16];
#pragma unroll
			for (int r4 = 0; r4 < 4; r4++) {
				const f32x4 d4 = *reinterpret_cast<const f32x4*>(sLse + 32 + r4 * 8 + 4 * g);
#pragma unroll
				for (int t = 0; t < 4; t++) ds[r4 * 4 + t] = p[r4 * 4 + t] * (dp[r4 * 4 + t] - d4[t]);
			}
			const bf16x8 dsf[2] = {pack8(ds), pack8(ds + 8)};
			// accumulator rows of register r: q = (r/4)*8 + 4g + r%4 -> four 8-byte groups per lane
#pragma unroll
			for (int u = 0; u < 2; u++) {
				const u32x4 w = __builtin_bit_cast(u32x4, dsf[u]);
				*reinterpret_cast<u32x2*>(sdS_cur + ds_t_offset(key_l, 16 * u + 4 * g)) = u32x2{w[0], w[1]};
				*reinterpret_cast<u32x2*>(sdS_cur + ds_t_offset(key_l, 16 * u + 8 + 4 * g)) = u32x2{w[2], w[3]};
			}
			dq_out(dq_prev_tile, dq, 8, 12);
			__builtin_amdgcn_sched_barrier(0);
			// dK^T[d][key] += Q^T[d][q] dS[q][key]
#pragma unroll
			for (int i = 0; i < NF; i++)
				acc_dk[i % DT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bC[i], dsf[i / DT], acc_dk[i % DT], 0, 0, 0);
			dq_out(dq_prev_tile, dq, 12, 16);
			dq_prev_tile = part + (int64_t)q0 * HqD + cur_h * D;
			if (++cur_qt == nqt_all) {
				cur_qt = qt_first;
				cur_h++;
			}
			// the next tile's loads were issued before this step's 4 partial stores and vector memory
			// operations complete in order: waiting until 4 are left waits for the loads only
			if (dq_wave) wait_vmcnt<4>();
			else wait_vmcnt<0>();
			__syncthreads();  // the next tile is in LDS, dS^T of this tile is complete, everyone is done with this tile
		}
		// drain: dQ product and partial of the last tile
		{
			const unsigned char* sdS_prev = sdS + ((n_iter + 1) & 1) * DS_BYTES;
			f32x16 dq;
#pragma unroll
			for (int r = 0; r < 16; r++) dq[r] = 0.f;
#pragma unroll
			for (int i = 0; i < NQ; i++)
				dq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktf[i], ds_t_frag(sdS_prev, i * 16, lane), dq, 0, 0, 0);
			dq_out(dq_prev_tile, dq, 0, 16);
		}

		// dK^T / dV^T accumulators: register r <-> d = dt*32 + (r/4)*8 + 4g + r%4, lane <-> key
		bf16_t* dkp = a.dk + (tok0 + wkey0 + kl) * a.lddk + hk * D;
		bf16_t* dvp = a.dv + (tok0 + wkey0 + kl) * a.lddv + hk * D;
		store_dk_dv<D>(acc_dk, acc_dv, dkp, dvp, a.scale, g, a.rope_cs ? a.rope_cs + (int64_t)(wkey0 + kl) * (D / 2) : nullptr);
	}
}

// The same pass for a wave that has its SIMD to itself (head_dim 128: K / V rows and accumulators fill the
// register file).  Nothing else fills its issue gaps, so the schedule is explicit: Q / dO tiles in a three-stage
// ring fetched two steps ahead, every fragment read issued one product ahead of its use into two buffers
// that alternate roles, and every MFMA pinned between its share of the reads and of the vector work.
// 2690 against 3650 cycles per tile; in the stream (between GEMMs) the call takes 1.04 against 1.13 ms.  At
// head_dim 64 the plain kernel above keeps two waves per SIMD, which this schedule's live ranges would cost.
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256) void attn_bwd_kernel_lone(AttnBwdArgs a) {
	using TL = BwdTile<D>;
	constexpr int BKV = 128, BQ = 32;
	constexpr int NF = D / 16;  // fragments per operand tile
	constexpr int DT = D / 32;
	constexpr int NQ = BKV / 16;  // fragments of the dQ product (all 128 keys); waves 0..DT-1 own one 32-column slice each
	constexpr int K_BYTES = BKV * TL::ROW_BYTES, Q_BYTES = BQ * TL::ROW_BYTES;
	constexpr int STAGE = 2 * Q_BYTES + 256;  // Q tile, dO tile, 32 nlse2 + 32 delta floats
	constexpr int NSTAGE = 3;                 // tiles are fetched two steps ahead
	constexpr int DS_BYTES = BKV * BQ * 2;
	constexpr int Q_LOADS = 8 / TL::RPI;  // DMA instructions per wave and tile (8 rows per wave)
	extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];
	unsigned char* const sKt = smem_raw;            // K tile, [key][d]
	unsigned char* const sStage = sKt + K_BYTES;       // NSTAGE x {Q [q][d], dO [q][d], nlse2, delta}
	unsigned char* const sdS = sStage + NSTAGE * STAGE;  // 2 x dS^T [key][q]

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int g = lane >> 5, kl = lane & 31;
	const int nkt = a.S / BKV;
	const int npair = CAUSAL ? (nkt + 1) / 2 : nkt;
	int pair = blockIdx.x % npair;
	int bh = blockIdx.x / npair;
	{
		// all key-tile workgroups of a (batch, kv head) group on one XCD (workgroup w runs on XCD w % 8)
		const int ngroups = (int)(gridDim.x / npair);
		if (ngroups % 8 == 0) {
			const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
			bh = xcd + 8 * (slot / npair);
			pair = slot % npair;
		}
	}
	const int hk = bh % a.Hkv, b = bh / a.Hkv;
	const int G = a.Hq / a.Hkv;
	const int64_t tok0 = (int64_t)b * a.S;
	const int64_t HqD = (int64_t)a.Hq * D;
	const float sc = a.scale * LOG2E;
	const bool dq_wave = DT == 4 || wave < DT;  // head_dim 64: two slices, waves 2 and 3 have no dQ share
	const int dq_dt = wave % DT;
	const int key_l = wave * 32 + kl;                        // this lane's key within the tile
	const int nqt_all = a.S / BQ;
	const int dq_lane = kl * (int)HqD + dq_dt * 32 + 4 * g;  // lane part of a dQ tile address (elements): query kl, first of 4 columns

	// DMA plan for one (Q, dO) tile pair: wave w moves rows [w*8, w*8+8) of each
	uint32_t qoff[Q_LOADS], dooff[Q_LOADS];
#pragma unroll
	for (int i = 0; i < Q_LOADS; i++) {
		const int row = wave * 8 + i * TL::RPI + lane / TL::CPR, slot = lane % TL::CPR;
		qoff[i] = (uint32_t)((row * a.ldq + ((slot ^ TL::swz(row)) << 3)) * 2);
		dooff[i] = (uint32_t)((row * a.lddo + ((slot ^ TL::swz(row)) << 3)) * 2);
	}
	auto zero_ds = [&](unsigned char* t) {
#pragma unroll
		for (int i = 0; i < 4; i++) *reinterpret_cast<u32x2*>(t + ds_t_offset(key_l, 8 * i + 4 * g)) = u32x2{0u, 0u};
	};
	// registers [r_lo, r_hi) of a dQ accumulator tile -> the partial buffer (issued a few at a time
	// between other work: a long burst backs up the memory pipeline and stalls the wave)
	auto dq_out = [&](bf16_t* tile, const f32x16& v, int r_lo, int r_hi) {
		if (!dq_wave) return;
#pragma unroll
		for (int j = 0; j < 4; j++)
			if (4 * j >= r_lo && 4 * j < r_hi) {
				bf16x4 o;
#pragma unroll
				for (int t = 0; t < 4; t++) o[t] = (bf16_t)v[4 * j + t];
				*reinterpret_cast<bf16x4*>(tile + dq_lane + 8 * j) = o;
			}
	};

	const int n_pass = (CAUSAL && nkt - 1 - pair != pair) ? 2 : 1;
#pragma unroll 1
	for (int pass = 0; pass < n_pass; pass++) {
		const int kt_idx = pass == 0 ? pair : nkt - 1 - pair;
		const int key0 = kt_idx * BKV;       // first key of the pass
		const int wkey0 = key0 + wave * 32;  // first key of this wave
		if (pass > 0) __syncthreads();       // every wave is done with the LDS of the previous pass

		// K tile -> LDS; this wave moves rows [wave*32, wave*32+32)
		{
			const bf16_t* kb = a.k + (tok0 + key0) * a.ldk + hk * D;
#pragma unroll
			for (int i = 0; i < 32 / TL::RPI; i++) {
				const int row = wave * 32 + i * TL::RPI + lane / TL::CPR, slot = lane % TL::CPR;
				dma16(kb, (uint32_t)((row * a.ldk + ((slot ^ TL::swz(row)) << 3)) * 2),
				      __builtin_amdgcn_readfirstlane(lds_addr(sKt) + (wave * 32 + i * TL::RPI) * TL::ROW_BYTES));
			}
		}
		// own K and V rows as B operands (n = key, 8 consecutive d) in registers
		bf16x8 kf[NF], vf[NF];
		{
			const bf16_t* kp = a.k + (tok0 + wkey0 + kl) * a.ldk + hk * D + 8 * g;
			const bf16_t* vp = a.v + (tok0 + wkey0 + kl) * a.ldv + hk * D + 8 * g;
#pragma unroll
			for (int ks = 0; ks < NF; ks++) {
				kf[ks] = *reinterpret_cast<const bf16x8*>(kp + ks * 16);
				vf[ks] = *reinterpret_cast<const bf16x8*>(vp + ks * 16);
				asm volatile("" : "+a"(kf[ks]), "+a"(vf[ks]));
			}
		}
		f32x16 acc_dk[DT], acc_dv[DT];
#pragma unroll
		for (int i = 0; i < DT; i++)
#pragma unroll
			for (int r = 0; r < 16; r++) acc_dk[i][r] = acc_dv[i][r] = 0.f;

		// Walk over (query head in group, query tile); causal: only tiles that reach key0.
		const int qt_first = CAUSAL ? key0 / BQ : 0;
		const int n_iter = G * (nqt_all - qt_first);

		// tile whose loads are issued next: running pointers, recomputed when the walk moves to the next head
		int ld_h = hk * G, ld_qt = qt_first;
		const bf16_t* ld_q;
		const bf16_t* ld_do;
		const float* ld_stat;  // lanes 0..31: nlse2 of the tile's queries, lanes 32..63: delta
		auto seek = [&]() {
			const int64_t row = tok0 + ld_qt * BQ;
			ld_q = a.q + row * a.ldq + ld_h * D;
			ld_do = a.dO + row * a.lddo + ld_h * D;
			ld_stat = (lane < 32 ? a.nlse2 : a.delta) + ((int64_t)b * a.Hq + ld_h) * a.S + ld_qt * BQ + (lane & 31);
		};
		seek();
		const uint32_t lds_stage = lds_addr(sStage) + wave * 8 * TL::ROW_BYTES;
		auto issue = [&](int stage) {
			const uint32_t st = lds_stage + (uint32_t)stage * STAGE;
#pragma unroll
			for (int i = 0; i < Q_LOADS; i++) {
				dma16(ld_q, qoff[i], __builtin_amdgcn_readfirstlane(st + i * TL::RPI * TL::ROW_BYTES));
				dma16(ld_do, dooff[i], __builtin_amdgcn_readfirstlane(st + Q_BYTES + i * TL::RPI * TL::ROW_BYTES));
			}
			if (wave == 0) dma4(ld_stat, __builtin_amdgcn_readfirstlane(st + 2 * Q_BYTES));
			if (++ld_qt == nqt_all) {
				ld_qt = qt_first;
				ld_h++;
				seek();
			} else {
				ld_q += BQ * a.ldq;
				ld_do += BQ * a.lddo;
				ld_stat += BQ;
			}
		};

		issue(0);
		if (n_iter > 1) issue(1);
		zero_ds(sdS + DS_BYTES);  // the "previous tile" of the first iteration
		wait_vmcnt<0>();
		__syncthreads();
		// this wave's slice of K as B operands of the dQ product (n = d column, k = key)
		bf16x8 ktf[NQ];
#pragma unroll
		for (int i = 0; i < NQ; i++) ktf[i] = TL::template cols<false>(sKt, i * 16, dq_dt * 32, lane);

		// position of the current tile; dq_prev_tile = where the dQ tile of iteration it-1 goes
		int cur_h = hk * G, cur_qt = qt_first;
		// rows of this key tile's slice: first query of the slice = key0 (causal) or 0
		bf16_t* const part = a.dq_part + ((int64_t)b * part_rows(a.S, CAUSAL) + part_row0(kt_idx, a.S, CAUSAL) - qt_first * BQ) * HqD;
		bf16_t* dq_prev_tile = part + (int64_t)(qt_first * BQ) * HqD + cur_h * D;

		// One step = one (head, 32-query tile).  Two fragment buffers alternate roles so that every LDS
		// read is issued one product ahead of the MFMAs that consume it (one wave per SIMD: nothing else
		// hides the latency): X enters holding the Q rows of this tile, read during the previous step
		// (the tile has been in LDS since the barrier before that step), and leaves free; Y leaves
		// holding the Q rows of the next tile, so the caller swaps the two for the next step.
		//   Y <- dS^T(prev)     | S  = X(Q) K^T
		//   X <- dO rows        | dQ(prev) = Y K            softmax on the vector pipe
		//   Y <- dO^T           | dP = X(dO) V^T
		//   X <- Q^T            | dV^T += Y(dO^T) P         dS on the vector pipe, dS^T -> LDS
		//   Y <- Q rows (next)  | dK^T += X(Q^T) dS
		int stage = 0;  // it % NSTAGE
		auto step = [&](bf16x8(&X)[NQ], bf16x8(&Y)[NQ], int it) {
			const int load_stage = stage == 0 ? 2 : stage - 1;  // (it + 2) % 3
			const unsigned char* sQ = sStage + stage * STAGE;
			const unsigned char* sdO = sQ + Q_BYTES;
			const float* sLse = reinterpret_cast<const float*>(sdO + Q_BYTES);
			stage = stage == NSTAGE - 1 ? 0 : stage + 1;
			const unsigned char* sQ_next = sStage + stage * STAGE;
			const unsigned char* sdS_prev = sdS + ((it + 1) & 1) * DS_BYTES;
			unsigned char* sdS_cur = sdS + (it & 1) * DS_BYTES;
			const int q0 = cur_qt * BQ;

			f32x16 dq, s, dp;
#pragma unroll
			for (int r = 0; r < 16; r++) dq[r] = s[r] = dp[r] = 0.f;
			// A single wave per SIMD issues in order, so matrix and vector work only overlap where the
			// program interleaves them: every product below is a loop of "one MFMA + its share of the
			// LDS reads and vector work that ride along", pinned by scheduling barriers.
			// causal mask: key > query  <=>  row index of the accumulator register < key - q0
			// (never true for a tile that lies wholly after the wave's keys; a wave whose keys lie
			// wholly after the tile gets P = 0 everywhere)
			const int kq = wkey0 + kl - q0 - 4 * g;
			f32x4 l4[4];
			// S = Q K^T, with the dS^T fragments of the previous tile on their way; the loads of the tile after
			// next and the reads of this tile's statistics go between the MFMAs too
#pragma unroll
			for (int i = 0; i < NF; i++) {
				if (dq_wave) {
#pragma unroll
					for (int j = i * (NQ / NF); j < (i + 1) * (NQ / NF); j++) Y[j] = ds_t_frag(sdS_prev, j * 16, lane);
				}
				s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(X[i], kf[i], s, 0, 0, 0);
				if (i == 0 && it + 2 < n_iter) issue(load_stage);
				if (i == NF / 2) {
#pragma unroll
					for (int r4 = 0; r4 < 4; r4++) l4[r4] = *reinterpret_cast<const f32x4*>(sLse + r4 * 8 + 4 * g);
				}
				__builtin_amdgcn_sched_barrier(0);
			}
			// dQ of the previous tile = dS K, with the dO rows on their way and P = exp2(S sc - lse) on the vector pipe
			float p[16];
			auto dq_and_softmax = [&](auto masked) {
#pragma unroll
				for (int i = 0; i < NQ; i++) {
					if (i < NF) X[i] = TL::rows(sdO, 0, i, lane);
					if (dq_wave) dq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktf[i], Y[i], dq, 0, 0, 0);
#pragma unroll
					for (int r = i * (16 / NQ); r < (i + 1) * (16 / NQ); r++) {
						float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], sc, l4[r >> 2][r & 3]));
						if (decltype(masked)::value && (r >> 2) * 8 + (r & 3) < kq) pr = 0.f;
						p[r] = pr;
					}
					__builtin_amdgcn_sched_barrier(0);
				}
			};
			// only the tiles on the diagonal (the wave's last key lies after the tile's first query) need the mask
			if (CAUSAL && wkey0 + 31 > q0) dq_and_softmax(std::true_type{});
			else dq_and_softmax(std::false_type{});
			const bf16x8 pf[2] = {pack8(p), pack8(p + 8)};
			f32x4 d4[4];
#pragma unroll
			for (int r4 = 0; r4 < 4; r4++) d4[r4] = *reinterpret_cast<const f32x4*>(sLse + 32 + r4 * 8 + 4 * g);
			// dP = dO V^T, with the dO^T fragments (rows d, k = queries in accumulator order) on their way and the
			// previous tile's dQ partial going out
#pragma unroll
			for (int i = 0; i < NF; i++) {
				Y[i] = TL::template cols<true>(sdO, (i / DT) * 16, (i % DT) * 32, lane);
				dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(X[i], vf[i], dp, 0, 0, 0);
				if ((i * 4) % NF == 0) dq_out(dq_prev_tile, dq, (i * 4 / NF) * 4, (i * 4 / NF) * 4 + 4);
				__builtin_amdgcn_sched_barrier(0);
			}
			// dV^T[d][key] += dO^T[d][q] P[q][key], with the Q^T fragments on their way and dS = P (dP - delta) on
			// the vector pipe
			// (dS in the first half of the slots, its packing and the dS^T writes in the next two)
			float ds[16];
			bf16x8 dsf[2];
#pragma unroll
			for (int i = 0; i < NF; i++) {
				X[i] = TL::template cols<true>(sQ, (i / DT) * 16, (i % DT) * 32, lane);
				acc_dv[i % DT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Y[i], pf[i / DT], acc_dv[i % DT], 0, 0, 0);
				if (i < NF / 2) {
#pragma unroll
					for (int r = i * (32 / NF); r < (i + 1) * (32 / NF); r++) ds[r] = p[r] * (dp[r] - d4[r >> 2][r & 3]);
				} else if (i < NF / 2 + 2) {
					// accumulator rows of register r: q = (r/4)*8 + 4g + r%4 -> four 8-byte groups per lane
					const int u = i - NF / 2;
					dsf[u] = pack8(ds + 8 * u);
					const u32x4 w = __builtin_bit_cast(u32x4, dsf[u]);
					*reinterpret_cast<u32x2*>(sdS_cur + ds_t_offset(key_l, 16 * u + 4 * g)) = u32x2{w[0], w[1]};
					*reinterpret_cast<u32x2*>(sdS_cur + ds_t_offset(key_l, 16 * u + 8 + 4 * g)) = u32x2{w[2], w[3]};
				}
				__builtin_amdgcn_sched_barrier(0);
			}
			// dK^T[d][key] += Q^T[d][q] dS[q][key], with the Q rows of the next tile on their way (past the last
			// tile: a stale stage, values unused)
#pragma unroll
			for (int i = 0; i < NF; i++) {
				Y[i] = TL::rows(sQ_next, 0, i, lane);
				acc_dk[i % DT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(X[i], dsf[i / DT], acc_dk[i % DT], 0, 0, 0);
				__builtin_amdgcn_sched_barrier(0);
			}
			dq_prev_tile = part + (int64_t)q0 * HqD + cur_h * D;
			if (++cur_qt == nqt_all) {
				cur_qt = qt_first;
				cur_h++;
			}
			// the loads of the tile after next were issued before this step's 4 partial stores and vector
			// memory operations complete in order: waiting until 4 are left waits for the loads only
			if (dq_wave) wait_counters<4, 0>();
			else wait_counters<0, 0>();
			__syncthreads();  // the tile after next is in LDS, dS^T of this tile is complete, everyone is done with this tile
		};

		bf16x8 fragA[NQ], fragB[NQ];
#pragma unroll
		for (int i = 0; i < NF; i++) fragA[i] = TL::rows(sStage, 0, i, lane);
		for (int it = 0; it < n_iter; it += 2) {
			step(fragA, fragB, it);
			if (it + 1 < n_iter) step(fragB, fragA, it + 1);
		}
		// drain: dQ product and partial of the last tile
		{
			const unsigned char* sdS_prev = sdS + ((n_iter + 1) & 1) * DS_BYTES;
			f32x16 dq;
#pragma unroll
			for (int r = 0; r < 16; r++) dq[r] = 0.f;
#pragma unroll
			for (int i = 0; i < NQ; i++)
				dq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktf[i], ds_t_frag(sdS_prev, i * 16, lane), dq, 0, 0, 0);
			dq_out(dq_prev_tile, dq, 0, 16);
		}

		// dK^T / dV^T accumulators: register r <-> d = dt*32 + (r/4)*8 + 4g + r%4, lane <-> key
		bf16_t* dkp = a.dk + (tok0 + wkey0 + kl) * a.lddk + hk * D;
		bf16_t* dvp = a.dv + (tok0 + wkey0 + kl) * a.lddv + hk * D;
		store_dk_dv<D>(acc_dk, acc_dv, dkp, dvp, a.scale, g, a.rope_cs ? a.rope_cs + (int64_t)(wkey0 + kl) * (D / 2) : nullptr);
	}
}

// dq[b, q, :] (bf16, row stride ld) = scale * sum over the key tiles that meet q of their partial rows,
// added in fp32 in ascending tile order.  A thread takes 8 columns of a head's first half and the 8 columns
// half a head further on; with a rotary embedding on the q heads (cs non-null) these are the pairs of the
// rotation, which is undone on the scaled, bf16-rounded sums before they are stored (what a separate RoPE
// pass over the stored gradient would compute).
__global__ __launch_bounds__(256) void dq_reduce_kernel(const bf16_t* __restrict__ part, bf16_t* __restrict__ dq, int B, int S, int cols,
                                                        int64_t ld, float scale, int causal, int D, const float2* __restrict__ cs) {
	const int half = D / 2, cph = half / 8;  // 8-column chunks per half head
	const int ppr = cols / 16;               // chunk pairs per row
	const int64_t n = (int64_t)B * S * ppr;
	const int nkt = S / 128;
	const int64_t rows_b = part_rows(S, causal);
	for (int64_t j = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; j < n; j += (int64_t)gridDim.x * blockDim.x) {
		// last rows first: under a causal mask they sum the most partials, and the launch then ends on the short ones
		const int64_t i = n - 1 - j;
		const int64_t row = i / ppr;
		const int pr = (int)(i - row * ppr);
		const int c = (pr / cph) * D + (pr % cph) * 8;
		const int b = (int)(row / S), q = (int)(row - (int64_t)b * S);
		const int ns = causal ? q / 128 + 1 : nkt;
		float lo[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, hi[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
		const bf16_t* pb = part + (int64_t)b * rows_b * cols + c;
#pragma unroll 8
		for (int kt = 0; kt < ns; kt++) {
			const bf16_t* pr_row = pb + (part_row0(kt, S, causal) + q - (causal ? 128 * kt : 0)) * cols;
			// read once: no point in keeping the partials in the caches
			const bf16x8 v = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(pr_row)), w = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(pr_row + half));
#pragma unroll
			for (int t = 0; t < 8; t++) {
				lo[t] += (float)v[t];
				hi[t] += (float)w[t];
			}
		}
		bf16x8 olo, ohi;
#pragma unroll
		for (int t = 0; t < 8; t++) {
			olo[t] = (bf16_t)(lo[t] * scale);
			ohi[t] = (bf16_t)(hi[t] * scale);
		}
		if (cs) {
			const float2* tab = cs + (int64_t)q * half + (pr % cph) * 8;
#pragma unroll
			for (int t = 0; t < 8; t++) {
				const float2 t2 = tab[t];
				float rl, rh;
				rope_rot((float)olo[t], (float)ohi[t], t2.x, -t2.y, rl, rh);
				olo[t] = (bf16_t)rl;
				ohi[t] = (bf16_t)rh;
			}
		}
		*reinterpret_cast<bf16x8*>(dq + row * ld + c) = olo;
		*reinterpret_cast<bf16x8*>(dq + row * ld + c + half) = ohi;
	}
}

template <int D, bool CAUSAL>
int launch_bwd(const AttnBwdArgs& a, dim3 grid, hipStream_t stream) {
	// K tile + the Q / dO ring (two stages, three for the lone-wave schedule) + two dS^T tiles
	constexpr bool LONE = D == 128;
	constexpr int smem = 128 * D * 2 + (LONE ? 3 : 2) * (2 * 32 * D * 2 + 256) + 2 * 128 * 32 * 2;
	auto kern = LONE ? attn_bwd_kernel_lone<D, CAUSAL> : attn_bwd_kernel<D, CAUSAL>;
	static bool attr_set = false;
	if (!attr_set) {
		ELF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
		attr_set = true;
	}
	ELF_LAUNCH(kern, grid, dim3(256), smem, stream, a);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

}  // namespace attn

using namespace attn;

int64_t attn_bwd_workspace_bytes(int B, int S, int Hq, int D, int causal) {
	// bf16 dQ partials of every key tile + delta + scaled log-sum-exp
	return (int64_t)B * part_rows(S, causal != 0) * Hq * D * 2 + 2 * (int64_t)B * S * Hq * 4;
}

int attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dO, const void* lse, void* dq,
             void* dk, void* dv, void* workspace, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo,
             int64_t lddq, int64_t lddk, int64_t lddv, int B, int S, int Hq, int Hkv, int D, int causal, float scale,
             hipStream_t stream, const void* rope_cs) {
	ELF_REQUIRE(q && k && v && o && dO && lse && dq && dk && dv && workspace, "attn_bwd: null pointer");
	ELF_REQUIRE(((uintptr_t)rope_cs % 16) == 0, "attn_bwd: misaligned rotary table");
	ELF_REQUIRE(B > 0 && S > 0 && S % 128 == 0, "attn_bwd: sequence length must be a multiple of 128 (S=%d)", S);
	ELF_REQUIRE(Hkv > 0 && Hq % Hkv == 0, "attn_bwd: Hq must be a multiple of Hkv (Hq=%d Hkv=%d)", Hq, Hkv);
	ELF_REQUIRE(D == 64 || D == 128, "attn_bwd: head_dim must be 64 or 128 (D=%d)", D);
	ELF_REQUIRE(ldq % 8 == 0 && ldk % 8 == 0 && ldv % 8 == 0 && ldo % 8 == 0 && lddo % 8 == 0 && lddq % 8 == 0 &&
	                lddk % 8 == 0 && lddv % 8 == 0,
	            "attn_bwd: strides must be multiples of 8");
	ELF_REQUIRE(((uintptr_t)workspace % 16) == 0, "attn_bwd: misaligned workspace");
	ELF_REQUIRE(((uintptr_t)o % 16) == 0 && ((uintptr_t)dO % 16) == 0, "attn_bwd: o and dO must be 16-byte aligned");
	ProfScope prof(PROF_ATTN_BWD, (causal ? 4.0 : 8.0) * B * Hq * (double)S * S * D, stream);
	const int64_t T = (int64_t)B * S;
	bf16_t* dq_part = (bf16_t*)workspace;
	float* delta = (float*)(dq_part + (int64_t)B * part_rows(S, causal != 0) * Hq * D);
	float* nlse2 = delta + T * Hq;
	{
		const int64_t rows = T * Hq, per_block = 256 / (D / 8);
		const int64_t want = (rows + per_block - 1) / per_block;
		ELF_LAUNCH(attn_delta_kernel, dim3((unsigned)(want < 8192 ? want : 8192)), dim3(256), 0, stream, (const bf16_t*)dO,
	                   (const bf16_t*)o, (const float*)lse, delta, nlse2, lddo, ldo, B, S, Hq, D);
	}
	AttnBwdArgs a{(const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, (const bf16_t*)dO, nlse2, delta, dq_part,
	              (bf16_t*)dk, (bf16_t*)dv, ldq, ldk, ldv, lddo, lddk, lddv, B, S, Hq, Hkv, scale, (const float2*)rope_cs};
	const int nkt = S / 128;
	const dim3 grid((unsigned)((int64_t)B * Hkv * (causal ? (nkt + 1) / 2 : nkt))), block(256);
	int rc;
	if (D == 128) rc = causal ? launch_bwd<128, true>(a, grid, stream) : launch_bwd<128, false>(a, grid, stream);
	else rc = causal ? launch_bwd<64, true>(a, grid, stream) : launch_bwd<64, false>(a, grid, stream);
	if (rc) return rc;
	const int64_t n16 = T * (Hq * D / 16);
	const int64_t blocks = (n16 + 255) / 256;
	ELF_LAUNCH(dq_reduce_kernel, dim3((unsigned)(blocks < 16384 ? blocks : 16384)), dim3(256), 0, stream, dq_part, (bf16_t*)dq, B, S,
	                   Hq * D, lddq, scale, causal, D, (const float2*)rope_cs);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

}  // namespace elf
