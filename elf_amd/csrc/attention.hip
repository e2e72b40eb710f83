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

// ------------------------------------------------------------------------------------------
// Forward.  K and V tiles (64 keys) are fetched straight into LDS (lds_dma.h) in a two-stage
// ring; tiles are unpadded (a wave instruction fills 1 KiB contiguously), so the 16-byte chunk
// index of every row is XOR-swizzled: for K (read along d, one row per lane) with a function
// of the row that spreads 16 consecutive rows over all 16 bank groups, for V (read with the
// transpose read, 4 rows x 32 B per 16 lanes) with an even value so that chunk pairs stay
// adjacent.
template <int D>
struct FwdTile {
	static constexpr int ROW_BYTES = D * 2;
	static constexpr int CPR = D / 8;                  // 16-byte chunks per row
	static constexpr int TILE_BYTES = 64 * ROW_BYTES;  // one operand, 64 keys
	static constexpr int RPI = 1024 / ROW_BYTES;       // rows per DMA wave instruction
	static constexpr int LOADS = TILE_BYTES / 1024 / 4;  // DMA instructions per wave and operand
	__device__ static __forceinline__ int k_swz(int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); }
	__device__ static __forceinline__ int v_swz(int row) { return D == 128 ? ((row & 7) << 1) : (((row >> 1) & 3) << 1); }
};

template <int D, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(AttnArgs a) {
	using TL = FwdTile<D>;
	constexpr int BQ = 128, BKV = 64;
	constexpr int KSTEPS = D / 16, DT = D / 32;
	constexpr int STAGE = 2 * TL::TILE_BYTES;
	extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int g = lane >> 5, ql = lane & 31;
	const int nqt = a.S / BQ;
	// heaviest (last) query tiles first when causal
	const int qt = CAUSAL ? (nqt - 1 - (int)(blockIdx.x % nqt)) : (int)(blockIdx.x % nqt);
	const int bh = blockIdx.x / nqt;
	const int h = bh % a.Hq, b = bh / a.Hq;
	const int hk = h / (a.Hq / a.Hkv);
	const int q0 = qt * BQ + wave * 32;  // first query (in sequence) of this wave
	const int64_t tok0 = (int64_t)b * a.S;

	// Q fragments as B operand (n = query, 8 consecutive d), straight from HBM.
	bf16x8 qf[KSTEPS];
	{
		const bf16_t* qp = a.q + (tok0 + q0 + ql) * a.ldq + h * D + 8 * g;
#pragma unroll
		for (int ks = 0; ks < KSTEPS; ks++) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + ks * 16);
	}

	// DMA plan: this wave moves rows [wave*LOADS*RPI, ...) of each 64-key tile
	uint32_t koff[TL::LOADS], voff[TL::LOADS];
#pragma unroll
	for (int i = 0; i < TL::LOADS; i++) {
		const int row = (wave * TL::LOADS + i) * TL::RPI + lane / TL::CPR, slot = lane % TL::CPR;
		koff[i] = (uint32_t)((row * a.ldk + ((slot ^ TL::k_swz(row)) << 3)) * 2);
		voff[i] = (uint32_t)((row * a.ldv + ((slot ^ TL::v_swz(row)) << 3)) * 2);
	}
	const bf16_t* kg = a.k + tok0 * a.ldk + hk * D;
	const bf16_t* vg = a.v + tok0 * a.ldv + hk * D;
	const uint32_t lds0 = lds_addr(smem_raw) + wave * (TL::LOADS * 1024);
	auto issue = [&](int j) {
		const uint32_t st = lds0 + (uint32_t)(j & 1) * STAGE;
		const bf16_t* kb = kg + (int64_t)j * BKV * a.ldk;
		const bf16_t* vb = vg + (int64_t)j * BKV * a.ldv;
#pragma unroll
		for (int i = 0; i < TL::LOADS; i++) dma16(kb, koff[i], __builtin_amdgcn_readfirstlane(st + i * 1024));
#pragma unroll
		for (int i = 0; i < TL::LOADS; i++) dma16(vb, voff[i], __builtin_amdgcn_readfirstlane(st + TL::TILE_BYTES + i * 1024));
	};

	f32x16 acc_o[DT];
#pragma unroll
	for (int i = 0; i < DT; i++)
#pragma unroll
		for (int r = 0; r < 16; r++) acc_o[i][r] = 0.f;
	float m_run = -INFINITY, l_run = 0.f;  // running max (in log2 units, already scaled) and sum
	const float sc = a.scale * LOG2E;
	const int qpos = q0 + ql;

	const int n_kv = CAUSAL ? ((qt + 1) * BQ) / BKV : a.S / BKV;
	issue(0);
	for (int j = 0; j < n_kv; j++) {
		wait_vmcnt<0>();
		__syncthreads();  // tile j is in LDS for everyone; everyone is done with tile j-1
		if (j + 1 < n_kv) issue(j + 1);
		const int k0 = j * BKV;
		if (CAUSAL && k0 > q0 + 31) continue;  // every key of the tile is in this wave's future
		const unsigned char* sK = smem_raw + (j & 1) * STAGE;
		const unsigned char* sV = sK + TL::TILE_BYTES;

		// S^T[key][q] for the two 32-key halves
		f32x16 s[2];
#pragma unroll
		for (int kt = 0; kt < 2; kt++) {
#pragma unroll
			for (int r = 0; r < 16; r++) s[kt][r] = 0.f;
			const int row = kt * 32 + ql;
			const unsigned char* rowp = sK + row * TL::ROW_BYTES;
#pragma unroll
			for (int ks = 0; ks < KSTEPS; ks++) {
				const bf16x8 kf = *reinterpret_cast<const bf16x8*>(rowp + (((2 * ks + g) ^ TL::k_swz(row)) << 4));
				s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], s[kt], 0, 0, 0);
			}
		}
		// causal mask only where the tile crosses the diagonal of this wave's queries
		if (CAUSAL && k0 + BKV - 1 > q0) {
#pragma unroll
			for (int kt = 0; kt < 2; kt++)
#pragma unroll
				for (int r = 0; r < 16; r++) {
					const int key = k0 + kt * 32 + (r >> 2) * 8 + 4 * g + (r & 3);
					if (key > qpos) s[kt][r] = -INFINITY;
				}
		}
		float mx = s[0][0];
#pragma unroll
		for (int kt = 0; kt < 2; kt++)
#pragma unroll
			for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[kt][r]);
		mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
		// every query sees key 0 in its first tile, so the running max is finite from then on
		const float m_new = fmaxf(m_run, mx * sc);
		float psum = 0.f;
#pragma unroll
		for (int kt = 0; kt < 2; kt++)
#pragma unroll
			for (int r = 0; r < 16; r++) {
				const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][r], sc, -m_new));
				s[kt][r] = p;
				psum += p;
			}
		// rescale only when some query of the wave raised its maximum
		if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
			const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
			l_run *= alpha;
#pragma unroll
			for (int i = 0; i < DT; i++)
#pragma unroll
				for (int r = 0; r < 16; r++) acc_o[i][r] *= alpha;
			m_run = m_new;
		}
		l_run += psum;
		// O^T[d][q] += V^T[d][key] P^T[key][q]
#pragma unroll
		for (int kt = 0; kt < 2; kt++) {
#pragma unroll
			for (int u = 0; u < 2; u++) {
				float pv[8];
#pragma unroll
				for (int t = 0; t < 8; t++) pv[t] = s[kt][u * 8 + t];
				const bf16x8 pf = pack8(pv);
				// keys {kk..kk+3} and {kk+8..kk+11}: the row order of the accumulator tile
				const int j16 = lane & 15;
				const int kk = kt * 32 + u * 16 + 4 * g + (j16 >> 2);
#pragma unroll
				for (int dt = 0; dt < DT; dt++) {
					const int c = (dt * 32 + 16 * (ql >> 4) + 4 * (j16 & 3)) >> 3;
					const unsigned char* p0 = sV + kk * TL::ROW_BYTES + ((c ^ TL::v_swz(kk)) << 4) + (j16 & 1) * 8;
					const unsigned char* p1 = sV + (kk + 8) * TL::ROW_BYTES + ((c ^ TL::v_swz(kk + 8)) << 4) + (j16 & 1) * 8;
					s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p0));
					s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p1));
					const bf16x8 vf = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
					acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, acc_o[dt], 0, 0, 0);
				}
			}
		}
	}

	const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
	const float inv = 1.f / l_tot;
	const int64_t tok = tok0 + q0 + ql;
	bf16_t* op = a.o + tok * a.ldo + h * D;
#pragma unroll
	for (int dt = 0; dt < DT; dt++) {
#pragma unroll
		for (int r4 = 0; r4 < 4; r4++) {
			bf16x4 o4;
#pragma unroll
			for (int t = 0; t < 4; t++) o4[t] = (bf16_t)(acc_o[dt][r4 * 4 + t] * inv);
			*reinterpret_cast<bf16x4*>(op + dt * 32 + r4 * 8 + 4 * g) = o4;
		}
	}
	if (g == 0) a.lse[((int64_t)b * a.Hq + h) * a.S + q0 + ql] = m_run * (1.f / LOG2E) + __logf(l_tot);
}

// ------------------------------------------------------------------------------------------
// delta[b,h,s] = sum_d dO * O   (one wave per token-head)
__global__ __launch_bounds__(256) void attn_delta_kernel(const bf16_t* __restrict__ dO, const bf16_t* __restrict__ O,
                                                         float* __restrict__ delta, int64_t ldd, int64_t ldo, int B, int S,
                                                         int Hq, int D) {
	const int lane = threadIdx.x & 63;
	const int64_t idx = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // token * Hq + h
	if (idx >= (int64_t)B * S * Hq) return;
	const int h = (int)(idx % Hq);
	const int64_t tok = idx / Hq;
	float s = 0.f;
	for (int c = lane * 2; c < D; c += 128) {
		bf16x2 x = *reinterpret_cast<const bf16x2*>(dO + tok * ldd + h * D + c);
		bf16x2 y = *reinterpret_cast<const bf16x2*>(O + tok * ldo + h * D + c);
		s += (float)x[0] * (float)y[0] + (float)x[1] * (float)y[1];
	}
	s = wave_sum(s);
	if (lane == 0) {
		const int64_t b = tok / S, sp = tok % S;
		delta[(b * Hq + h) * S + sp] = s;
	}
}

struct AttnBwdArgs {
	const bf16_t* q;
	const bf16_t* k;
	const bf16_t* v;
	const bf16_t* dO;
	const float* lse;
	const float* delta;
	float* dq_acc;  // fp32 [T, Hq*D], zero-initialised by the caller side of the launcher
	bf16_t* dk;
	bf16_t* dv;
	int64_t ldq, ldk, ldv, lddo, lddk, lddv;
	int B, S, Hq, Hkv;
	float scale;
};

template <int D, bool CAUSAL>
__global__ __launch_bounds__(256) void attn_bwd_kernel(AttnBwdArgs a) {
	constexpr int BKV = 128, BQ = 32;
	constexpr int LD = AttnSmem<D>::LDT;  // one stride for tiles that are read both ways
	constexpr int LDS_ = BKV + 8;         // dS tile [q][key]
	constexpr int KSTEPS = D / 16, DT = D / 32;
	constexpr int CHQ = (BQ * D / 8 + 255) / 256;  // 16-byte chunks per thread for a 32 x D tile
	extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
	bf16_t* sKt = reinterpret_cast<bf16_t*>(smem_raw);  // K tile, [key][d]
	bf16_t* const sQ0 = sKt + BKV * LD;       // Q tiles, [q][d]
	bf16_t* const sdO0 = sQ0 + 2 * BQ * LD;   // dO tiles, [q][d]
	bf16_t* const sdS = sdO0 + 2 * BQ * LD;   // [q][key]
	float* const sLse0 = reinterpret_cast<float*>(sdS + BQ * LDS_);
	float* const sDelta0 = sLse0 + 2 * BQ;
	auto sQ = [&](int i) { return sQ0 + i * (BQ * LD); };
	auto sdO = [&](int i) { return sdO0 + i * (BQ * LD); };
	auto sLse = [&](int i) { return sLse0 + i * BQ; };
	auto sDelta = [&](int i) { return sDelta0 + i * BQ; };

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int g = lane >> 5, kl = lane & 31;
	const int nkt = a.S / BKV;
	const int kt_idx = blockIdx.x % nkt;
	const int bh = blockIdx.x / nkt;
	const int hk = bh % a.Hkv, b = bh / a.Hkv;
	const int G = a.Hq / a.Hkv;
	const int64_t tok0 = (int64_t)b * a.S;
	const int key0 = kt_idx * BKV;        // first key of the workgroup
	const int wkey0 = key0 + wave * 32;   // first key of this wave
	const float sc = a.scale * LOG2E;

	// K tile to LDS (needed by all waves for dQ); own K and V rows as B operands in registers.
	{
		constexpr int CHK = BKV * D / 8 / 256;
		u32x4 r[CHK];
		copy_tile_g2r<BKV, D, LD, 256>(a.k + (tok0 + key0) * a.ldk + hk * D, a.ldk, tid, r);
		copy_tile_r2s<BKV, D, LD, 256>(sKt, tid, r);
	}
	bf16x8 kf[KSTEPS], vf[KSTEPS];
	{
		const bf16_t* kp = a.k + (tok0 + wkey0 + kl) * a.ldk + hk * D + 8 * g;
		const bf16_t* vp = a.v + (tok0 + wkey0 + kl) * a.ldv + hk * D + 8 * g;
#pragma unroll
		for (int ks = 0; ks < KSTEPS; ks++) {
			kf[ks] = *reinterpret_cast<const bf16x8*>(kp + ks * 16);
			vf[ks] = *reinterpret_cast<const bf16x8*>(vp + ks * 16);
		}
	}
	f32x16 acc_dk[DT], acc_dv[DT];
#pragma unroll
	for (int i = 0; i < DT; i++)
#pragma unroll
		for (int r = 0; r < 16; r++) acc_dk[i][r] = acc_dv[i][r] = 0.f;

	// Flattened walk over (query head in group, query tile); causal: only tiles that reach key0.
	const int qt_first = CAUSAL ? key0 / BQ : 0;
	const int nqt = a.S / BQ - qt_first;
	const int n_iter = G * nqt;

	auto tile_ptrs = [&](int it, const bf16_t*& qp, const bf16_t*& dop, const float*& lp, const float*& dp, int& h, int& q0) {
		const int hg = it / nqt;
		q0 = (qt_first + it % nqt) * BQ;
		h = hk * G + hg;
		qp = a.q + (tok0 + q0) * a.ldq + h * D;
		dop = a.dO + (tok0 + q0) * a.lddo + h * D;
		lp = a.lse + ((int64_t)b * a.Hq + h) * a.S + q0;
		dp = a.delta + ((int64_t)b * a.Hq + h) * a.S + q0;
	};

	u32x4 qr[CHQ], dor[CHQ];
	float lse_r = 0.f, delta_r = 0.f;
	auto load_regs = [&](int it) {
		const bf16_t *qp, *dop;
		const float *lp, *dp;
		int h, q0;
		tile_ptrs(it, qp, dop, lp, dp, h, q0);
		constexpr int CPR = D / 8;
#pragma unroll
		for (int i = 0; i < CHQ; i++) {
			const int c = tid + i * 256;
			if (c < BQ * CPR) {
				qr[i] = *reinterpret_cast<const u32x4*>(qp + (int64_t)(c / CPR) * a.ldq + (c % CPR) * 8);
				dor[i] = *reinterpret_cast<const u32x4*>(dop + (int64_t)(c / CPR) * a.lddo + (c % CPR) * 8);
			}
		}
		if (tid < BQ) {
			lse_r = lp[tid] * LOG2E;
			delta_r = dp[tid];
		}
	};
	auto store_lds = [&](int buf) {
		constexpr int CPR = D / 8;
#pragma unroll
		for (int i = 0; i < CHQ; i++) {
			const int c = tid + i * 256;
			if (c < BQ * CPR) {
				*reinterpret_cast<u32x4*>(sQ(buf) + (c / CPR) * LD + (c % CPR) * 8) = qr[i];
				*reinterpret_cast<u32x4*>(sdO(buf) + (c / CPR) * LD + (c % CPR) * 8) = dor[i];
			}
		}
		if (tid < BQ) {
			sLse(buf)[tid] = lse_r;
			sDelta(buf)[tid] = delta_r;
		}
	};

	if (n_iter > 0) {
		load_regs(0);
		store_lds(0);
	}
	__syncthreads();

	for (int it = 0; it < n_iter; it++) {
		const int cur = it & 1;
		const bool more = (it + 1) < n_iter;
		if (more) load_regs(it + 1);
		const bf16_t *qp_, *dop_;
		const float *lp_, *dp_;
		int h, q0;
		tile_ptrs(it, qp_, dop_, lp_, dp_, h, q0);
		// causal: this wave's keys all lie after every query of the tile -> P = 0
		const bool active = !CAUSAL || (wkey0 <= q0 + BQ - 1);

		f32x16 ds;  // becomes dS[q][key] (scaled), lane <-> key, rows <-> queries
#pragma unroll
		for (int r = 0; r < 16; r++) ds[r] = 0.f;
		if (active) {
			// S[q][key] = Q K^T ; dP[q][key] = dO V^T
			f32x16 s, dp;
#pragma unroll
			for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.f;
#pragma unroll
			for (int ks = 0; ks < KSTEPS; ks++) {
				bf16x8 qf = frag_rows<LD>(sQ(cur), 0, ks * 16, lane);
				s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf, kf[ks], s, 0, 0, 0);
			}
#pragma unroll
			for (int ks = 0; ks < KSTEPS; ks++) {
				bf16x8 dof = frag_rows<LD>(sdO(cur), 0, ks * 16, lane);
				dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dof, vf[ks], dp, 0, 0, 0);
			}
			float p[16];
			const int key = wkey0 + kl;
#pragma unroll
			for (int r4 = 0; r4 < 4; r4++) {
				const f32x4 l4 = *reinterpret_cast<const f32x4*>(&sLse(cur)[r4 * 8 + 4 * g]);
				const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sDelta(cur)[r4 * 8 + 4 * g]);
#pragma unroll
				for (int t = 0; t < 4; t++) {
					const int r = r4 * 4 + t;
					float pr = exp2f(s[r] * sc - l4[t]);
					if (CAUSAL) {
						const int qpos = q0 + r4 * 8 + 4 * g + t;
						if (key > qpos) pr = 0.f;
					}
					p[r] = pr;
					ds[r] = pr * (dp[r] - d4[t]) * a.scale;
				}
			}
			// dV^T[d][key] += dO^T[d][q] P[q][key] ; dK^T[d][key] += Q^T[d][q] dS[q][key]
#pragma unroll
			for (int u = 0; u < 2; u++) {
				const bf16x8 pf = pack8(p + u * 8);
				float dsv[8];
#pragma unroll
				for (int t = 0; t < 8; t++) dsv[t] = ds[u * 8 + t];
				const bf16x8 dsf = pack8(dsv);
#pragma unroll
				for (int dt = 0; dt < DT; dt++) {
					bf16x8 dot = frag_cols_acc_order<LD>(sdO(cur), u * 16, dt * 32, lane);
					acc_dv[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dot, pf, acc_dv[dt], 0, 0, 0);
					bf16x8 qt = frag_cols_acc_order<LD>(sQ(cur), u * 16, dt * 32, lane);
					acc_dk[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qt, dsf, acc_dk[dt], 0, 0, 0);
				}
			}
		}
		// dS to LDS as [q][key] (inactive waves publish zeros)
#pragma unroll
		for (int r = 0; r < 16; r++) {
			const int qrow = (r >> 2) * 8 + 4 * g + (r & 3);
			sdS[qrow * LDS_ + wave * 32 + kl] = (bf16_t)ds[r];
		}
		__syncthreads();
		// dQ[q][d-slice] = sum over the 128 keys of dS[q][key] K[key][d]; wave w owns d-slices
		// w, w+4, ... (32 columns each)
		for (int dt = wave; dt < DT; dt += 4) {
			f32x16 dq;
#pragma unroll
			for (int r = 0; r < 16; r++) dq[r] = 0.f;
#pragma unroll
			for (int ks = 0; ks < BKV / 16; ks++) {
				bf16x8 af = frag_rows<LDS_>(sdS, 0, ks * 16, lane);
				bf16x8 bfr = frag_cols<LD>(sKt, ks * 16, dt * 32, lane);
				dq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bfr, dq, 0, 0, 0);
			}
			float* dqp = a.dq_acc + (tok0 + q0) * ((int64_t)a.Hq * D) + h * D + dt * 32 + kl;
#pragma unroll
			for (int r = 0; r < 16; r++) {
				const int qrow = (r >> 2) * 8 + 4 * g + (r & 3);
				unsafeAtomicAdd(dqp + (int64_t)qrow * a.Hq * D, dq[r]);
			}
		}
		if (more) store_lds(cur ^ 1);
		__syncthreads();
	}

	// dK^T / dV^T accumulators: register r <-> d = dt*32 + (r/4)*8 + 4g + r%4, lane <-> key
	bf16_t* dkp = a.dk + (tok0 + wkey0 + kl) * a.lddk + hk * D;
	bf16_t* dvp = a.dv + (tok0 + wkey0 + kl) * a.lddv + hk * D;
#pragma unroll
	for (int dt = 0; dt < DT; dt++) {
#pragma unroll
		for (int r4 = 0; r4 < 4; r4++) {
			bf16x4 k4, v4;
#pragma unroll
			for (int t = 0; t < 4; t++) {
				k4[t] = (bf16_t)acc_dk[dt][r4 * 4 + t];
				v4[t] = (bf16_t)acc_dv[dt][r4 * 4 + t];
			}
			*reinterpret_cast<bf16x4*>(dkp + dt * 32 + r4 * 8 + 4 * g) = k4;
			*reinterpret_cast<bf16x4*>(dvp + dt * 32 + r4 * 8 + 4 * g) = v4;
		}
	}
}

// dq(bf16, row stride ld) = dq_acc(fp32, contiguous [T, cols])
__global__ __launch_bounds__(256) void cvt_f32_bf16_kernel(const float* __restrict__ src, bf16_t* __restrict__ dst, int64_t T,
                                                           int cols, int64_t ld) {
	const int cpr = cols / 4;
	const int64_t n = T * cpr;
	for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
		const int64_t row = i / cpr;
		const int c = (int)(i - row * cpr) * 4;
		const f32x4 v = *reinterpret_cast<const f32x4*>(src + row * cols + c);
		bf16x4 o;
#pragma unroll
		for (int t = 0; t < 4; t++) o[t] = (bf16_t)v[t];
		*reinterpret_cast<bf16x4*>(dst + row * ld + c) = o;
	}
}

__global__ __launch_bounds__(256) void fill_zero_kernel(f32x4* __restrict__ p, int64_t n4) {
	for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
		f32x4 z = {0.f, 0.f, 0.f, 0.f};
		p[i] = z;
	}
}

template <int D, bool CAUSAL>
int launch_fwd(const AttnArgs& a, dim3 grid, hipStream_t stream) {
	constexpr int smem = 2 * 2 * FwdTile<D>::TILE_BYTES;
	auto kern = attn_fwd_kernel<D, CAUSAL>;
	static bool attr_set = false;
	if (!attr_set) {
		ELF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
		attr_set = true;
	}
	hipLaunchKernelGGL(kern, grid, dim3(256), smem, stream, a);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

template <int D, bool CAUSAL>
int launch_bwd(const AttnBwdArgs& a, dim3 grid, hipStream_t stream) {
	constexpr int LD = AttnSmem<D>::LDT;
	constexpr int smem = (128 * LD + 4 * 32 * LD + 32 * (128 + 8)) * (int)sizeof(bf16_t) + 4 * 32 * (int)sizeof(float);
	auto kern = attn_bwd_kernel<D, CAUSAL>;
	static bool attr_set = false;
	if (!attr_set) {
		ELF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
		attr_set = true;
	}
	hipLaunchKernelGGL(kern, grid, dim3(256), smem, stream, a);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

}  // namespace attn

using namespace attn;

int attn_fwd(const void* q, const void* k, const void* v, void* o, void* lse, int64_t ldq, int64_t ldk, int64_t ldv,
             int64_t ldo, int B, int S, int Hq, int Hkv, int D, int causal, float scale, hipStream_t stream) {
	ELF_REQUIRE(q && k && v && o && lse, "attn_fwd: null pointer");
	ELF_REQUIRE(B > 0 && S > 0 && S % 128 == 0, "attn_fwd: sequence length must be a multiple of 128 (S=%d)", S);
	ELF_REQUIRE(Hkv > 0 && Hq % Hkv == 0, "attn_fwd: Hq must be a multiple of Hkv (Hq=%d Hkv=%d)", Hq, Hkv);
	ELF_REQUIRE(D == 64 || D == 128, "attn_fwd: head_dim must be 64 or 128 (D=%d)", D);
	ELF_REQUIRE(ldq % 8 == 0 && ldk % 8 == 0 && ldv % 8 == 0 && ldo % 8 == 0, "attn_fwd: strides must be multiples of 8");
	ELF_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0 && ((uintptr_t)o % 8) == 0,
	            "attn_fwd: misaligned pointer");
	ProfScope prof(PROF_ATTN_FWD, (causal ? 2.0 : 4.0) * B * Hq * (double)S * S * D, stream);
	AttnArgs a{(const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, (bf16_t*)o, (float*)lse, ldq, ldk, ldv, ldo, B, S, Hq, Hkv, scale};
	const dim3 grid((unsigned)((int64_t)B * Hq * (S / 128))), block(256);
	int rc;
	if (D == 128) rc = causal ? launch_fwd<128, true>(a, grid, stream) : launch_fwd<128, false>(a, grid, stream);
	else rc = causal ? launch_fwd<64, true>(a, grid, stream) : launch_fwd<64, false>(a, grid, stream);
	if (rc) return rc;
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

int64_t attn_bwd_workspace_bytes(int B, int S, int Hq, int D) {
	// fp32 dQ accumulator + delta
	return (int64_t)B * S * Hq * D * 4 + (int64_t)B * S * Hq * 4;
}

int attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dO, const void* lse, void* dq,
             void* dk, void* dv, void* workspace, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo,
             int64_t lddq, int64_t lddk, int64_t lddv, int B, int S, int Hq, int Hkv, int D, int causal, float scale,
             hipStream_t stream) {
	ELF_REQUIRE(q && k && v && o && dO && lse && dq && dk && dv && workspace, "attn_bwd: null pointer");
	ELF_REQUIRE(B > 0 && S > 0 && S % 128 == 0, "attn_bwd: sequence length must be a multiple of 128 (S=%d)", S);
	ELF_REQUIRE(Hkv > 0 && Hq % Hkv == 0, "attn_bwd: Hq must be a multiple of Hkv (Hq=%d Hkv=%d)", Hq, Hkv);
	ELF_REQUIRE(D == 64 || D == 128, "attn_bwd: head_dim must be 64 or 128 (D=%d)", D);
	ELF_REQUIRE(ldq % 8 == 0 && ldk % 8 == 0 && ldv % 8 == 0 && ldo % 8 == 0 && lddo % 8 == 0 && lddq % 8 == 0 &&
	                lddk % 8 == 0 && lddv % 8 == 0,
	            "attn_bwd: strides must be multiples of 8");
	ELF_REQUIRE(((uintptr_t)workspace % 16) == 0, "attn_bwd: misaligned workspace");
	ProfScope prof(PROF_ATTN_BWD, (causal ? 4.0 : 8.0) * B * Hq * (double)S * S * D, stream);
	const int64_t T = (int64_t)B * S;
	float* dq_acc = (float*)workspace;
	float* delta = dq_acc + T * Hq * D;
	// zero the dQ accumulator with a fill kernel (memset nodes misbehave under graph replay)
	hipLaunchKernelGGL(fill_zero_kernel, dim3(2048), dim3(256), 0, stream, (f32x4*)dq_acc, T * Hq * D / 4);
	hipLaunchKernelGGL(attn_delta_kernel, dim3((unsigned)((T * Hq + 3) / 4)), dim3(256), 0, stream, (const bf16_t*)dO,
	                   (const bf16_t*)o, delta, lddo, ldo, B, S, Hq, D);
	AttnBwdArgs a{(const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, (const bf16_t*)dO, (const float*)lse, delta, dq_acc,
	              (bf16_t*)dk, (bf16_t*)dv, ldq, ldk, ldv, lddo, lddk, lddv, B, S, Hq, Hkv, scale};
	const dim3 grid((unsigned)((int64_t)B * Hkv * (S / 128))), block(256);
	int rc;
	if (D == 128) rc = causal ? launch_bwd<128, true>(a, grid, stream) : launch_bwd<128, false>(a, grid, stream);
	else rc = causal ? launch_bwd<64, true>(a, grid, stream) : launch_bwd<64, false>(a, grid, stream);
	if (rc) return rc;
	const int64_t n4 = T * (Hq * D / 4);
	const int64_t blocks = (n4 + 255) / 256;
	hipLaunchKernelGGL(cvt_f32_bf16_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, stream, dq_acc,
	                   (bf16_t*)dq, T, Hq * D, lddq);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

}  // namespace elf
