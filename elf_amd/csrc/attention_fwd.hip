// Attention forward kernel (see attention_common.h for the layout conventions).
#include "attention_common.h"

namespace elf {
namespace attn {

// ------------------------------------------------------------------------------------------
// Forward.  K and V tiles (64 keys) are fetched straight into LDS (lds_dma.h) in a two-stage
// ring; tiles are unpadded (a wave instruction fills 1 KiB contiguously), so the 16-byte chunk
// index of every row is XOR-swizzled: for K (read along d, one row per lane) with a function
// of the row that spreads 16 consecutive rows over all 16 bank groups, for V (read with the
// transpose read: a half-wave takes 64 contiguous bytes from each of four consecutive rows) with
// a multiple of four chunks, so that the four rows land in four different 64-byte bank groups.
template <int D>
struct FwdTile {
	static constexpr int ROW_BYTES = D * 2;
	static constexpr int CPR = D / 8;                  // 16-byte chunks per row
	static constexpr int TILE_BYTES = 64 * ROW_BYTES;  // one operand, 64 keys
	static constexpr int RPI = 1024 / ROW_BYTES;       // rows per DMA wave instruction
	static constexpr int LOADS = TILE_BYTES / 1024 / 4;  // DMA instructions per wave and operand
	__device__ static __forceinline__ int k_swz(int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); }
	__device__ static __forceinline__ int v_swz(int row) { return D == 128 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); }
};

template <int D, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(AttnArgs a) {
	using TL = FwdTile<D>;
	constexpr int BQ = 128, BKV = 64, KT = BKV / 32;
	constexpr int KSTEPS = D / 16, DT = D / 32;
	constexpr int NF = D == 128 ? 8 : 4;  // LDS fragments in flight ahead of the MFMA that uses them
	constexpr int STAGE = 2 * TL::TILE_BYTES;
	extern __shared__ __attribute__((aligned(1024))) unsigned char smem_raw[];

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int g = lane >> 5, ql = lane & 31;
	const int nqt = a.S / BQ;
	// Workgroup order: query tile by query tile over all (batch, head) pairs; causal: the heaviest (last)
	// query tiles first, so that the workgroups that start last are the lightest ones (with the tiles
	// of one head after the other, the last head's heaviest tile started when most of the grid was done
	// and ran on alone for a third of the kernel's time).  Workgroups go to the 8 XCDs round-robin:
	// index j within a batch element is mapped to head (j % 8) * (Hq / 8) + j / 8, so that an XCD works
	// on a contiguous range of heads — the query heads that share a K/V head read it through one L2.
	const int nbh = a.B * a.Hq;
	const int qr = (int)(blockIdx.x / nbh), bj = (int)(blockIdx.x % nbh);
	const int qt = CAUSAL ? nqt - 1 - qr : qr;
	const int b = bj / a.Hq, j = bj % a.Hq;
	const int h = a.Hq % 8 == 0 ? (j & 7) * (a.Hq >> 3) + (j >> 3) : j;
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
	// One tile, in the LDS stage at byte offset `stage`.
	auto tile = [&](int j, int stage) __attribute__((always_inline)) {
		wait_vmcnt<0>();
		__syncthreads();  // tile j is in LDS for everyone; everyone is done with tile j-1
		if (j + 1 < n_kv) issue(j + 1);
		const int k0 = j * BKV;
		if (CAUSAL && k0 > q0 + 31) return;  // every key of the tile is in this wave's future
		const unsigned char* sK = smem_raw + stage;
		const unsigned char* sV = sK + TL::TILE_BYTES;

		// S^T[key][q] for the two 32-key halves.  Fragment i = (k step i / KT, key half i % KT): the two accumulators
		// alternate, and a fragment is read NF MFMAs before its use (left to itself the compiler reads each one
		// right before its MFMA, into one register quad, and every MFMA waits out an LDS round trip).
		f32x16 s[KT];
#pragma unroll
		for (int kt = 0; kt < KT; kt++)
#pragma unroll
			for (int r = 0; r < 16; r++) s[kt][r] = 0.f;
		{
			auto kread = [&](int i) __attribute__((always_inline)) {
				const int row = (i % KT) * 32 + ql, ks = i / KT;
				return *reinterpret_cast<const bf16x8*>(sK + row * TL::ROW_BYTES + (((2 * ks + g) ^ TL::k_swz(row)) << 4));
			};
			bf16x8 kf[NF];
#pragma unroll
			for (int i = 0; i < NF; i++) kf[i] = kread(i);
			__builtin_amdgcn_sched_barrier(0);
#pragma unroll
			for (int i = 0; i < KT * KSTEPS; i++) {
				s[i % KT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % NF], qf[i / KT], s[i % KT], 0, 0, 0);
				if (i + NF < KT * KSTEPS) kf[i % NF] = kread(i + NF);
				__builtin_amdgcn_sched_barrier(0);
			}
		}
		// causal mask only where the tile crosses the diagonal of this wave's queries
		if (CAUSAL && k0 + BKV - 1 > q0) {
#pragma unroll
			for (int kt = 0; kt < KT; kt++)
#pragma unroll
				for (int r = 0; r < 16; r++) {
					const int key = k0 + kt * 32 + (r >> 2) * 8 + 4 * g + (r & 3);
					if (key > qpos) s[kt][r] = -INFINITY;
				}
		}
		// The exponentials are taken against a reference point per query that follows the running maximum lazily: any
		// reference gives the same quotient, and as long as the weights stay moderate they are as exact in fp32 and
		// bf16 as those against the maximum.  A reference never lies above the running maximum, so nothing underflows
		// that would not against the maximum.  Every query sees key 0 in its first tile, so the reference is finite
		// from then on.
		f32x16 pr[KT];
		float psum = 0.f;
		auto weights = [&]() __attribute__((always_inline)) {
			psum = 0.f;
#pragma unroll
			for (int kt = 0; kt < KT; kt++)
#pragma unroll
				for (int r = 0; r < 16; r++) {
					const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][r], sc, -m_run));
					pr[kt][r] = p;
					psum += p;
				}
		};
		auto tile_max = [&]() __attribute__((always_inline)) {
			float mx = s[0][0];
#pragma unroll
			for (int kt = 0; kt < KT; kt++)
#pragma unroll
				for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[kt][r]);
			return fmaxf(mx, __shfl_xor(mx, 32, 64)) * sc;
		};
		auto move_reference = [&](float mx) __attribute__((always_inline)) {
			const float m_new = fmaxf(m_run, mx);
			const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
			l_run *= alpha;
#pragma unroll
			for (int i = 0; i < DT; i++)
#pragma unroll
				for (int r = 0; r < 16; r++) acc_o[i][r] *= alpha;
			m_run = m_new;
		};
		if constexpr (D == 128) {
			// The common tile computes no maximum at all: only when a lane's weights sum past LIMIT (or are not finite:
			// the first tile, whose reference is -inf) does the wave move the references to the running maxima, rescale
			// sums and output, and take the tile's exponentials again.
			constexpr float LIMIT = 0x1p20f;
			weights();
			if (__builtin_amdgcn_ballot_w64(!(psum < LIMIT)) != 0) {
				move_reference(tile_max());
				weights();
			}
		} else {
			// (with four waves on a SIMD there are no registers to keep the scores beside the weights) the reference is
			// the running maximum itself; output and sums are rescaled when some query of the wave raised it
			const float mx = tile_max();
			if (__builtin_amdgcn_ballot_w64(mx > m_run) != 0) move_reference(mx);
			weights();
		}
		l_run += psum;
		// O^T[d][q] += V^T[d][key] P^T[key][q].  Fragment i = (16-key group i / DT, 32-wide d block i % DT), read NF MFMAs
		// ahead like the K fragments above.
		{
			auto vread = [&](int i) __attribute__((always_inline)) {
				// keys {kk..kk+3} and {kk+8..kk+11}: the row order of the accumulator tile
				const int j16 = lane & 15, dt = i % DT;
				const int kk = (i / DT) * 16 + 4 * g + (j16 >> 2);
				const int c = (dt * 32 + 16 * (ql >> 4) + 4 * (j16 & 3)) >> 3;
				const unsigned char* p0 = sV + kk * TL::ROW_BYTES + ((c ^ TL::v_swz(kk)) << 4) + (j16 & 1) * 8;
				const unsigned char* p1 = sV + (kk + 8) * TL::ROW_BYTES + ((c ^ TL::v_swz(kk + 8)) << 4) + (j16 & 1) * 8;
				s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p0));
				s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p1));
				return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
			};
			bf16x8 vf[NF];
#pragma unroll
			for (int i = 0; i < NF; i++) vf[i] = vread(i);
			bf16x8 pf;
#pragma unroll
			for (int i = 0; i < 2 * KT * DT; i++) {
				if (i % DT == 0) {
					float pv[8];
#pragma unroll
					for (int t = 0; t < 8; t++) pv[t] = pr[i / DT / 2][(i / DT % 2) * 8 + t];
					pf = pack8(pv);
				}
				__builtin_amdgcn_sched_barrier(0);
				acc_o[i % DT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[i % NF], pf, acc_o[i % DT], 0, 0, 0);
				if (i + NF < 2 * KT * DT) vf[i % NF] = vread(i + NF);
			}
			__builtin_amdgcn_sched_barrier(0);
		}
	};
	if constexpr (D == 128) {
		// tiles in pairs (their number is even: 128 queries, sequences of a multiple of 128, 64-key tiles): the stage is a
		// constant in each copy of the body and travels in the LDS instructions' offset fields instead of being added to
		// every address
		for (int j = 0; j < n_kv; j += 2) {
			tile(j, 0);
			tile(j + 1, STAGE);
		}
	} else {
		// (the two copies cost the registers that keep four waves on a SIMD)
		for (int j = 0; j < n_kv; j++) tile(j, (j & 1) * STAGE);
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

template <int D, bool CAUSAL>
int launch_fwd(const AttnArgs& a, dim3 grid, hipStream_t stream) {
	constexpr int smem = 2 * 2 * FwdTile<D>::TILE_BYTES;
	auto kern = attn_fwd_kernel<D, CAUSAL>;
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

}  // namespace elf
