// bf16 MFMA GEMM for gfx950 (CDNA4): C[M,N] (+)= sum_k A(m,k) * B(n,k), fp32 accumulation.
//
// The three contractions of a linear layer under the split backward map onto one kernel:
//   forward  Y  = X  . W^T   A = X  [M,K] k-contiguous ("R"), B = W  [N,K] k-contiguous ("R")
//   dX       dX = dY . W     A = dY [M,K] k-contiguous ("R"), B = W  [K,N] n-contiguous ("T")
//   dW       dW += dY^T . X  A = dY [K,M] m-contiguous ("T"), B = X  [K,N] n-contiguous ("T")
// (reference semantics: elf/zb_utils.py:20 forward, :34-37 dX, :235-244 dW accumulate).
//
// Tiling: one workgroup owns a BM x BN tile of C and walks K in steps of 64.  Global loads
// are 16 B per lane into registers, then written to a double-buffered LDS tile, so the loads
// of step k+1 are in flight while the MFMAs of step k run.  "R" operands are stored [row][k]
// with 8 elements of padding and read with ds_read_b128; "T" operands are stored [k][row] as
// they sit in memory and read with ds_read_b64_tr_b16, the LDS transpose read of gfx950, so
// no operand is ever transposed through HBM.  Each wave owns a (BM/WR) x (BN/WC) sub-tile
// built from v_mfma_f32_32x32x16_bf16.
#include <atomic>

#include "common.h"
#include "kernels.h"
#include "lds_dma.h"

namespace elf {

constexpr int BK = 64;
// turn counters of split tiles (see gemm_kernel)
constexpr int TURN_RS_SLOTS = 4096;
static __device__ uint32_t turn_rs[TURN_RS_SLOTS];
// polls of ~1 us: about a millisecond, several times a predecessor's epilogue; a workgroup that uses them up is counted
constexpr int TURN_RS_SPIN_LIMIT = 1 << 10;
static __device__ unsigned int turn_rs_giveups;

// One sequence of tags for every launch of every GEMM kernel that splits tiles: a counter value left behind by any
// earlier launch then never equals a value a later launch waits for.
uint32_t next_turn_tag() {
	static std::atomic<uint32_t> launch_tag{0};
	return (launch_tag.fetch_add(1) % 0xFFFFFFu) + 1;
}
int dma_turn_giveups(uint64_t* out);  // gemm_dma.hip
// Split-K workgroups / waves (both GEMM kernel families, this device) that stopped waiting for their turn and added out
// of turn since the library was loaded: the sums are right, only bit-reproducibility lapsed for those launches.
int gemm_turn_giveups(uint64_t* out) {
	unsigned int n = 0;
	uint64_t d = 0;
	ELF_CHECK_HIP(hipMemcpyFromSymbol(&n, HIP_SYMBOL(turn_rs_giveups), sizeof(n)));
	if (int rc = dma_turn_giveups(&d)) return rc;
	*out = d + n;
	return 0;
}
constexpr int PAD_R = 8;    // elements of padding per row of an "R" tile ([row][BK+8])
constexpr int PAD_T = 16;   // elements of padding per row of a "T" tile ([k][rows+16])

struct GemmArgs {
	const bf16_t* A;
	const bf16_t* B;
	void* C;
	const bf16_t* R;  // residual (EPI_BF16_RESID)
	int64_t lda, ldb, ldc, ldr;
	int M, N, K;
	int tiles_m, tiles_n;
	int k_splits;      // >1: split-K with fp32 atomics (EPI_F32_ACC only)
	uint32_t turn_tag; // split-K: this launch's tag in the turn counters, 0 = the splits add in any order
};

template <int ROWS, bool T>
struct TileShape {
	static constexpr int LD = T ? (ROWS + PAD_T) : (BK + PAD_R);
	static constexpr int ELEMS = T ? BK * LD : ROWS * LD;
};

// Global -> register staging of one operand tile. NT threads cooperatively fetch ROWS x BK
// (or BK x ROWS) elements as 16-byte chunks.
template <int ROWS, bool T, int NT>
struct TileLoader {
	static constexpr int CHUNKS = ROWS * BK / 8 / NT;  // 16-byte chunks per thread
	static constexpr int CPR = T ? ROWS / 8 : BK / 8;  // chunks per stored row
	static constexpr int RPP = NT / CPR;               // stored rows per pass
	static_assert(CHUNKS >= 1 && (NT % CPR) == 0, "tile/threads mismatch");

	u32x4 regs[CHUNKS];

	// p points at the tile origin: for R, &A[row0][k0]; for T, &A[k0][row0].
	__device__ __forceinline__ void load(const bf16_t* __restrict__ p, int64_t ld, int tid) {
		const int c = tid % CPR, r = tid / CPR;
#pragma unroll
		for (int i = 0; i < CHUNKS; i++) {
			const bf16_t* q = p + (int64_t)(r + i * RPP) * ld + c * 8;
			regs[i] = *reinterpret_cast<const u32x4*>(q);
		}
	}
	__device__ __forceinline__ void store(bf16_t* lds, int tid) const {
		constexpr int LD = TileShape<ROWS, T>::LD;
		const int c = tid % CPR, r = tid / CPR;
#pragma unroll
		for (int i = 0; i < CHUNKS; i++) {
			*reinterpret_cast<u32x4*>(lds + (r + i * RPP) * LD + c * 8) = regs[i];
		}
	}
};

// One MFMA operand fragment (8 consecutive k for row lane%32, k-group lane/32) for the
// 32-row slab starting at `row`, k-step `ks` (16 wide).
template <int ROWS, bool T>
__device__ __forceinline__ bf16x8 read_frag(const bf16_t* lds, int row, int ks, int lane) {
	constexpr int LD = TileShape<ROWS, T>::LD;
	if constexpr (!T) {
		const bf16_t* p = lds + (row + (lane & 31)) * LD + ks * 16 + 8 * (lane >> 5);
		return *reinterpret_cast<const bf16x8*>(p);
	} else {
		// Transposing read: inside each group of 16 lanes, lane j supplies the address of the
		// 8-byte chunk (k = k0 + j/4, rows 4*(j%4)..+3) and receives rows (j) of k0..k0+3.
		const int j = lane & 15;
		const int rbase = row + 16 * ((lane & 31) >> 4) + 4 * (j & 3);
		const int k0 = ks * 16 + 8 * (lane >> 5) + (j >> 2);
		const bf16_t* p0 = lds + k0 * LD + rbase;
		const bf16_t* p1 = p0 + 4 * LD;
		s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p0));
		s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p1));
		s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
		return __builtin_bit_cast(bf16x8, v);
	}
}

template <int BM, int BN, int WR, int WC, bool AT, bool BT, int EPI>
__global__ __launch_bounds__(WR* WC * 64) void gemm_kernel(GemmArgs g) {
	constexpr int NT = WR * WC * 64;
	constexpr int WM = BM / WR, WN = BN / WC;
	constexpr int TM = WM / 32, TN = WN / 32;
	constexpr int A_ELEMS = TileShape<BM, AT>::ELEMS;
	constexpr int B_ELEMS = TileShape<BN, BT>::ELEMS;

	extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
	// Buffers are addressed as smem + integer offset (never through an array of pointers) so that
	// every access stays a DS instruction; a generic pointer would turn them into FLAT accesses
	// that also wait on the global-load counter.
	bf16_t* const smem = reinterpret_cast<bf16_t*>(smem_raw);
	constexpr int STAGE = A_ELEMS + B_ELEMS;

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = tid >> 6;
	const int wr = wave / WC, wc = wave % WC;

	// Tile assignment. Workgroups are dealt round-robin to the 8 XCDs, each with a private
	// L2: give every XCD a contiguous run of tile ids, then walk tiles in column-major
	// groups of GROUP_M tile rows so that a group shares its B panel and A rows in L2.
	int pid = blockIdx.x;
	const int ntiles = g.tiles_m * g.tiles_n;
	int ksplit = 0;
	if (g.k_splits > 1) {
		ksplit = pid / ntiles;
		pid = pid % ntiles;
	}
	if ((ntiles & 7) == 0) pid = (pid & 7) * (ntiles >> 3) + (pid >> 3);
	constexpr int GROUP_M = 8;
	const int per_group = GROUP_M * g.tiles_n;
	const int group = pid / per_group;
	const int first_m = group * GROUP_M;
	const int gsz = min(g.tiles_m - first_m, GROUP_M);
	const int tm_idx = first_m + (pid % per_group) % gsz;
	const int tn_idx = (pid % per_group) / gsz;
	const int m0 = tm_idx * BM, n0 = tn_idx * BN;

	const int nk_total = g.K / BK;
	const int nk_per = (nk_total + g.k_splits - 1) / g.k_splits;
	const int kt_begin = ksplit * nk_per;
	const int kt_end = min(nk_total, kt_begin + nk_per);
	// Split tiles add in turn (bit-reproducible sums): split s starts its atomics when turn_rs[tile] holds this
	// launch's tag with count s and publishes s + 1 when they have been performed.  Splits of lower index are
	// dispatched first, so the one waited for is running or done; the wait is bounded, and a workgroup that gives
	// up adds out of turn (the right sum, only its rounding may differ).
	uint32_t* const my_turn = turn_rs + (((uint32_t)pid + g.turn_tag * 977u) % (uint32_t)TURN_RS_SLOTS);
	const uint32_t turn_want = (g.turn_tag << 8) | (uint32_t)ksplit;
	// The poll and the publication are relaxed: the adds are atomics performed at the memory side, so what has to
	// be known is only that they have been performed - every lane awaits the acknowledgement of its own
	// (vmcnt(0)) before the workgroup barrier that precedes the publication.
	auto take_turn = [&]() {
		if (g.k_splits > 1 && g.turn_tag) {
			if (tid == 0 && ksplit > 0) {
				int spin = 0;
				for (; spin < TURN_RS_SPIN_LIMIT && __hip_atomic_load(my_turn, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != turn_want; spin++)
					__builtin_amdgcn_s_sleep(8);
				if (spin >= TURN_RS_SPIN_LIMIT) atomicAdd(&turn_rs_giveups, 1u);
			}
			__syncthreads();
		}
	};
	auto pass_turn = [&]() {
		if (g.k_splits > 1 && g.turn_tag) {
			wait_vmcnt<0>();
			__syncthreads();
			if (tid == 0) __hip_atomic_store(my_turn, turn_want + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		}
	};
	if (kt_begin >= kt_end) {
		take_turn();
		pass_turn();
		return;
	}

	const bf16_t* Ap = AT ? g.A + (int64_t)kt_begin * BK * g.lda + m0 : g.A + (int64_t)m0 * g.lda + (int64_t)kt_begin * BK;
	const bf16_t* Bp = BT ? g.B + (int64_t)kt_begin * BK * g.ldb + n0 : g.B + (int64_t)n0 * g.ldb + (int64_t)kt_begin * BK;
	const int64_t a_step = AT ? (int64_t)BK * g.lda : BK;
	const int64_t b_step = BT ? (int64_t)BK * g.ldb : BK;

	TileLoader<BM, AT, NT> la;
	TileLoader<BN, BT, NT> lb;

	f32x16 acc[TM][TN];
#pragma unroll
	for (int i = 0; i < TM; i++)
#pragma unroll
		for (int j = 0; j < TN; j++)
#pragma unroll
			for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

	la.load(Ap, g.lda, tid);
	lb.load(Bp, g.ldb, tid);
	la.store(smem, tid);
	lb.store(smem + A_ELEMS, tid);
	__syncthreads();

	for (int kt = kt_begin; kt < kt_end; kt++) {
		const int cur = (kt - kt_begin) & 1;
		const bool more = (kt + 1) < kt_end;
		if (more) {
			Ap += a_step;
			Bp += b_step;
			la.load(Ap, g.lda, tid);
			lb.load(Bp, g.ldb, tid);
		}
		const bf16_t* a_s = smem + cur * STAGE;
		const bf16_t* b_s = a_s + A_ELEMS;
#pragma unroll
		for (int ks = 0; ks < BK / 16; ks++) {
			bf16x8 af[TM], bfr[TN];
#pragma unroll
			for (int i = 0; i < TM; i++) af[i] = read_frag<BM, AT>(a_s, wr * WM + i * 32, ks, lane);
#pragma unroll
			for (int j = 0; j < TN; j++) bfr[j] = read_frag<BN, BT>(b_s, wc * WN + j * 32, ks, lane);
#pragma unroll
			for (int i = 0; i < TM; i++)
#pragma unroll
				for (int j = 0; j < TN; j++)
					acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
		}
		if (more) {
			la.store(smem + (cur ^ 1) * STAGE, tid);
			lb.store(smem + (cur ^ 1) * STAGE + A_ELEMS, tid);
		}
		__syncthreads();
	}

	// Epilogue. Accumulator register r of a 32x32 tile holds row (r/4)*8 + (lane/32)*4 + r%4,
	// column lane%32: lanes 0..31 cover 32 consecutive columns of one row.
	if constexpr (EPI == EPI_F32_ACC) take_turn();
	const int col_l = lane & 31;
	const int row_l = (lane >> 5) * 4;
#pragma unroll
	for (int i = 0; i < TM; i++) {
#pragma unroll
		for (int j = 0; j < TN; j++) {
			const int col = n0 + wc * WN + j * 32 + col_l;
#pragma unroll
			for (int r = 0; r < 16; r++) {
				const int row = m0 + wr * WM + i * 32 + (r >> 2) * 8 + row_l + (r & 3);
				const float v = acc[i][j][r];
				if constexpr (EPI == EPI_BF16) {
					reinterpret_cast<bf16_t*>(g.C)[(int64_t)row * g.ldc + col] = f2bf(v);
				} else if constexpr (EPI == EPI_BF16_RESID) {
					const float res = bf2f(g.R[(int64_t)row * g.ldr + col]);
					reinterpret_cast<bf16_t*>(g.C)[(int64_t)row * g.ldc + col] = f2bf(v + res);
				} else if constexpr (EPI == EPI_F32_ACC) {
					float* c = reinterpret_cast<float*>(g.C) + (int64_t)row * g.ldc + col;
					if (g.k_splits > 1) {
						unsafeAtomicAdd(c, v);
					} else {
						*c += v;
					}
				} else {
					reinterpret_cast<float*>(g.C)[(int64_t)row * g.ldc + col] = v;
				}
			}
		}
	}
	if constexpr (EPI == EPI_F32_ACC) pass_turn();
}

template <int BM, int BN, int WR, int WC, bool AT, bool BT, int EPI>
static int launch_cfg(const GemmArgs& g, hipStream_t stream) {
	constexpr int smem = 2 * (TileShape<BM, AT>::ELEMS + TileShape<BN, BT>::ELEMS) * (int)sizeof(bf16_t);
	auto kern = gemm_kernel<BM, BN, WR, WC, AT, BT, EPI>;
	static bool attr_set = false;
	if (!attr_set) {
		ELF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
		                                  hipFuncAttributeMaxDynamicSharedMemorySize, smem));
		attr_set = true;
	}
	GemmArgs a = g;
	a.tiles_m = g.M / BM;
	a.tiles_n = g.N / BN;
	a.turn_tag = EPI == EPI_F32_ACC && a.k_splits > 1 && a.tiles_m * a.tiles_n <= TURN_RS_SLOTS ? next_turn_tag() : 0;
	const int grid = a.tiles_m * a.tiles_n * a.k_splits;
	ELF_LAUNCH(kern, dim3(grid), dim3(WR * WC * 64), smem, stream, a);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

template <bool AT, bool BT, int EPI>
static int launch_layout(GemmArgs& g, int tile_cfg, hipStream_t stream) {
	const int M = g.M, N = g.N;
	// Tile choice: the 256x256 tile (8 waves, 128x64 each) has the best MFMA : HBM ratio;
	// smaller tiles keep all 256 CUs busy when the output is small.
	int cfg = tile_cfg;
	if (cfg <= 0) {
		const int64_t t256 = (M % 256 == 0 && N % 256 == 0) ? (int64_t)(M / 256) * (N / 256) : 0;
		const int64_t t128 = (M % 128 == 0 && N % 128 == 0) ? (int64_t)(M / 128) * (N / 128) : 0;
		if (t256 >= 256) cfg = 1;
		else if (t128 >= 128) cfg = 2;
		else cfg = 3;
	}
	if (EPI == EPI_F32_ACC && g.k_splits <= 0) {
		// Split K when the weight-gradient tile count cannot fill the chip.
		int bm = cfg == 1 ? 256 : cfg == 2 ? 128 : 64;
		int64_t tiles = (int64_t)(M / bm) * (N / bm);
		int ks = 1;
		while (tiles * ks < 256 && (g.K / BK) / (ks * 2) >= 8 && ks < 16) ks *= 2;
		g.k_splits = ks;
	}
	if (g.k_splits <= 0 || EPI != EPI_F32_ACC) g.k_splits = 1;
	switch (cfg) {
		case 1:
			ELF_REQUIRE(M % 256 == 0 && N % 256 == 0, "gemm: tile 256 needs M,N multiples of 256 (M=%d N=%d)", M, N);
			return launch_cfg<256, 256, 2, 4, AT, BT, EPI>(g, stream);
		case 2:
			ELF_REQUIRE(M % 128 == 0 && N % 128 == 0, "gemm: tile 128 needs M,N multiples of 128 (M=%d N=%d)", M, N);
			return launch_cfg<128, 128, 2, 2, AT, BT, EPI>(g, stream);
		case 3:
			ELF_REQUIRE(M % 64 == 0 && N % 64 == 0, "gemm: M and N must be multiples of 64 (M=%d N=%d)", M, N);
			return launch_cfg<64, 64, 2, 2, AT, BT, EPI>(g, stream);
		case 5:
			ELF_REQUIRE(M % 256 == 0 && N % 128 == 0, "gemm: tile 256x128 needs M%%256==0, N%%128==0 (M=%d N=%d)", M, N);
			return launch_cfg<256, 128, 2, 2, AT, BT, EPI>(g, stream);
		default:
			set_error("gemm: unknown tile config %d", cfg);
			return -1;
	}
}

template <bool AT, bool BT>
static int launch_epi(GemmArgs& g, int epi, int tile_cfg, hipStream_t stream) {
	switch (epi) {
		case EPI_BF16: return launch_layout<AT, BT, EPI_BF16>(g, tile_cfg, stream);
		case EPI_BF16_RESID: return launch_layout<AT, BT, EPI_BF16_RESID>(g, tile_cfg, stream);
		case EPI_F32_ACC: return launch_layout<AT, BT, EPI_F32_ACC>(g, tile_cfg, stream);
		case EPI_F32_STORE: return launch_layout<AT, BT, EPI_F32_STORE>(g, tile_cfg, stream);
		default: set_error("gemm: unknown epilogue %d", epi); return -1;
	}
}

// Which direct-to-LDS tile a forward / input-gradient product runs on: 256 rows when 192 or more such tiles fill
// the chip, else 128 rows (k-contiguous A) when 128 or more of those do, else neither (0).  A choice by estimated
// rounds of workgroups x time per workgroup - 128-row tiles where the 256-row ones leave a mostly empty last round,
// e.g. 8192 x 2304 x 768 - wins 4-11 % back to back on operands that stay cached and loses 3.6 % inside the
// GPT-2-small stream, where they are cold and the narrower tile fetches B twice as often: not used.
static int dma_tile_rows(bool a_t, int M, int N, int K) {
	if (N % 256 != 0 || K % 64 != 0) return 0;
	if (M % 256 == 0 && (int64_t)(M / 256) * (N / 256) >= 192) return 256;
	if (M % 128 == 0 && !a_t && (int64_t)(M / 128) * (N / 256) >= 128) return 128;
	return 0;
}

// K split of a weight gradient on 256x256 direct-to-LDS tiles when the caller leaves it open: *k_splits ways for the last
// *tail_tiles tiles (-1: all of them).
static void dw_split_plan(int M, int N, int K, int* k_splits, int* tail_tiles) {
	const int64_t tiles = (int64_t)(M / 256) * (N / 256);
	const int nk = K / 64;
	*k_splits = 1;
	*tail_tiles = -1;
	if (tiles < 256) {
		// too few tiles for the chip: split them all, down to 32 slices per workgroup (shorter
		// ranges pay more in pipeline fill and atomics than the extra workgroups bring)
		while (tiles * *k_splits * 2 <= 256 && nk / (*k_splits * 2) >= 32 && *k_splits < 16) *k_splits *= 2;
	} else if (const int rem = (int)(tiles % 256); rem != 0 && rem <= 128) {
		// the last round of workgroups would leave at least half of the CUs idle: split just those
		// tiles so that they fill it with proportionally shorter workgroups
		*k_splits = rem <= 64 ? 4 : 2;
		*tail_tiles = rem;
		if (nk / *k_splits < 16) *k_splits = 1;
	}
}

int gemm_bf16(int a_t, int b_t, int M, int N, int K, const void* A, int64_t lda, const void* B, int64_t ldb,
              void* C, int64_t ldc, int epi, const void* R, int64_t ldr, int tile_cfg, int k_splits,
              hipStream_t stream) {
	ELF_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: empty problem M=%d N=%d K=%d", M, N, K);
	ELF_REQUIRE(K % BK == 0, "gemm: K must be a multiple of %d (K=%d)", BK, K);
	ELF_REQUIRE(A && B && C, "gemm: null operand");
	ELF_REQUIRE(lda % 8 == 0 && ldb % 8 == 0, "gemm: leading dimensions must be multiples of 8 elements");
	ELF_REQUIRE(((uintptr_t)A % 16) == 0 && ((uintptr_t)B % 16) == 0, "gemm: operands must be 16-byte aligned");
	ELF_REQUIRE(lda >= (a_t ? M : K) && ldb >= (b_t ? N : K) && ldc >= N, "gemm: leading dimension too small");
	// ldr == 0: R is one row of N values added to every row of C (the bias of a linear layer)
	ELF_REQUIRE(epi != EPI_BF16_RESID || (R != nullptr && (ldr >= N || ldr == 0)), "gemm: residual epilogue needs R");
	// the turn counters of split tiles hold the split index in 8 bits next to the launch tag
	ELF_REQUIRE(k_splits <= 255, "gemm: k_splits must be at most 255 (got %d)", k_splits);
	ProfScope prof(PROF_GEMM, 2.0 * M * N * K, stream);
	GemmArgs g;
	g.A = (const bf16_t*)A;
	g.B = (const bf16_t*)B;
	g.C = C;
	g.R = (const bf16_t*)R;
	g.lda = lda;
	g.ldb = ldb;
	g.ldc = ldc;
	g.ldr = ldr;
	g.M = M;
	g.N = N;
	g.K = K;
	g.tiles_m = g.tiles_n = 0;
	g.k_splits = k_splits;
	// small weight gradients (12..128 tiles of 128x256, e.g. 2304x768 or 2048x2048 at K = 8192): 128x256 tiles with K
	// split so that the workgroups just fill the chip once - 7-28 % faster than 256x256 tiles split further.  A split
	// keeps at least 32 K slices, 16 where the tiles are so few (768x768: 18) that half of the chip would idle otherwise
	if (tile_cfg <= 0 && epi == EPI_F32_ACC && a_t && b_t && k_splits <= 0 && M % 128 == 0 && N % 256 == 0 && K >= 4096) {
		const int64_t tiles = (int64_t)(M / 128) * (N / 256);
		if (tiles >= 12 && tiles <= 128) {
			int ks = (int)(256 / tiles);
			const int min_slices = tiles < 24 ? 16 : 32;
			if (ks > K / 64 / min_slices) ks = K / 64 / min_slices;
			return gemm_bf16_dma(a_t, b_t, M, N, K, A, lda, B, ldb, C, ldc, epi, R, ldr, ks < 1 ? 1 : ks, -1, 128, stream);
		}
	}
	// Tile choice when the caller leaves it open: the direct-to-LDS 256x256 kernel whenever its
	// tiles can fill the chip, the register-staged kernels (smaller tiles) otherwise.
	if (tile_cfg <= 0 && epi == EPI_F32_ACC && M % 256 == 0 && N % 256 == 0 && K % 64 == 0) {
		// weight gradients (long K, fp32 accumulate) also when the tiles are few: K is split instead
		const int64_t tiles = (int64_t)(M / 256) * (N / 256);
		if (tiles >= 192 || (tiles >= 24 && K >= 4096)) tile_cfg = 7;
	}
	if (tile_cfg <= 0 && epi != EPI_F32_ACC) {
		const int rows = dma_tile_rows(a_t, M, N, K);
		tile_cfg = rows == 256 ? 7 : rows == 128 ? 8 : tile_cfg;
	}
	if (tile_cfg == 7) {
		int tail_tiles = -1;  // an explicit k_splits splits every tile
		if (epi == EPI_F32_ACC && k_splits <= 0) dw_split_plan(M, N, K, &k_splits, &tail_tiles);
		return gemm_bf16_dma(a_t, b_t, M, N, K, A, lda, B, ldb, C, ldc, epi, R, ldr, k_splits, tail_tiles, 256, stream);
	}
	if (tile_cfg == 8) return gemm_bf16_dma(a_t, b_t, M, N, K, A, lda, B, ldb, C, ldc, epi, R, ldr, epi == EPI_F32_ACC && k_splits > 1 ? k_splits : 1, -1, 128, stream);
	if (!a_t && !b_t) return launch_epi<false, false>(g, epi, tile_cfg, stream);
	if (!a_t && b_t) return launch_epi<false, true>(g, epi, tile_cfg, stream);
	if (a_t && b_t) return launch_epi<true, true>(g, epi, tile_cfg, stream);
	set_error("gemm: layout A=T,B=R is not used by any stage contraction");
	return -1;
}

int gemm_act_bf16(int act, int M, int F, int K, const void* A, int64_t lda, const void* W, int64_t ldw, void* pre,
                  int64_t ldpre, void* out, int64_t ldout, hipStream_t stream) {
	ELF_REQUIRE(act == ACT_GELU || act == ACT_SWIGLU, "gemm_act: unknown activation %d", act);
	ELF_REQUIRE(M > 0 && F > 0 && K > 0 && A && W && pre && out, "gemm_act: empty problem or null operand");
	const int N = act == ACT_SWIGLU ? 2 * F : F;
	// the same tile choice as gemm_bf16 makes for this shape; the SwiGLU epilogue pairs 64 gate with 64 up
	// columns per wave, so a 256-column tile covers 128 outputs
	int bm = 0;
	if (act == ACT_SWIGLU && K % 64 == 0 && N % 256 == 0 && lda % 8 == 0 && ldw % 8 == 0 && ldpre >= N && ldout >= F && ldpre % 8 == 0 && ldout % 8 == 0 &&
	    ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)pre % 16) == 0 && ((uintptr_t)out % 16) == 0 && lda >= K && ldw >= K) {
		bm = dma_tile_rows(false, M, N, K);
	}
	if (bm) {
		ProfScope prof(PROF_GEMM, 2.0 * M * N * K, stream);
		return gemm_bf16_dma(0, 0, M, N, K, A, lda, W, ldw, pre, ldpre, EPI_BF16_SWIGLU, nullptr, 0, 1, 0,
		                     bm, stream, out, ldout);
	}
	ELF_REQUIRE(ldpre == N && ldout == F, "gemm_act: the unfused path needs dense outputs");
	if (int rc = gemm_bf16(0, 0, M, N, K, A, lda, W, ldw, pre, ldpre, EPI_BF16, nullptr, 0, 0, 0, stream)) return rc;
	return act == ACT_SWIGLU ? swiglu_fwd(pre, out, M, F, stream) : gelu_fwd(pre, out, (int64_t)M * F, stream);
}

int gemm_dw_final(int M, int N, int K, const void* dY, int64_t lddy, const void* X, int64_t ldx, float* acc, void* grad_bf16, float scale,
                  hipStream_t stream) {
	ELF_REQUIRE(M > 0 && N > 0 && K > 0 && dY && X && acc && grad_bf16, "gemm_dw_final: bad argument");
	const bool fused = M % 256 == 0 && N % 256 == 0 && K % 64 == 0 && (int64_t)(M / 256) * (N / 256) >= 192 && lddy % 8 == 0 && ldx % 8 == 0 && lddy >= M &&
	                   ldx >= N && ((uintptr_t)dY % 16) == 0 && ((uintptr_t)X % 16) == 0 && ((uintptr_t)acc % 16) == 0 && ((uintptr_t)grad_bf16 % 8) == 0;
	if (fused) {
		// the same K split as the plain weight gradient (same rounding); tiles shared by several workgroups along K have no
		// single epilogue that could scale them: a small kernel behind the GEMM does those
		int k_splits, tail_tiles;
		dw_split_plan(M, N, K, &k_splits, &tail_tiles);
		ProfScope prof(PROF_GEMM, 2.0 * M * N * K, stream);
		return gemm_bf16_dma(1, 1, M, N, K, dY, lddy, X, ldx, acc, N, EPI_F32_ACC_SCALE, nullptr, 0, k_splits, tail_tiles, 256, stream, grad_bf16, N, nullptr, 0, 0, 0, scale);
	}
	if (int rc = gemm_bf16(1, 1, M, N, K, dY, lddy, X, ldx, acc, N, EPI_F32_ACC, nullptr, 0, 0, 0, stream)) return rc;
	return scale_grads(acc, grad_bf16, (int64_t)M * N, scale, stream);
}

bool gemm_rope_fused(int M, int N, int K, int D) {
	if (!(M > 0 && N > 0 && K > 0 && K % 64 == 0 && N % 256 == 0 && (D == 64 || D == 128))) return false;
	// the tile choice gemm_bf16 makes for this shape
	return dma_tile_rows(false, M, N, K) != 0;
}

int gemm_rope_bf16(int M, int N, int K, const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, const void* cs,
                   int S, int n_rot_heads, int D, hipStream_t stream) {
	ELF_REQUIRE(M > 0 && N > 0 && K > 0 && A && W && C && cs, "gemm_rope: empty problem or null operand");
	ELF_REQUIRE(S > 0 && M % S == 0 && n_rot_heads >= 0 && (int64_t)n_rot_heads * D <= N, "gemm_rope: bad head layout (S=%d, heads=%d, D=%d, N=%d)", S, n_rot_heads, D, N);
	if (gemm_rope_fused(M, N, K, D) && lda % 8 == 0 && ldw % 8 == 0 && ldc % 8 == 0 && lda >= K && ldw >= K && ldc >= N && ((uintptr_t)A % 16) == 0 &&
	    ((uintptr_t)W % 16) == 0 && ((uintptr_t)C % 16) == 0 && ((uintptr_t)cs % 16) == 0) {
		// the rotation's arithmetic is not counted: the figure stays the GEMM's
		ProfScope prof(PROF_GEMM, 2.0 * M * N * K, stream);
		const int bm = dma_tile_rows(false, M, N, K);
		return gemm_bf16_dma(0, 0, M, N, K, A, lda, W, ldw, C, ldc, EPI_BF16_ROPE, nullptr, 0, 1, 0, bm, stream, nullptr, 0, cs, S, n_rot_heads * D, D);
	}
	if (int rc = gemm_bf16(0, 0, M, N, K, A, lda, W, ldw, C, ldc, EPI_BF16, nullptr, 0, 0, 0, stream)) return rc;
	return n_rot_heads ? rope_apply(C, cs, M, S, (int)ldc, n_rot_heads, D, 0, stream) : 0;
}

bool gemm_swiglu_bwd_fused(int M, int F, int K) {
	return M > 0 && F > 0 && K > 0 && M % 256 == 0 && F % 256 == 0 && K % 64 == 0 && (int64_t)(M / 256) * (F / 256) >= 192;
}

int gemm_swiglu_bwd_bf16(int M, int F, int K, const void* dY, int64_t lddy, const void* W, int64_t ldw, const void* gu,
                         int64_t ldgu, void* dgu, int64_t lddgu, void* scratch, hipStream_t stream, void* act, int64_t ldact) {
	ELF_REQUIRE(M > 0 && F > 0 && K > 0 && dY && W && gu && dgu, "gemm_swiglu_bwd: empty problem or null operand");
	if (gemm_swiglu_bwd_fused(M, F, K) && lddy >= K && ldw >= F && ldgu >= 2 * F && lddgu >= 2 * F && lddy % 8 == 0 && ldw % 8 == 0 && ldgu % 8 == 0 &&
	    lddgu % 8 == 0 && ((uintptr_t)dY % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)dgu % 16) == 0) {
		// the activation backward's arithmetic is not counted: the figure stays the GEMM's
		ProfScope prof(PROF_GEMM, 2.0 * M * F * K, stream);
		ELF_REQUIRE(!act || (ldact >= F && ldact % 8 == 0 && ((uintptr_t)act % 16) == 0), "gemm_swiglu_bwd: bad activation output");
		return gemm_bf16_dma(0, 1, M, F, K, dY, lddy, W, ldw, dgu, lddgu, EPI_BF16_SWIGLU_BWD, gu, ldgu, 1, 0, 256, stream, act, ldact);
	}
	ELF_REQUIRE(scratch, "gemm_swiglu_bwd: this shape needs a scratch buffer of M x F bf16");
	ELF_REQUIRE(ldgu == 2 * F && lddgu == 2 * F, "gemm_swiglu_bwd: the unfused path needs dense [M, 2F] buffers");
	if (int rc = gemm_bf16(0, 1, M, F, K, dY, lddy, W, ldw, scratch, F, EPI_BF16, nullptr, 0, 0, 0, stream)) return rc;
	ELF_REQUIRE(!act || ldact == F, "gemm_swiglu_bwd: the unfused path needs a dense activation output");
	return swiglu_bwd(scratch, gu, dgu, M, F, stream, act);
}

}  // namespace elf
