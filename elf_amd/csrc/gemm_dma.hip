// 256x256 (and 128x256) bf16 MFMA GEMM tile kernel with direct global->LDS loads, for gfx950.
//
// Same contraction and layouts as gemm_bf16.hip (C (+)= sum_k A(m,k) B(n,k); "R" operands are
// k-contiguous, "T" operands reduction-major), different data movement:
//   * global_load_lds_dwordx4 moves 16 B per lane straight into LDS (no VGPR staging, no
//     ds_write); two 64-wide K slices (2 x 64 KiB) alternate, the next slice being fetched while
//     the current one is multiplied.  64 bf16 = one full 128-byte cache line per operand row;
//   * a wave instruction fills 1 KiB of LDS contiguously, so tiles cannot be padded; bank
//     conflicts are avoided by an XOR swizzle of the 16-byte chunk index, applied on the global
//     side when choosing which chunk a lane fetches and undone when fragments are read;
//   * the contraction runs on v_mfma_f32_16x16x32_bf16; the 256x256 tile is worked by four waves with
//     128x128 sub-tiles (one per SIMD; k-contiguous A) or by eight with 64x128 sub-tiles (two per SIMD;
//     both operands reduction-major), the 128x256 tile by four with 64x128 sub-tiles.
// The DMA loads are issued through inline assembly: the compiler cannot see that they write
// LDS, which is what allows partial vmcnt waits (its own tracking would force vmcnt(0) before
// every LDS read).  Ordering is explicit: s_waitcnt vmcnt(n) for this wave's slice, then a
// workgroup barrier for the other waves' slices and for the reuse of the oldest stage.
#include "common.h"
#include "kernels.h"
#include "lds_dma.h"
#include <type_traits>

namespace elf {

namespace dma {

constexpr int BN = 256, BKS = 64;
constexpr int PERS_WORKGROUPS = 256;  // one per compute unit: the persistent kernel's grid
constexpr int B_BYTES = BN * BKS * 2;  // 32 KiB per stage

// Shape of one workgroup: NW waves arranged (NW / 2) x 2, each owning RT x 4 accumulator tiles of
// 32 x 32, so the workgroup tile is BM x 256 with BM = (NW / 2) * RT * 32.
template <int NW, int RT>
struct Shape {
	static constexpr int BM = (NW / 2) * RT * 32;
	// K slices in the LDS ring: two of 64 KiB for the 256-row tile; the 128-row tile's slices are 48 KiB and three of
	// them fit, so its loads run two slices ahead of their use (its shapes are the small ones, whose short K
	// ranges per workgroup leave a slice's loads less than a trip to memory when fetched one slice ahead)
	static constexpr int NST = BM == 128 ? 3 : 2;
	static constexpr int A_BYTES = BM * BKS * 2;
	static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
	// 1 KiB pieces (one wave instruction each) per wave, stage and operand
	static constexpr int LOADS_A = A_BYTES / 1024 / NW, LOADS_B = B_BYTES / 1024 / NW;
	static constexpr int LOADS_PER_STAGE = LOADS_A + LOADS_B;
	static_assert(LOADS_PER_STAGE % 2 == 0, "the loads of a slice are issued in two halves");
};

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), unrolled at compile time.
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
	if constexpr (N > 0) {
		static_for<N - 1>(f);
		f(std::integral_constant<int, N - 1>{});
	}
}

struct Args {
	const bf16_t* A;
	const bf16_t* B;
	void* C;
	const bf16_t* R;
	bf16_t* C2;  // SwiGLU epilogue: the activated output
	int64_t lda, ldb, ldc, ldr, ldc2;
	int M, N, K;
	int tiles_m, tiles_n;
	int k_splits;    // K is split this many ways (fp32 atomics epilogue) for the last tail_tiles tiles
	int tail_tiles;  // tiles_m * tiles_n for a uniform split, 0 when nothing is split
	int walk;        // 1: all XCDs share one band of 16 tile rows at a time (see the tile assignment)
	// EPI_BF16_ROPE: (cos, sin) table [rope_S, rope_D / 2], columns below rope_cols are rotated, heads are rope_D wide
	const float2* rope_cs;
	int rope_S, rope_cols, rope_D;
	// split tiles: this launch's tag in the turn counters (see turn[] below); 0 = the splits add in any order
	uint32_t turn_tag;
	float scale;  // EPI_F32_ACC_SCALE
	uint32_t turn_base;  // split tiles: the first of this problem's turn counters
};

// Turn counters of split tiles.  The workgroups that share a tile along K add their parts with fp32 atomics; to make
// the sum independent of the order in which they finish, split s only starts adding when turn[slot] holds this
// launch's tag with count s, and publishes count s + 1 when its adds have been performed.  The tag changes with every
// launch, so a value left by an earlier launch never matches and nothing has to be cleared.  Workgroups are
// dispatched in index order and the splits of a tile have consecutive indices, so the one a workgroup waits for is
// always running or done; the wait is bounded all the same, and a workgroup that gives up (counters shared with a
// concurrent launch on another stream) adds out of turn: still the right sum, only its rounding may differ.
// A counter covers one 32-row strip of one wave (up to 16 per tile), so a split starts on a strip as soon as its
// predecessor is through with that strip and the splits of a tile overlap except for about one strip.
constexpr int TURN_TILES = 4096, TURN_PER_TILE = 16;
static __device__ uint32_t turn[TURN_TILES * TURN_PER_TILE];
// polls of ~1 us each: about a millisecond in all, several times what a predecessor's epilogue takes (the splits of a
// tile start together and run equal K ranges).  One budget per wave for the whole epilogue; a wave that uses it up is
// counted in turn_giveups (gemm_turn_giveups() reads it) and adds out of turn from then on.
constexpr int TURN_SPIN_LIMIT = 1 << 10;
static __device__ unsigned int turn_giveups;
__device__ __forceinline__ void note_turn_giveup() { atomicAdd(&turn_giveups, 1u); }

// Byte offsets (relative to the tile origin of the current K slice) of the 16-byte chunks this
// lane fetches for one operand (< 2^31: 256 rows of at most 64 K elements).  "R" tiles are
// [256 rows][128 B], "T" tiles [64 k][512 B] ([64 k][256 B] for the 128 rows of A in a 128x256 tile); LDS chunk slot s of a row holds global chunk
// s ^ f(row) with f chosen so that the lanes of a fragment read spread over all banks: an "R"
// read takes one chunk from each of 32 rows (f = (row / 2) % 8), a "T" transpose read takes 64
// contiguous bytes from each of four k rows per half-wave (f = 4 * (k % 8): the four rows land in
// four different 64-byte bank groups; with 2 * (k % 8) pairs of rows shared one and the bank-conflict
// counter read half of the LDS-active cycles).
// chunk swizzle of reduction-major ("T") tiles as a function of the k row
// ROWS = 128 (a k row is 256 bytes, exactly one row of banks): the four k rows of a half-wave's transpose read
// are moved into four different 64-byte groups by (k % 4) * 4 chunks, rows k and k + 8 apart by two chunks
template <int ROWS = 256>
__device__ __forceinline__ int t_swz(int k) {
	return ((k & (ROWS == 256 ? 7 : 3)) << 2) ^ (((k >> 3) & 1) << 1);
}

// PAIRED (k-contiguous operands only): the 256 tile rows are not 256 consecutive operand rows but, for
// each 128-row half, 64 consecutive rows followed by the 64 rows `pair_rows` further down — the gate and
// up rows of the same 64 SwiGLU columns, which thereby land in one wave's accumulators.
template <bool T, int LPO, bool PAIRED = false, int ROWS = 256>
__device__ __forceinline__ void lane_offsets(int wave, int lane, int64_t ld, uint32_t (&off)[LPO], int64_t pair_rows = 0) {
#pragma unroll
	for (int i = 0; i < LPO; i++) {
		const int q = wave * LPO + i;  // which 1 KiB piece of the operand tile
		if constexpr (!T) {
			const int row = q * 8 + (lane >> 3), slot = lane & 7;
			const int64_t grow = PAIRED ? (row >> 7) * 64 + (row & 63) + ((row >> 6) & 1) * pair_rows : row;
			off[i] = (uint32_t)((grow * ld + ((slot ^ ((row >> 1) & 7)) << 3)) * 2);
		} else {
			constexpr int CPR = ROWS / 8;  // 16-byte chunks per k row; a 1 KiB piece holds 64 / CPR k rows
			const int krow = q * (64 / CPR) + lane / CPR, slot = lane % CPR;
			off[i] = (uint32_t)((krow * ld + ((slot ^ t_swz<ROWS>(krow)) << 3)) * 2);
		}
	}
}

// Operand fragment of v_mfma_f32_16x16x32_bf16 for the 16-row slab at `row0` and the k32 half `kq`
// of the current slice: lane l holds row (or column) row0 + l % 16 at k = 32 kq + 8 (l / 16) .. + 7.
// "R" tiles give it with one 16-byte read; "T" tiles with two transpose reads, each of which hands
// the 16 lanes of a group the 4 (k) x 16 (rows) block they address row-wise.
template <bool T, int ROWS = 256>
__device__ __forceinline__ bf16x8 frag(const unsigned char* base, int row0, int kq, int lane) {
	if constexpr (!T) {
		const int r = row0 + (lane & 15);
		const int c = (4 * kq + (lane >> 4)) ^ ((r >> 1) & 7);
		return *reinterpret_cast<const bf16x8*>(base + r * 128 + c * 16);
	} else {
		const int j = lane & 15;
		const int m = row0 + 4 * (j & 3);
		const int kk = kq * 32 + 8 * (lane >> 4) + (j >> 2);
		const int c0 = (m >> 3) ^ t_swz<ROWS>(kk);
		const int c1 = (m >> 3) ^ t_swz<ROWS>(kk + 4);
		const unsigned char* p0 = base + kk * (ROWS * 2) + c0 * 16 + (j & 1) * 8;
		const unsigned char* p1 = base + (kk + 4) * (ROWS * 2) + c1 * 16 + (j & 1) * 8;
		s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p0));
		s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(p1));
		return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
	}
}

// The two byte offsets (within the operand tile of stage 0, k32 half 0) that frag<true> reads for the
// 16-row slab at row0, and the fragment read from them for k32 half kq of the tile at `base`.
template <int ROWS = 256>
__device__ __forceinline__ void frag_t_offsets(int row0, int lane, uint32_t (&o)[2]) {
	const int j = lane & 15;
	const int m = row0 + 4 * (j & 3);
	const int kk = 8 * (lane >> 4) + (j >> 2);
	o[0] = (uint32_t)(kk * (ROWS * 2) + (((m >> 3) ^ t_swz<ROWS>(kk)) << 4) + (j & 1) * 8);
	o[1] = (uint32_t)((kk + 4) * (ROWS * 2) + (((m >> 3) ^ t_swz<ROWS>(kk + 4)) << 4) + (j & 1) * 8);
}
// o: LDS byte addresses; imm: a compile-time byte offset (stage and k32 half) that ends up in the
// instructions' offset fields.  t_swz only looks at k % 16, so the second k32 half of a tile lies 32 rows
// (of 2 * ROWS bytes) further on.
__device__ __forceinline__ bf16x8 frag_t_at(const uint32_t (&o)[2], uint32_t imm) {
	s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(uintptr_t)(o[0] + imm));
	s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 ELF_LDS*)(uintptr_t)(o[1] + imm));
	return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// NW = 4, RT = 4: 256x256 workgroup tile, one wave per SIMD with a 128x128 wave tile: 16 fragment reads per
// k32 for 64 MFMAs, a third less LDS traffic per FLOP than the eight-wave shape, which on this power-limited
// part is worth 2-4 % (forward and dX GEMMs).  It needs two things a lone wave does not forgive: all 256
// accumulator registers are live, so the MFMAs are tied in place by hand (mfma_acc), and nothing else
// fills issue gaps, so the next half-step's fragment reads and the slice's loads are dealt between the
// MFMAs one at a time (half_step).  Left to the builtin and to bursts of reads it ran 12 % slower than
// the eight-wave shape.
// NW = 8, RT = 2: 256x256 workgroup tile, two waves per SIMD with 64x128 wave tiles (12 fragment reads per
// k32 and 32 MFMAs); the two waves fill each other's issue gaps and barrier waits.  Used when both
// operands are reduction-major (dW): each of their fragments costs two transpose reads and an address.
// NW = 4, RT = 2: 128x256 workgroup tile for outputs with too few 256x256 tiles to fill the chip.  One wave per SIMD
// as well, so it runs the same interleaved loop (+35-40 % on the GPT-2-small shapes over read bursts).
// Which of the `half` load pieces dealt over a half-step of `nm` MFMAs goes out after MFMA n (-1: none): piece k after
// MFMA 2 * floor(k * (nm / 2) / half) - always an even one, because the fragment reads go out after the odd ones and a
// read and a load behind the same MFMA do not fit under it.
constexpr int piece_in_slot(int n, int nm, int half) {
	for (int k = 0; k < half; k++)
		if (2 * ((k * (nm / 2)) / half) == n) return k;
	return -1;
}

// every piece has a slot of its own within the half-step
constexpr bool pieces_have_slots(int nm, int half) {
	for (int k = 0; k < half; k++) {
		int hits = 0;
		for (int n = 0; n < nm; n++) hits += piece_in_slot(n, nm, half) == k;
		if (hits != 1) return false;
	}
	return true;
}

// acc += a b as one in-place instruction on accumulator registers — the builtin leaves source and
// destination accumulators untied, and when all 256 accumulator registers are live (128x128 wave tiles) the
// allocator then copies accumulator tiles around inside the loop (192 copies per K slice).  Every
// accumulator tile is touched once per half-step, so consecutive MFMAs never depend on each other, and the
// epilogue reads the accumulators only after a wait and a workgroup barrier.
__device__ __forceinline__ void mfma_acc(f32x4& acc, const bf16x8& a, const bf16x8& b) {
	asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}


// Origin (m0, n0) of tile `pid` of the launch: see "Tile assignment" in gemm_dma_kernel for the two walks.
template <int BM>
__device__ __forceinline__ void tile_origin(const Args& g, int pid, int& m0, int& n0) {
	if (g.walk == 2) {  // tiles in plain order, down the rows first (the launch places them on the XCDs itself)
		m0 = (pid % g.tiles_m) * BM;
		n0 = (pid / g.tiles_m) * BN;
		return;
	}
	const int ntiles = g.tiles_m * g.tiles_n;
	const int nsb = ntiles >> 5, nrem = nsb & 7;
	if (g.walk == 1 && (g.tiles_m & 7) == 0 && (g.tiles_n & 3) == 0 && (nrem == 0 || nrem == 1 || nrem == 2 || nrem == 4)) {
		const int x = pid & 7, i = pid >> 3, nfull = nsb >> 3;
		int sb, jj;
		if (i < nfull * 32) {
			sb = (i >> 5) * 8 + x;
			jj = i & 31;
		} else {
			const int k = 8 / nrem;
			sb = nfull * 8 + x / k;
			jj = (x % k) * (32 / k) + (i - nfull * 32);
		}
		const int nsb_n = g.tiles_n >> 2, nsb_m = g.tiles_m >> 3;
		const int band = sb / (2 * nsb_n), within = sb - band * 2 * nsb_n;
		const bool pair = 2 * band + 1 < nsb_m;
		const int sbm = 2 * band + (pair ? within & 1 : 0), sbn = pair ? within >> 1 : within;
		m0 = (sbm * 8 + (jj & 7)) * BM;
		n0 = (sbn * 4 + (jj >> 3)) * BN;
	} else {
		if ((ntiles & 7) == 0) pid = (pid & 7) * (ntiles >> 3) + (pid >> 3);
		constexpr int GROUP_M = 8;
		const int per_group = GROUP_M * g.tiles_n;
		const int first_m = (pid / per_group) * GROUP_M;
		const int gsz = min(g.tiles_m - first_m, GROUP_M);
		m0 = (first_m + (pid % per_group) % gsz) * BM;
		n0 = ((pid % per_group) / gsz) * BN;
	}
}

// Tile, K range and turn counter of workgroup `bid` of the problem `g` (the block index of a launch with one problem).
// The first ntiles - tail_tiles tiles are computed whole, one workgroup each; each of the last tail_tiles is shared by
// k_splits workgroups that take a K range each and add their part with atomics.  Splitting only the tail turns the
// last, partly filled round of workgroups of a launch into a full round of shorter ones.
__device__ __forceinline__ void locate_tile(const Args& g, const int bid, int& pid, int& ksplit, int& splits, int& turn_slot) {
	const int ntiles = g.tiles_m * g.tiles_n;
	const int full = ntiles - g.tail_tiles;
	pid = bid, ksplit = 0, splits = 1;
	if (pid >= full) {
		const int q = pid - full;
		splits = g.k_splits;
		if (((ntiles | full) & 7) == 0) {  // keep workgroup index = tile index (mod 8): same XCD as its neighbours
			const int rest = q >> 3;
			ksplit = rest % splits;
			pid = full + (rest / splits) * 8 + (q & 7);
		} else {
			ksplit = q % splits;
			pid = full + q / splits;
		}
	}
	// split tiles: the turn counter of this tile (tiles of one launch get distinct counters, consecutive launches different ones)
	turn_slot = (int)(((uint32_t)(pid - full) + g.turn_base) % (uint32_t)TURN_TILES);
}

// One workgroup: tile `pid` of the problem `g`, K range `ksplit` of `splits`; a split tile's turn counters are those of
// `turn_slot`.
template <int NW, int RT, bool AT, bool BT, int EPI>
__device__ __forceinline__ void gemm_dma_tile(const Args& g, const int pid, const int ksplit, const int splits, const int turn_slot) {
	using Sh = Shape<NW, RT>;
	constexpr int BM = Sh::BM, A_BYTES = Sh::A_BYTES, STAGE_BYTES = Sh::STAGE_BYTES;
	constexpr int LOADS_A = Sh::LOADS_A, LOADS_B = Sh::LOADS_B, LOADS_PER_STAGE = Sh::LOADS_PER_STAGE, NST = Sh::NST;
	constexpr bool PAIRED = EPI == EPI_BF16_SWIGLU;
	static_assert(!PAIRED || !BT, "the paired row order is defined for a k-contiguous B");
	extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wr = wave >> 1, wc = wave & 1;

	// Tile assignment (tile_origin).  Workgroup w runs on XCD w % 8, whose 32 CUs hold 32 tiles at a time (a round);
	// both walks give an XCD 8 tile rows x 4 tile columns per round (12 operand slabs through its L2 for
	// 32 tiles) and differ in where the 8 XCDs are relative to each other:
	//  * default: each XCD owns a contiguous run of tiles (8 tile rows at a time, along the columns).  The
	//    XCDs work on different row groups; a row slab of A is needed in as many rounds as the row has
	//    column groups, so A has to stay in the memory-side cache between them;
	//  * walk = 1: the 8 XCDs share a 16 x 16 block of tiles per round, bands of 16 tile rows walked along the
	//    columns; a row slab of A is live for one band only, B is fetched once per band (weight gradient of
	//    the gate/up projection, 28672 x 4096 at K = 8192, A = 470 MB: 5-7 % faster).  A last, partly filled
	//    round shares each 8 x 4 block between several XCDs.
	int m0, n0;
	tile_origin<BM>(g, pid, m0, n0);
	m0 = __builtin_amdgcn_readfirstlane(m0);
	n0 = __builtin_amdgcn_readfirstlane(n0);

	const int nk_total = g.K / BKS;
	const int nk_per = (nk_total + splits - 1) / splits;
	const int kt0 = ksplit * nk_per;
	const int nk = min(nk_total, kt0 + nk_per) - kt0;
	if (nk <= 0) {
		// a split without a K range of its own still takes and passes its turn on every strip
		if (splits > 1 && g.turn_tag && lane == 0) {
			const uint32_t want = (g.turn_tag << 8) | (uint32_t)ksplit;
			int patience = TURN_SPIN_LIMIT;
			for (int i = 0; i < RT; i++) {
				uint32_t* t = turn + turn_slot * TURN_PER_TILE + wave * RT + i;
				int spin = 0;
				for (; ksplit > 0 && spin < patience && __hip_atomic_load(t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != want; spin++)
					__builtin_amdgcn_s_sleep(8);
				if (ksplit > 0 && spin >= patience) {
					if (patience > 0) note_turn_giveup();
					patience = 0;
				} else {
					patience -= spin;
				}
				__hip_atomic_store(t, want + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			}
		}
		return;
	}

	const bf16_t* Ap = AT ? g.A + (int64_t)kt0 * BKS * g.lda + m0 : g.A + (int64_t)m0 * g.lda + (int64_t)kt0 * BKS;
	// paired rows: tile column n0 of the (gate | up interleaved) product starts at operand row n0 / 2
	const bf16_t* Bp = BT ? g.B + (int64_t)kt0 * BKS * g.ldb + n0 : g.B + (int64_t)(PAIRED ? n0 / 2 : n0) * g.ldb + (int64_t)kt0 * BKS;
	const int64_t a_step = AT ? (int64_t)BKS * g.lda : BKS;
	const int64_t b_step = BT ? (int64_t)BKS * g.ldb : BKS;
	uint32_t aoff[LOADS_A], boff[LOADS_B];
	lane_offsets<AT, LOADS_A, false, BM>(wave, lane, g.lda, aoff);
	lane_offsets<BT, LOADS_B, PAIRED>(wave, lane, g.ldb, boff, g.N / 2);

	// this wave's first 1 KiB piece of each operand in stage 0
	const uint32_t lds_a = lds_addr(smem) + wave * (LOADS_A * 1024);
	const uint32_t lds_b = lds_addr(smem) + NST * A_BYTES + wave * (LOADS_B * 1024);

	// Loads of one K slice: its operand pointers and the LDS addresses of this wave's first piece of
	// each operand in the slice's stage.  Piece P (compile-time) is one wave instruction filling 1 KiB;
	// the first LOADS_A pieces belong to A, the rest to B.  A slice past the end of K is fetched from
	// the last slice into a scratch area behind the ring (shared by all waves: nobody reads it), so
	// that the main loop needs no branches around its loads and the accumulators stay put in registers.
	struct SliceLoads {
		const bf16_t* pa;
		const bf16_t* pb;
		uint32_t la, lb;
	};
	const uint32_t lds_dummy = lds_addr(smem) + NST * STAGE_BYTES;
	auto slice_loads = [&](int step) {
		const bool ok = step < nk;
		const int sc = ok ? step : nk - 1;
		const uint32_t st = (uint32_t)(sc % NST);
		return SliceLoads{Ap + (int64_t)sc * a_step, Bp + (int64_t)sc * b_step, ok ? lds_a + st * A_BYTES : lds_dummy, ok ? lds_b + st * B_BYTES : lds_dummy};
	};
	auto issue_piece = [&](const SliceLoads& sl, auto pc) {
		constexpr int P = decltype(pc)::value;
		if constexpr (P < LOADS_A) dma16_at<P * 1024>(sl.pa, aoff[P], sl.la);
		else dma16_at<(P - LOADS_A) * 1024>(sl.pb, boff[P - LOADS_A], sl.lb);
	};

	// 16x16 accumulator tiles: RT * 2 down, 8 across (the 16x16x32 MFMA moves half as many accumulator
	// registers per FLOP as the 32x32x16 one, and sustains a higher clock under the power limit)
	constexpr int RF = RT * 2;
	f32x4 acc[RF][8];
#pragma unroll
	for (int i = 0; i < RF; i++)
#pragma unroll
		for (int j = 0; j < 8; j++)
#pragma unroll
			for (int r = 0; r < 4; r++) acc[i][j][r] = 0.f;

	// Software pipeline.  A slice is four half-steps (k32 half kq = 0, 1 x column half h = 0, 1) of RF * 4
	// MFMAs; the fragments of a half-step are read during the one before it (B: four 16-column slabs
	// per half-step, ping-pong; A: RF slabs per k32 half, ping-pong).  The barrier that publishes slice
	// kt+1 sits before the LAST half-step of slice kt: by then every wave has read all of slice kt (its
	// last fragments are in registers), so the same barrier frees that stage and the fetch of slice
	// kt+2 starts a full slice ahead of its use.
	constexpr int HALF = LOADS_PER_STAGE / 2;
	static_assert(pieces_have_slots(RF * 4, HALF), "a half-step has too few even MFMA slots for half a slice's loads");
	{
		// slices 0 .. NST-2 whole and the first half of slice NST-1; slice 0 has to have landed
		static_for<NST - 1>([&](auto sc) {
			const SliceLoads sl = slice_loads(decltype(sc)::value);
			static_for<LOADS_PER_STAGE>([&](auto pc) { issue_piece(sl, pc); });
		});
		const SliceLoads sh = slice_loads(NST - 1);
		static_for<HALF>([&](auto pc) { issue_piece(sh, pc); });
		wait_vmcnt<(NST - 2) * LOADS_PER_STAGE + HALF>();
	}
	__syncthreads();

	bf16x8 fa[2][RF], fb[2][4];
	auto load_a = [&](int buf, int step, int kq) {
		const unsigned char* sa = smem + (step % NST) * A_BYTES;
#pragma unroll
		for (int i = 0; i < RF; i++) fa[buf][i] = frag<AT, BM>(sa, wr * (RT * 32) + i * 16, kq, lane);
	};
	auto load_b = [&](int buf, int step, int kq, int h) {
		const unsigned char* sb = smem + NST * A_BYTES + (step % NST) * B_BYTES;
#pragma unroll
		for (int j = 0; j < 4; j++) fb[buf][j] = frag<BT>(sb, wc * 128 + (h * 4 + j) * 16, kq, lane);
	};
	// One half-step: RF * 4 MFMAs with the fragment reads of the next half-step (one read per two MFMAs, B
	// slabs first: they are needed first) and, in two of the four half-steps, half of this wave's loads of a
	// slice dealt between them one at a time.  A lone wave per SIMD has nothing else to fill its issue
	// gaps, and a wave that issues its loads in one burst (64 KiB per slice through a 64 B/clk path) sits in
	// the queue for ~1000 cycles with its MFMAs behind it.  With two waves per SIMD the wave also raises
	// its issue priority for the length of the half-step: the one feeding the matrix pipe goes first.
	// Reduction-major operands in this loop: the two transpose-read addresses of every fragment are computed
	// once (k32 half 0 of stage 0); the k32 half and the stage are compile-time here (the loop is unrolled
	// by two slices) and go into the instructions' offset fields, so the loop has no address arithmetic.
	uint32_t ta[AT ? RF : 1][2], tb[BT ? 8 : 1][2];
	{
		if constexpr (AT)
#pragma unroll
			for (int i = 0; i < RF; i++) {
				frag_t_offsets<BM>(wr * (RT * 32) + i * 16, lane, ta[i]);
				ta[i][0] += lds_addr(smem), ta[i][1] += lds_addr(smem);
				// opaque from here on: folded into these, the tile's base would push the loop's offsets past 16 bits
				asm volatile("" : "+v"(ta[i][0]), "+v"(ta[i][1]));
			}
		if constexpr (BT)
#pragma unroll
			for (int i = 0; i < 8; i++) {
				frag_t_offsets(wc * 128 + i * 16, lane, tb[i]);
				tb[i][0] += lds_addr(smem) + NST * A_BYTES, tb[i][1] += lds_addr(smem) + NST * A_BYTES;
				asm volatile("" : "+v"(tb[i][0]), "+v"(tb[i][1]));
			}
	}
	auto half_step = [&](int abuf, int bbuf, auto hc, int pb_buf, auto pb_stage, int pb_kq, int pb_h, bool pa, int pa_buf, auto pa_stage, int pa_kq,
	                     const SliceLoads& sl, auto piece0) {
		constexpr int PIECE0 = decltype(piece0)::value, H = decltype(hc)::value, NM = RF * 4;
		constexpr int SA = decltype(pa_stage)::value, SB = decltype(pb_stage)::value;
		const unsigned char* sa = smem + SA * A_BYTES;
		const unsigned char* sb = smem + NST * A_BYTES + SB * B_BYTES;
		if constexpr (NW == 8) __builtin_amdgcn_s_setprio(1);
		static_for<NM>([&](auto nc) {
			constexpr int n = decltype(nc)::value, i = n / 4, j = n % 4;
			mfma_acc(acc[i][H * 4 + j], fa[abuf][i], fb[bbuf][j]);
			if constexpr (n % 2 == 1) {
				constexpr int r = n / 2;
				if constexpr (r < 4) {
					if constexpr (BT) fb[pb_buf][r] = frag_t_at(tb[pb_h * 4 + r], (uint32_t)(SB * B_BYTES + pb_kq * (32 * 512)));
					else fb[pb_buf][r] = frag<BT>(sb, wc * 128 + (pb_h * 4 + r) * 16, pb_kq, lane);
				} else if constexpr (r - 4 < RF) {
					if (pa) {
						if constexpr (AT) fa[pa_buf][r - 4] = frag_t_at(ta[r - 4], (uint32_t)(SA * A_BYTES + pa_kq * (32 * BM * 2)));
						else fa[pa_buf][r - 4] = frag<AT, BM>(sa, wr * (RT * 32) + (r - 4) * 16, pa_kq, lane);
					}
				}
			}
			if constexpr (PIECE0 >= 0 && piece_in_slot(n, NM, HALF) >= 0) issue_piece(sl, std::integral_constant<int, (PIECE0 < 0 ? 0 : PIECE0) + (piece_in_slot(n, NM, HALF) < 0 ? 0 : piece_in_slot(n, NM, HALF))>{});
			__builtin_amdgcn_sched_barrier(0);
		});
		if constexpr (NW == 8) __builtin_amdgcn_s_setprio(0);
	};
	// one K slice held in stage S; the next one's fragments come from stage 1 - S
	auto slice = [&](auto sc, int kt) {
		constexpr int S = decltype(sc)::value;
		constexpr std::integral_constant<int, S> CUR{};
		constexpr std::integral_constant<int, (S + 1) % NST> NXT{};
		constexpr std::integral_constant<int, 0> H0{};
		constexpr std::integral_constant<int, 1> H1{};
		constexpr std::integral_constant<int, -1> NO_DMA{};
		// where this slice's loads go: scalar work
		const SliceLoads next1 = slice_loads(kt + NST - 1), next2 = slice_loads(kt + NST);
		half_step(0, 0, H0, 1, CUR, 0, 1, false, 0, CUR, 0, next1, std::integral_constant<int, HALF>{});
		half_step(0, 1, H1, 0, CUR, 1, 0, true, 1, CUR, 1, next1, NO_DMA);
		half_step(1, 0, H0, 1, CUR, 1, 1, false, 0, CUR, 0, next1, NO_DMA);
		// vmcnt: slice kt+1 landed (with three stages slice kt+2's loads may still be in flight); lgkmcnt(0): slice kt fully read
		wait_counters<(NST - 2) * LOADS_PER_STAGE, 0>();
		__syncthreads();
		// with the first half of slice kt+NST's loads into the stage the barrier just freed; past the end the
		// fragment reads hit a stale stage and their values are unused
		half_step(1, 1, H1, 0, NXT, 0, 0, true, 0, NXT, 0, next2, std::integral_constant<int, 0>{});
	};

	load_a(0, 0, 0);
	load_b(0, 0, 0, 0);
	for (int kt = 0; kt < nk; kt += NST) {
		slice(std::integral_constant<int, 0>{}, kt);
		if (kt + 1 < nk) slice(std::integral_constant<int, 1>{}, kt + 1);
		if constexpr (NST == 3)
			if (kt + 2 < nk) slice(std::integral_constant<int, 2>{}, kt + 2);
	}

	// Epilogue through LDS (free once every wave has left the main loop).  Register r of a 16x16
	// accumulator tile holds row (lane/16)*4 + r, column lane%16; each wave parks one 32 x 128 fp32 strip
	// (two rows of accumulator tiles) at a time in its own LDS region (row pitch 136 floats) and reads it
	// back row-wise, so that global accesses are 16 bytes per lane over 256..512 contiguous bytes per row
	// and accumulators leave the AGPRs only via ds_write.
	wait_vmcnt<0>();  // the loads past the end of K issued by the last iterations land in LDS too
	__syncthreads();
	constexpr int PITCH = 136;
	float* ws = reinterpret_cast<float*>(smem) + wave * (32 * PITCH);
	[[maybe_unused]] int turn_patience = TURN_SPIN_LIMIT;
	const int col_l = lane & 15;
	const int row_l = (lane >> 4) * 4;
#pragma unroll
	for (int i = 0; i < RT; i++) {
#pragma unroll
		for (int ii = 0; ii < 2; ii++)
#pragma unroll
			for (int j = 0; j < 8; j++)
#pragma unroll
				for (int r = 0; r < 4; r++) ws[(ii * 16 + row_l + r) * PITCH + j * 16 + col_l] = acc[i * 2 + ii][j][r];
		const int grow0 = m0 + wr * (RT * 32) + i * 32;
		const int gcol0 = n0 + wc * 128;
		if constexpr (EPI == EPI_BF16_SWIGLU) {
			// the strip's columns are 64 gate columns then the 64 up columns of the same outputs: both go to
			// their places in C = [gate | up] (kept for the backward) and silu(gate) * up, computed from the
			// rounded values exactly as a separate pass over C would, to C2
			const int F = g.N / 2, cg0 = n0 / 2 + wc * 64;
#pragma unroll
			for (int it = 0; it < 4; it++) {
				const int row = it * 8 + (lane >> 3), c8 = (lane & 7) * 8;
				const float* w = ws + row * PITCH + c8;
				const f32x4 g0 = *reinterpret_cast<const f32x4*>(w), g1 = *reinterpret_cast<const f32x4*>(w + 4);
				const f32x4 u0 = *reinterpret_cast<const f32x4*>(w + 64), u1 = *reinterpret_cast<const f32x4*>(w + 68);
				bf16x8 og, ou, oa;
#pragma unroll
				for (int t = 0; t < 8; t++) {
					og[t] = (bf16_t)(t < 4 ? g0[t] : g1[t - 4]);
					ou[t] = (bf16_t)(t < 4 ? u0[t] : u1[t - 4]);
					oa[t] = (bf16_t)swiglu_f((float)og[t], (float)ou[t]);
				}
				bf16_t* c = reinterpret_cast<bf16_t*>(g.C) + (int64_t)(grow0 + row) * g.ldc + cg0 + c8;
				*reinterpret_cast<bf16x8*>(c) = og;
				*reinterpret_cast<bf16x8*>(c + F) = ou;
				*reinterpret_cast<bf16x8*>(g.C2 + (int64_t)(grow0 + row) * g.ldc2 + cg0 + c8) = oa;
			}
		} else if constexpr (EPI == EPI_BF16_SWIGLU_BWD) {
			// the tile is d = dY W over F columns; g and u of the same rows and columns lie F columns apart in R,
			// their gradients likewise in C.  All loads of the strip first (see the residual epilogue below); d is
			// rounded to bf16 before it is used, as a separate pass over a stored d would read it
			const int F = g.N;
			bf16x8 gs[8], us[8];
#pragma unroll
			for (int it = 0; it < 8; it++) {
				const bf16_t* r = g.R + (int64_t)(grow0 + it * 4 + (lane >> 4)) * g.ldr + gcol0 + (lane & 15) * 8;
				gs[it] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(r));  // the pre-activation is read this once in B
				us[it] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(r + F));
			}
#pragma unroll
			for (int it = 0; it < 8; it++) {
				const int row = it * 4 + (lane >> 4), c8 = (lane & 15) * 8;
				const f32x4 lo = *reinterpret_cast<const f32x4*>(ws + row * PITCH + c8);
				const f32x4 hi = *reinterpret_cast<const f32x4*>(ws + row * PITCH + c8 + 4);
				bf16x8 og, ou;
#pragma unroll
				for (int t = 0; t < 8; t++) {
					const float d = (float)(bf16_t)(t < 4 ? lo[t] : hi[t - 4]);
					float dg, du;
					swiglu_bwd_f(d, (float)gs[it][t], (float)us[it][t], dg, du);
					og[t] = (bf16_t)dg;
					ou[t] = (bf16_t)du;
				}
				bf16_t* c = reinterpret_cast<bf16_t*>(g.C) + (int64_t)(grow0 + row) * g.ldc + gcol0 + c8;
				*reinterpret_cast<bf16x8*>(c) = og;
				*reinterpret_cast<bf16x8*>(c + F) = ou;
				if (g.C2) {
					// a stash that dropped the activation gets it back here, from the g and u this epilogue holds anyway (the
					// forward's own arithmetic: the bits of swiglu_fwd)
					bf16x8 oa;
#pragma unroll
					for (int t = 0; t < 8; t++) oa[t] = (bf16_t)swiglu_f((float)gs[it][t], (float)us[it][t]);
					*reinterpret_cast<bf16x8*>(g.C2 + (int64_t)(grow0 + row) * g.ldc2 + gcol0 + c8) = oa;
				}
			}
		} else if constexpr (EPI == EPI_BF16_ROPE) {
			// A 128-column strip holds whole heads (rope_D = 64 or 128).  A lane takes, for one row, 8 columns of a
			// head's first half and the 8 columns half a head further on: the (x_i, x_{i + D/2}) pairs of the rotation.
			// The accumulator is rounded to bf16 first, as the RoPE kernel would read it from memory.  The table
			// entries of the whole strip are fetched before the first store (see the residual epilogue below).
			const int half = g.rope_D >> 1, cph = half >> 3;  // chunks of 8 columns per half head
			const int j = lane & 7;
			const int c_lo = (j / cph) * g.rope_D + (j % cph) * 8, c_hi = c_lo + half;
			const bool rot = gcol0 + c_lo < g.rope_cols;
			f32x4 tab[4][4];
			if (rot) {
#pragma unroll
				for (int it = 0; it < 4; it++) {
					const int pos = (grow0 + it * 8 + (lane >> 3)) % g.rope_S;
					const f32x4* tp = reinterpret_cast<const f32x4*>(g.rope_cs + (int64_t)pos * half + (j % cph) * 8);
#pragma unroll
					for (int q = 0; q < 4; q++) tab[it][q] = tp[q];
				}
			}
#pragma unroll
			for (int it = 0; it < 4; it++) {
				const int row = it * 8 + (lane >> 3);
				const float* w = ws + row * PITCH;
				const f32x4 a0 = *reinterpret_cast<const f32x4*>(w + c_lo), a1 = *reinterpret_cast<const f32x4*>(w + c_lo + 4);
				const f32x4 b0 = *reinterpret_cast<const f32x4*>(w + c_hi), b1 = *reinterpret_cast<const f32x4*>(w + c_hi + 4);
				bf16x8 olo, ohi;
#pragma unroll
				for (int t = 0; t < 8; t++) {
					const float a = (float)(bf16_t)(t < 4 ? a0[t] : a1[t - 4]), b = (float)(bf16_t)(t < 4 ? b0[t] : b1[t - 4]);
					float ra = a, rb = b;
					if (rot) rope_rot(a, b, tab[it][t >> 1][(t & 1) * 2], tab[it][t >> 1][(t & 1) * 2 + 1], ra, rb);
					olo[t] = (bf16_t)ra;
					ohi[t] = (bf16_t)rb;
				}
				bf16_t* c = reinterpret_cast<bf16_t*>(g.C) + (int64_t)(grow0 + row) * g.ldc + gcol0;
				*reinterpret_cast<bf16x8*>(c + c_lo) = olo;
				*reinterpret_cast<bf16x8*>(c + c_hi) = ohi;
			}
		} else if constexpr (EPI == EPI_BF16 || EPI == EPI_BF16_RESID) {
			// the strip's residual values first, all loads in flight together: read inside the loop below each
			// one would be awaited (a full trip to HBM) before the store that follows it in program order
			bf16x8 rs[EPI == EPI_BF16_RESID ? 8 : 1];
			if constexpr (EPI == EPI_BF16_RESID) {
#pragma unroll
				for (int it = 0; it < 8; it++)
					rs[it] = *reinterpret_cast<const bf16x8*>(g.R + (int64_t)(grow0 + it * 4 + (lane >> 4)) * g.ldr + gcol0 + (lane & 15) * 8);
			}
#pragma unroll
			for (int it = 0; it < 8; it++) {
				const int row = it * 4 + (lane >> 4), c8 = (lane & 15) * 8;
				const f32x4 lo = *reinterpret_cast<const f32x4*>(ws + row * PITCH + c8);
				const f32x4 hi = *reinterpret_cast<const f32x4*>(ws + row * PITCH + c8 + 4);
				float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
				if constexpr (EPI == EPI_BF16_RESID) {
#pragma unroll
					for (int t = 0; t < 8; t++) v[t] += (float)rs[it][t];
				}
				bf16x8 o;
#pragma unroll
				for (int t = 0; t < 8; t++) o[t] = (bf16_t)v[t];
				*reinterpret_cast<bf16x8*>(reinterpret_cast<bf16_t*>(g.C) + (int64_t)(grow0 + row) * g.ldc + gcol0 + c8) = o;
			}
		} else {
			if ((EPI == EPI_F32_ACC || EPI == EPI_F32_ACC_SCALE) && splits > 1) {  // (split tiles of a scaling launch are scaled by scale_tail_kernel)
				uint32_t* const my_turn = turn + turn_slot * TURN_PER_TILE + wave * RT + i;
				if (g.turn_tag && ksplit > 0) {
					// wait for this split's turn on this strip (see turn[]); every lane polls the same word.  Plain
					// (cache-bypassing) loads: nothing is read after the wait, the adds are performed at the memory side
					const uint32_t want = (g.turn_tag << 8) | (uint32_t)ksplit;
					int spin = 0;
					for (; spin < turn_patience && __hip_atomic_load(my_turn, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != want; spin++)
						__builtin_amdgcn_s_sleep(8);
					// a wave that gave up once (its counters are shared with a concurrent launch) does not wait again
					if (spin >= turn_patience) {
						if (turn_patience > 0 && lane == 0) note_turn_giveup();
						turn_patience = 0;
					} else {
						turn_patience -= spin;
					}
				}
				// several workgroups add into this tile: fp32 atomics, one scalar per lane so that a wave
				// instruction covers two whole 128-byte rows of 32 columns (16 bytes per lane would touch a
				// quarter of eight lines per instruction and run at half the speed)
#pragma unroll
				for (int it = 0; it < 16; it++) {
					const int row = it * 2 + (lane >> 5);
					float* c = reinterpret_cast<float*>(g.C) + (int64_t)(grow0 + row) * g.ldc + gcol0 + (lane & 31);
#pragma unroll
					for (int cg = 0; cg < 4; cg++) unsafeAtomicAdd(c + cg * 32, ws[row * PITCH + cg * 32 + (lane & 31)]);
				}
				if (g.turn_tag) {
					// wait until this wave's adds have been performed (they complete in vmcnt; no cache write-back is
					// needed for atomics), then the next split may add to this strip
					wait_vmcnt<0>();
					if (lane == 0) __hip_atomic_store(my_turn, (g.turn_tag << 8) | (uint32_t)(ksplit + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				}
				continue;
			}
			// fp32 accumulate: the strip's 16 loads of C all in flight before the first store (left inside the
			// loop each load is awaited on its own, 16 trips to HBM in a row per strip: 43 k cycles of a
			// 360 k-cycle dW tile)
			constexpr bool ACCUM = EPI == EPI_F32_ACC || EPI == EPI_F32_ACC_SCALE;
			f32x4 cv[ACCUM ? 16 : 1];
			if constexpr (ACCUM) {
#pragma unroll
				for (int it = 0; it < 16; it++)
					cv[it] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(g.C) + (int64_t)(grow0 + it * 2 + (lane >> 5)) * g.ldc + gcol0 + (lane & 31) * 4));
			}
#pragma unroll
			for (int it = 0; it < 16; it++) {
				const int row = it * 2 + (lane >> 5), c4 = (lane & 31) * 4;
				f32x4 v = *reinterpret_cast<const f32x4*>(ws + row * PITCH + c4);
				float* c = reinterpret_cast<float*>(g.C) + (int64_t)(grow0 + row) * g.ldc + gcol0 + c4;
				if constexpr (ACCUM) v += cv[it];
				if constexpr (EPI == EPI_F32_ACC_SCALE) {
					// the step's last weight-gradient pass: the gradient scale and the bf16 copy that scale_grads would make
					// in a pass of its own over the accumulator (same operations on the same values: same bits)
					v *= g.scale;
					bf16x4 o;
#pragma unroll
					for (int t = 0; t < 4; t++) o[t] = (bf16_t)v[t];
					*reinterpret_cast<bf16x4*>(g.C2 + (int64_t)(grow0 + row) * g.ldc2 + gcol0 + c4) = o;
				}
				if constexpr (ACCUM) __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(c));  // next touched by the next W pass
				else *reinterpret_cast<f32x4*>(c) = v;
			}
		}
	}
}

template <int NW, int RT, bool AT, bool BT, int EPI>
__global__ __launch_bounds__(NW * 64) void gemm_dma_kernel(Args g) {
	int pid, ksplit, splits, turn_slot;
	locate_tile(g, (int)blockIdx.x, pid, ksplit, splits, turn_slot);
	gemm_dma_tile<NW, RT, AT, BT, EPI>(g, pid, ksplit, splits, turn_slot);
}

// Several weight gradients in one launch (the W pass of a stage: every linear layer's dW += dY^T X over the same
// tokens).  The chip's workgroup slots refill across problem boundaries, so only the launch's last round is partly
// filled, and small problems that would each need their tiles split many ways to fill the chip fill it together.
//  * compact = 0 (a problem of 256 tiles or more among them): the workgroups of problem p are first[p] .. first[p] +
//    count[p] - 1, each first[p] a multiple of 8 so that a workgroup's index within its problem names its XCD as in a
//    launch of its own (the workgroups in the gaps leave at once); every problem keeps its own walk and its own tail.
//  * compact = 1 (small problems only): the tiles of all problems form one sequence (problem after problem, down the
//    rows first; first[p] = problem p's first tile in it) and XCD x takes a contiguous eighth of its whole tiles, then
//    of its split tiles with the `splits` workgroups of a tile side by side: the 32 tiles an XCD holds at a time are
//    neighbours that share their operand slabs in its L2 (taken in launch order, neighbouring tiles of a 3-row problem
//    land on different XCDs and every slab is fetched by all eight).
constexpr int GROUP_MAX = 16;
struct GroupArgs {
	int n, compact;
	int tiles, tail, splits;  // compact: all tiles of the launch, how many of the last are split, and how many ways
	uint32_t turn_base;
	int first[GROUP_MAX], count[GROUP_MAX];
	Args a[GROUP_MAX];
};
template <int EPI>
__global__ __launch_bounds__(512) void gemm_dw_group_kernel(GroupArgs ga) {
	int p = 0, pid, ksplit = 0, splits = 1, turn_slot = 0;
	if (ga.compact) {
		const int x = blockIdx.x & 7, slot = blockIdx.x >> 3;
		const int full = ga.tiles - ga.tail, chunk_f = (full + 7) >> 3, chunk_t = (ga.tail + 7) >> 3;
		int gt;
		if (slot < chunk_f) {
			gt = x * chunk_f + slot;
			if (gt >= full) return;
		} else {
			const int q = slot - chunk_f, tt = x * chunk_t + q / ga.splits;
			if (tt >= ga.tail) return;
			gt = full + tt;
			ksplit = q % ga.splits;
			splits = ga.splits;
			turn_slot = (int)(((uint32_t)tt + ga.turn_base) % (uint32_t)TURN_TILES);
		}
		for (int i = 1; i < ga.n; i++)
			if (gt >= ga.first[i]) p = i;
		p = __builtin_amdgcn_readfirstlane(p);
		pid = gt - ga.first[p];
	} else {
		for (int i = 1; i < ga.n; i++)
			if ((int)blockIdx.x >= ga.first[i]) p = i;
		p = __builtin_amdgcn_readfirstlane(p);
		const int bid = (int)blockIdx.x - ga.first[p];
		if (bid >= ga.count[p]) return;
		locate_tile(ga.a[p], bid, pid, ksplit, splits, turn_slot);
	}
	gemm_dma_tile<8, 2, true, true, EPI>(ga.a[p], pid, ksplit, splits, turn_slot);
}

// ------------------------------------------------------------------------------------------------------------
// Persistent forward kernel: both operands k-contiguous, 256x256 tiles, four waves with 128x128 wave tiles - the loop
// of gemm_dma_kernel<4, 4, false, false, .> with two changes that take the tile boundary out of the matrix pipe's way.
//
//  * The epilogue leaves from registers.  The MFMA operands are swapped (the weight rows feed the m side), so a lane
//    holds four consecutive columns of ONE output row per accumulator tile, and the order in which weight rows enter
//    the four column slabs of a half-step is permuted (slab jj, m slot 4 g + r  <-  column 32 (jj / 2) + 8 g + 4 (jj % 2) + r)
//    so that the lane's 16 values of a half-step are two runs of 8 consecutive columns: one 16-byte store each, the four
//    lane groups of a row together 64 contiguous bytes.  No LDS staging, no barrier, a quarter of the instructions.
//    For column slab jj of half h and k32 half kq lane l reads tile row wc * 128 + h * 64 + 32 (jj / 2) + 8 ((l % 16) / 4)
//    + 4 (jj % 2) + l % 4 at k = 32 kq + 8 (l / 16) .. + 7; the B tile's chunk swizzle follows these rows (rb_swz) so
//    that the 16 lanes of a k chunk still hit 16 different 16-byte bank groups.
//  * A workgroup walks tiles pid, pid + grid, ... and its K-slice pipeline never drains: the last two slices of a tile
//    fetch the first two of the next (the loop's "slice past the end of K" is the next tile's slice 0), the LDS ring is
//    not needed by the epilogue, and the first MFMAs of a tile write their accumulators (C = 0 form) instead of adding
//    to cleared ones.  K / 64 must be even so that a tile starts in ring stage 0.
// Results are bit-identical to gemm_dma_kernel's: same products, same accumulation order along K, same roundings.
__device__ __forceinline__ int rb_swz(int row) { return (((row >> 3) & 3) << 1) | ((row >> 1) & 1); }

template <bool PAIRED>
__device__ __forceinline__ void lane_offsets_rb(int wave, int lane, int64_t ld, uint32_t (&off)[8], int64_t pair_rows) {
#pragma unroll
	for (int i = 0; i < 8; i++) {
		const int q = wave * 8 + i;
		const int row = q * 8 + (lane >> 3), slot = lane & 7;
		const int64_t grow = PAIRED ? (row >> 7) * 64 + (row & 63) + ((row >> 6) & 1) * pair_rows : row;
		off[i] = (uint32_t)((grow * ld + ((slot ^ rb_swz(row)) << 3)) * 2);
	}
}

// acc = a b: the first MFMA of an accumulator tile in a tile's K loop
__device__ __forceinline__ void mfma_init(f32x4& acc, const bf16x8& a, const bf16x8& b) {
	asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));
}

template <int EPI>
__global__ __launch_bounds__(256) void gemm_pers_kernel(Args g) {
	using Sh = Shape<4, 4>;
	constexpr int BM = 256, RT = 4, RF = 8, NST = 2, A_BYTES = Sh::A_BYTES, STAGE_BYTES = Sh::STAGE_BYTES;
	constexpr int LOADS_A = Sh::LOADS_A, LOADS_B = Sh::LOADS_B, LOADS_PER_STAGE = Sh::LOADS_PER_STAGE, HALF = LOADS_PER_STAGE / 2;
	constexpr bool PAIRED = EPI == EPI_BF16_SWIGLU;
	static_assert(Sh::NST == 2 && LOADS_A == 8 && LOADS_B == 8, "ring of two 64 KiB stages");
	extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wr = wave >> 1, wc = wave & 1;
	const int ntiles = g.tiles_m * g.tiles_n;
	const int nk = g.K / BKS;  // even

	uint32_t aoff[LOADS_A], boff[LOADS_B];
	lane_offsets<false, LOADS_A, false, BM>(wave, lane, g.lda, aoff);
	lane_offsets_rb<PAIRED>(wave, lane, g.ldb, boff, g.N / 2);
	const uint32_t lds_a = lds_addr(smem) + wave * (LOADS_A * 1024);
	const uint32_t lds_b = lds_addr(smem) + NST * A_BYTES + wave * (LOADS_B * 1024);
	const uint32_t lds_dummy = lds_addr(smem) + NST * STAGE_BYTES;

	auto tile_ptrs = [&](int tile, int& m0, int& n0, const bf16_t*& Ap, const bf16_t*& Bp) {
		tile_origin<BM>(g, tile, m0, n0);
		m0 = __builtin_amdgcn_readfirstlane(m0);
		n0 = __builtin_amdgcn_readfirstlane(n0);
		Ap = g.A + (int64_t)m0 * g.lda;
		Bp = g.B + (int64_t)(PAIRED ? n0 / 2 : n0) * g.ldb;
	};
	int tile = blockIdx.x, m0, n0, m0_n = 0, n0_n = 0;
	const bf16_t *Ap, *Bp, *Ap_n, *Bp_n;
	tile_ptrs(tile, m0, n0, Ap, Bp);
	Ap_n = Ap, Bp_n = Bp;
	bool has_next = false;

	struct SliceLoads {
		const bf16_t* pa;
		const bf16_t* pb;
		uint32_t la, lb;
	};
	// slice `step` of the current tile; steps nk and nk + 1 are slices 0 and 1 of the next tile (same ring stage: nk is
	// even), or, behind the workgroup's last tile, loads nobody reads into the scratch area behind the ring
	auto slice_loads = [&](int step) {
		const bool cur = step < nk;
		const int sc = cur ? step : step - nk;
		const bool ok = cur || has_next;
		const uint32_t st = (uint32_t)(sc & 1);
		return SliceLoads{(cur ? Ap : Ap_n) + (int64_t)sc * BKS, (cur ? Bp : Bp_n) + (int64_t)sc * BKS, ok ? lds_a + st * A_BYTES : lds_dummy,
		                  ok ? lds_b + st * B_BYTES : lds_dummy};
	};
	auto issue_piece = [&](const SliceLoads& sl, auto pc) {
		constexpr int P = decltype(pc)::value;
		if constexpr (P < LOADS_A) dma16_at<P * 1024>(sl.pa, aoff[P], sl.la);
		else dma16_at<(P - LOADS_A) * 1024>(sl.pb, boff[P - LOADS_A], sl.lb);
	};

	f32x4 acc[RF][8];
	bf16x8 fa[2][RF], fb[2][4];
	static_assert(pieces_have_slots(RF * 4, HALF), "a half-step has too few even MFMA slots for half a slice's loads");
	{
		const SliceLoads s0 = slice_loads(0);
		static_for<LOADS_PER_STAGE>([&](auto pc) { issue_piece(s0, pc); });
		const SliceLoads s1 = slice_loads(1);
		static_for<HALF>([&](auto pc) { issue_piece(s1, pc); });
		wait_vmcnt<HALF>();
	}
	__syncthreads();
	// Per-lane LDS addresses of the fragment reads for the two k32 halves of a slice (the chunk swizzles only look at
	// lane bits); stage, row slab and column slab are compile-time byte offsets in the read instructions.
	uint32_t a_lane[2], b_lane[2];
	{
		const int l15 = lane & 15, q4 = lane >> 4;
#pragma unroll
		for (int kq = 0; kq < 2; kq++) {
			a_lane[kq] = lds_addr(smem) + (uint32_t)((wr * 128 + l15) * 128 + (((4 * kq + q4) ^ ((l15 >> 1) & 7)) << 4));
			b_lane[kq] = lds_addr(smem) + NST * A_BYTES + (uint32_t)((wc * 128 + 8 * (l15 >> 2) + (l15 & 3)) * 128 + (((4 * kq + q4) ^ rb_swz(8 * (l15 >> 2) + (l15 & 3))) << 4));
			asm volatile("" : "+v"(a_lane[kq]), "+v"(b_lane[kq]));
		}
	}
	auto read_a = [&](auto stage, int kq, auto ic) -> bf16x8 {
		constexpr uint32_t IMM = decltype(stage)::value * A_BYTES + decltype(ic)::value * (16 * 128);
		return *reinterpret_cast<const bf16x8 ELF_LDS*>((uintptr_t)(a_lane[kq] + IMM));
	};
	auto read_b = [&](auto stage, int kq, int h, auto jc) -> bf16x8 {
		constexpr int JJ = decltype(jc)::value;
		constexpr uint32_t IMM = decltype(stage)::value * B_BYTES + (32 * (JJ >> 1) + 4 * (JJ & 1)) * 128;
		return *reinterpret_cast<const bf16x8 ELF_LDS*>((uintptr_t)(b_lane[kq] + IMM + (uint32_t)h * (64 * 128)));
	};
	static_for<RF>([&](auto ic) { fa[0][decltype(ic)::value] = read_a(std::integral_constant<int, 0>{}, 0, ic); });
	static_for<4>([&](auto jc) { fb[0][decltype(jc)::value] = read_b(std::integral_constant<int, 0>{}, 0, 0, jc); });

	// One half-step (see gemm_dma_kernel): RF * 4 MFMAs, the next half-step's fragment reads behind the odd ones, half of
	// a slice's loads behind even ones.  FIRST: the accumulator tiles of this half-step are written, not added to.
	auto half_step = [&](int abuf, int bbuf, auto hc, auto first, int pb_buf, auto pb_stage, int pb_kq, int pb_h, bool pa, int pa_buf, auto pa_stage, int pa_kq,
	                     const SliceLoads& sl, auto piece0) {
		constexpr int PIECE0 = decltype(piece0)::value, H = decltype(hc)::value, NM = RF * 4;
		constexpr int SA = decltype(pa_stage)::value, SB = decltype(pb_stage)::value;
		constexpr bool FIRST = decltype(first)::value;
		static_for<NM>([&](auto nc) {
			constexpr int n = decltype(nc)::value, i = n / 4, j = n % 4;
			if constexpr (FIRST) mfma_init(acc[i][H * 4 + j], fb[bbuf][j], fa[abuf][i]);
			else mfma_acc(acc[i][H * 4 + j], fb[bbuf][j], fa[abuf][i]);
			if constexpr (n % 2 == 1) {
				constexpr int r = n / 2;
				if constexpr (r < 4) {
					fb[pb_buf][r] = read_b(std::integral_constant<int, SB>{}, pb_kq, pb_h, std::integral_constant<int, r>{});
				} else if constexpr (r - 4 < RF) {
					if (pa) fa[pa_buf][r - 4] = read_a(std::integral_constant<int, SA>{}, pa_kq, std::integral_constant<int, r - 4>{});
				}
			}
			if constexpr (PIECE0 >= 0 && piece_in_slot(n, NM, HALF) >= 0) issue_piece(sl, std::integral_constant<int, (PIECE0 < 0 ? 0 : PIECE0) + (piece_in_slot(n, NM, HALF) < 0 ? 0 : piece_in_slot(n, NM, HALF))>{});
			__builtin_amdgcn_sched_barrier(0);
		});
	};
	auto slice = [&](auto sc, auto first, int kt) {
		constexpr int S = decltype(sc)::value;
		constexpr std::integral_constant<int, S> CUR{};
		constexpr std::integral_constant<int, (S + 1) % NST> NXT{};
		constexpr std::integral_constant<int, 0> H0{};
		constexpr std::integral_constant<int, 1> H1{};
		constexpr std::integral_constant<int, -1> NO_DMA{};
		constexpr std::false_type ADD{};
		const SliceLoads next1 = slice_loads(kt + 1), next2 = slice_loads(kt + 2);
		half_step(0, 0, H0, first, 1, CUR, 0, 1, false, 0, CUR, 0, next1, std::integral_constant<int, HALF>{});
		half_step(0, 1, H1, first, 0, CUR, 1, 0, true, 1, CUR, 1, next1, NO_DMA);
		half_step(1, 0, H0, ADD, 1, CUR, 1, 1, false, 0, CUR, 0, next1, NO_DMA);
		wait_counters<0, 0>();  // slice kt + 1 landed (and the previous tile's stores acknowledged); slice kt fully read
		__syncthreads();
		half_step(1, 1, H1, ADD, 0, NXT, 0, 0, true, 0, NXT, 0, next2, std::integral_constant<int, 0>{});
	};

	const int g4 = lane >> 4, rr = lane & 15;
	for (;;) {
		const int tile_n = tile + (int)gridDim.x;
		has_next = tile_n < ntiles;
		if (has_next) tile_ptrs(tile_n, m0_n, n0_n, Ap_n, Bp_n);

		slice(std::integral_constant<int, 0>{}, std::true_type{}, 0);
		slice(std::integral_constant<int, 1>{}, std::false_type{}, 1);
		for (int kt = 2; kt < nk; kt += 2) {
			slice(std::integral_constant<int, 0>{}, std::false_type{}, kt);
			slice(std::integral_constant<int, 1>{}, std::false_type{}, kt + 1);
		}

		// Epilogue from registers, while the next tile's first two slices are on their way into the ring.  The MFMAs were
		// issued through inline assembly, so the compiler places no wait states between the last of them and the first
		// read of an accumulator: 32 of them here (an 8-pass MFMA needs 11).
		asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
		const int grow0 = m0 + wr * 128 + rr;
		const int gcol0 = n0 + wc * 128;
		// the lane's run t (0..3) of 8 consecutive columns: columns (t / 2) * 64 + (t % 2) * 32 + 8 g4 .. + 7 of the wave's 128
		auto run = [&](int i, int t, float (&v)[8]) {
#pragma unroll
			for (int e = 0; e < 8; e++) v[e] = acc[i][(t >> 1) * 4 + (t & 1) * 2 + (e >> 2)][e & 3];
		};
		auto run_col = [&](int t) { return (t >> 1) * 64 + (t & 1) * 32 + g4 * 8; };
		if constexpr (EPI == EPI_BF16_SWIGLU) {
			// the wave's columns are 64 gate columns (first half-step) and the 64 up columns of the same outputs (second)
			const int F = g.N / 2, cg0 = n0 / 2 + wc * 64;
#pragma unroll
			for (int i = 0; i < RF; i++) {
				__builtin_amdgcn_sched_barrier(0);  // one row group at a time (see the residual epilogue below)
				const int64_t row = grow0 + i * 16;
#pragma unroll
				for (int t = 0; t < 2; t++) {
					float gv[8], uv[8];
					run(i, t, gv);
					run(i, 2 + t, uv);
					bf16x8 og, ou, oa;
#pragma unroll
					for (int e = 0; e < 8; e++) {
						og[e] = (bf16_t)gv[e];
						ou[e] = (bf16_t)uv[e];
						oa[e] = (bf16_t)swiglu_f((float)og[e], (float)ou[e]);
					}
					const int c = cg0 + t * 32 + g4 * 8;
					bf16_t* cp = reinterpret_cast<bf16_t*>(g.C) + row * g.ldc + c;
					*reinterpret_cast<bf16x8*>(cp) = og;
					*reinterpret_cast<bf16x8*>(cp + F) = ou;
					*reinterpret_cast<bf16x8*>(g.C2 + row * g.ldc2 + c) = oa;
				}
			}
		} else {
			static_assert(EPI == EPI_BF16 || EPI == EPI_BF16_RESID, "epilogues of the persistent forward kernel");
			// residual (or bias row, ldr = 0): every load of the wave's 128 x 128 share goes out before the first store (a lone
			// wave has nothing else to cover the trips to memory with; inside the store loop each would be awaited alone)
			bf16x8 rs[EPI == EPI_BF16_RESID ? RF : 1][4];
			if constexpr (EPI == EPI_BF16_RESID) {
#pragma unroll
				for (int i = 0; i < RF; i++)
#pragma unroll
					for (int t = 0; t < 4; t++) rs[i][t] = *reinterpret_cast<const bf16x8*>(g.R + (int64_t)(grow0 + i * 16) * g.ldr + gcol0 + run_col(t));
			}
			// (left to itself the scheduler reads all 256 accumulators into vector registers first and then has room for
			// two loads at a time: the row groups are fenced off from each other and from the loads)
			__builtin_amdgcn_sched_barrier(0);
#pragma unroll
			for (int i = 0; i < RF; i++) {
				__builtin_amdgcn_sched_barrier(0);
				bf16_t* cp = reinterpret_cast<bf16_t*>(g.C) + (int64_t)(grow0 + i * 16) * g.ldc + gcol0;
#pragma unroll
				for (int t = 0; t < 4; t++) {
					float v[8];
					run(i, t, v);
					bf16x8 o;
#pragma unroll
					for (int e = 0; e < 8; e++) {
						if constexpr (EPI == EPI_BF16_RESID) v[e] += (float)rs[i][t][e];
						o[e] = (bf16_t)v[e];
					}
					*reinterpret_cast<bf16x8*>(cp + run_col(t)) = o;
				}
			}
		}
		if (!has_next) break;
		tile = tile_n, m0 = m0_n, n0 = n0_n, Ap = Ap_n, Bp = Bp_n;
		asm volatile("s_nop 7" ::: "memory");  // accumulator reads above, accumulator writes by the next tile's first MFMAs
	}
	wait_vmcnt<0>();  // the loads past the last tile land in LDS too
}

template <int EPI>
static int launch_pers(const Args& a, hipStream_t stream) {
	using Sh = Shape<4, 4>;
	constexpr int smem = Sh::NST * Sh::STAGE_BYTES + Sh::LOADS_A * 1024;
	auto kern = gemm_pers_kernel<EPI>;
	static bool attr_set = false;
	if (!attr_set) {
		ELF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
		attr_set = true;
	}
	const int ntiles = a.tiles_m * a.tiles_n;
	ELF_LAUNCH(kern, dim3(ntiles < PERS_WORKGROUPS ? ntiles : PERS_WORKGROUPS), dim3(256), smem, stream, a);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}


// The split tiles of a launch with the scaling accumulate epilogue: their workgroups add partial sums and none of them
// holds the finished tile, so the scale and the bf16 copy of those (few, at most 128) tiles are applied here, behind the
// GEMM on the same stream.  Eight workgroups per tile (32 rows each); tile index and origin as in the GEMM.
__global__ __launch_bounds__(256) void scale_tail_kernel(Args g) {
	const int ntiles = g.tiles_m * g.tiles_n;
	const int pid = ntiles - g.tail_tiles + (int)(blockIdx.x >> 3);
	int m0, n0;
	tile_origin<256>(g, pid, m0, n0);
	m0 += (int)(blockIdx.x & 7) * 32;
	float* C = reinterpret_cast<float*>(g.C);
	for (int i = threadIdx.x; i < 32 * 64; i += 256) {
		const int row = i >> 6, c4 = (i & 63) * 4;
		float* c = C + (int64_t)(m0 + row) * g.ldc + n0 + c4;
		f32x4 v = *reinterpret_cast<const f32x4*>(c);
		v *= g.scale;
		bf16x4 o;
#pragma unroll
		for (int t = 0; t < 4; t++) o[t] = (bf16_t)v[t];
		*reinterpret_cast<f32x4*>(c) = v;
		*reinterpret_cast<bf16x4*>(g.C2 + (int64_t)(m0 + row) * g.ldc2 + n0 + c4) = o;
	}
}

template <int NW, int RT, bool AT, bool BT, int EPI>
static int launch(const Args& a, hipStream_t stream) {
	// the ring + the target of the loads past the end of K (as many KiB as a wave issues loads per
	// operand); the epilogue needs a 32 x 136 fp32 strip per wave
	using Sh = Shape<NW, RT>;
	constexpr int ring = Sh::NST * Sh::STAGE_BYTES + (Sh::LOADS_A > Sh::LOADS_B ? Sh::LOADS_A : Sh::LOADS_B) * 1024, epi = NW * 32 * 136 * 4;
	constexpr int smem = ring > epi ? ring : epi;
	auto kern = gemm_dma_kernel<NW, RT, AT, BT, EPI>;
	static bool attr_set = false;
	if (!attr_set) {
		ELF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
		attr_set = true;
	}
	ELF_LAUNCH(kern, dim3(a.tiles_m * a.tiles_n + a.tail_tiles * (a.k_splits - 1)), dim3(NW * 64), smem, stream, a);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

template <int NW, int RT, bool AT, bool BT>
static int launch_epi(const Args& a, int epi, hipStream_t stream) {
	switch (epi) {
		case EPI_BF16: return launch<NW, RT, AT, BT, EPI_BF16>(a, stream);
		case EPI_BF16_RESID: return launch<NW, RT, AT, BT, EPI_BF16_RESID>(a, stream);
		case EPI_F32_ACC: return launch<NW, RT, AT, BT, EPI_F32_ACC>(a, stream);
		case EPI_F32_STORE: return launch<NW, RT, AT, BT, EPI_F32_STORE>(a, stream);
	}
	if constexpr (!AT && !BT) {
		if (epi == EPI_BF16_SWIGLU) return launch<NW, RT, AT, BT, EPI_BF16_SWIGLU>(a, stream);
		if (epi == EPI_BF16_ROPE) return launch<NW, RT, AT, BT, EPI_BF16_ROPE>(a, stream);
	}
	if constexpr (NW == 4 && RT == 4 && !AT && BT) {
		if (epi == EPI_BF16_SWIGLU_BWD) return launch<NW, RT, AT, BT, EPI_BF16_SWIGLU_BWD>(a, stream);
	}
	if constexpr (NW == 8 && AT && BT) {
		if (epi == EPI_F32_ACC_SCALE) return launch<NW, RT, AT, BT, EPI_F32_ACC_SCALE>(a, stream);
	}
	set_error("gemm: unknown epilogue %d", epi);
	return -1;
}

}  // namespace dma

// Waves of this file's kernels that stopped waiting for their turn since the library was loaded (this device).
int dma_turn_giveups(uint64_t* out) {
	unsigned int n = 0;
	ELF_CHECK_HIP(hipMemcpyFromSymbol(&n, HIP_SYMBOL(dma::turn_giveups), sizeof(n)));
	*out = n;
	return 0;
}

// Arguments are validated by gemm_bf16() before it dispatches here.
int gemm_bf16_dma(int a_t, int b_t, int M, int N, int K, const void* A, int64_t lda, const void* B, int64_t ldb, void* C,
                  int64_t ldc, int epi, const void* R, int64_t ldr, int k_splits, int tail_tiles, int bm, hipStream_t stream,
                  void* C2, int64_t ldc2, const void* rope_cs, int rope_S, int rope_cols, int rope_D, float scale) {
	ELF_REQUIRE(bm == 256 || bm == 128, "gemm (dma tile): 256- or 128-row tiles");
	ELF_REQUIRE(M % bm == 0 && N % dma::BN == 0 && K % dma::BKS == 0, "gemm (dma tile): M multiple of %d, N of 256 and K of 64 required", bm);
	const int ntiles = (M / bm) * (N / dma::BN);
	ELF_REQUIRE(epi != EPI_BF16_SWIGLU || (C2 && !a_t && !b_t), "gemm (dma tile): the SwiGLU epilogue needs k-contiguous operands and a second output");
	// the paired rows of the SwiGLU epilogue are addressed with 32-bit byte offsets from the tile's first row
	ELF_REQUIRE(epi != EPI_BF16_SWIGLU || (int64_t)(N / 2 + 256) * ldb * 2 < (int64_t(1) << 31), "gemm (dma tile): weight too large for the paired-row epilogue");
	ELF_REQUIRE(epi != EPI_F32_ACC_SCALE || (C2 && a_t && b_t && bm == 256), "gemm (dma tile): the scaling accumulate epilogue needs reduction-major operands, 256-row tiles and a bf16 output");
	ELF_REQUIRE(epi != EPI_BF16_ROPE || (rope_cs && rope_S > 0 && !a_t && !b_t && (rope_D == 64 || rope_D == 128) && rope_cols % rope_D == 0 && rope_cols <= N),
	            "gemm (dma tile): the RoPE epilogue needs k-contiguous operands, a table and heads of 64 or 128 columns");
	dma::Args a{(const bf16_t*)A, (const bf16_t*)B, C, (const bf16_t*)R, (bf16_t*)C2, lda, ldb, ldc, ldr, ldc2, M, N, K, M / bm, N / dma::BN, k_splits < 1 ? 1 : k_splits,
	            tail_tiles < 0 || tail_tiles > ntiles ? ntiles : tail_tiles, 0, (const float2*)rope_cs, rope_S, rope_cols, rope_D, 0, scale};
	// The band walk fetches every row slab of A from HBM in one round only and B once per band; the default
	// walk wants A in the 256 MB memory-side cache for the whole launch and streams B once.  Inside the stage's
	// stream (operands cold, per-shape times from a kernel trace) the bands are 0-5 % faster on every shape but
	// the one with a small A and a B beyond that cache (gate/up projection forward, 67 MB against 235 MB: 2 %
	// slower), which keeps the default.
	const int64_t big = int64_t(160) << 20;
	a.walk = !((int64_t)M * K * 2 < big && (int64_t)N * K * 2 >= big);
	if ((epi != EPI_F32_ACC && epi != EPI_F32_ACC_SCALE) || a.k_splits == 1) a.k_splits = 1, a.tail_tiles = 0;
	// split tiles add in a fixed order (bit-reproducible weight gradients) as long as each has a counter of its own
	a.turn_tag = a.tail_tiles > 0 && a.tail_tiles <= dma::TURN_TILES ? next_turn_tag() : 0;
	a.turn_base = a.turn_tag * 977u;  // consecutive launches on different counters
	if (bm == 128) {
		if (!a_t && !b_t) return dma::launch_epi<4, 2, false, false>(a, epi, stream);
		if (!a_t && b_t) return dma::launch_epi<4, 2, false, true>(a, epi, stream);
		if (a_t && b_t) return dma::launch_epi<4, 2, true, true>(a, epi, stream);
		set_error("gemm: layout A=T,B=R is not used by any stage contraction");
		return -1;
	}
	// k-contiguous A (forward, dX): four waves with 128x128 wave tiles; both operands reduction-major (dW): eight
	// waves with 64x128 wave tiles (with two transpose reads per fragment on both operands the lone wave wins on
	// some shapes by 2-3 % and loses on most by 1-10 %)
	if (!a_t && !b_t && (K / dma::BKS) % 2 == 0 && !getenv("ELF_NO_PERSISTENT_GEMM")) {
		// forward shapes: persistent workgroups, register epilogue (the QKV projection with its rotary epilogue stays on the
		// one-tile kernel: with the table fetches in a lone wave's register epilogue the persistent form ran 3 % slower)
		switch (epi) {
			case EPI_BF16: return dma::launch_pers<EPI_BF16>(a, stream);
			case EPI_BF16_RESID: return dma::launch_pers<EPI_BF16_RESID>(a, stream);
			case EPI_BF16_SWIGLU: return dma::launch_pers<EPI_BF16_SWIGLU>(a, stream);
		}
	}
	if (!a_t && !b_t) return dma::launch_epi<4, 4, false, false>(a, epi, stream);
	if (!a_t && b_t) return dma::launch_epi<4, 4, false, true>(a, epi, stream);
	if (a_t && b_t) {
		if (int rc = dma::launch_epi<8, 2, true, true>(a, epi, stream)) return rc;
		if (epi == EPI_F32_ACC_SCALE && a.tail_tiles > 0) {
			ELF_LAUNCH(dma::scale_tail_kernel, dim3(a.tail_tiles * 8), dim3(256), 0, stream, a);
			ELF_CHECK_HIP(hipGetLastError());
		}
		return 0;
	}
	set_error("gemm: layout A=T,B=R is not used by any stage contraction");
	return -1;
}

bool gemm_dw_groupable(int M, int N, int K, const void* dY, int64_t lddy, const void* X, int64_t ldx, const void* acc) {
	return M > 0 && N > 0 && K > 0 && M % 256 == 0 && N % dma::BN == 0 && K % dma::BKS == 0 && lddy % 8 == 0 && ldx % 8 == 0 && lddy >= M && ldx >= N &&
	       ((uintptr_t)dY % 16) == 0 && ((uintptr_t)X % 16) == 0 && ((uintptr_t)acc % 16) == 0;
}

int gemm_dw_group(int n, const DwProblem* pr, int K, float scale, hipStream_t stream) {
	ELF_REQUIRE(n > 0 && n <= dma::GROUP_MAX && pr, "gemm_dw_group: 1..%d problems", dma::GROUP_MAX);
	int64_t tiles = 0;
	double flops = 0;
	for (int i = 0; i < n; i++) {
		ELF_REQUIRE(pr[i].dY && pr[i].X && pr[i].acc && gemm_dw_groupable(pr[i].M, pr[i].N, K, pr[i].dY, pr[i].lddy, pr[i].X, pr[i].ldx, pr[i].acc),
		            "gemm_dw_group: problem %d (M=%d N=%d K=%d) needs M, N multiples of 256, K of 64 and 16-byte aligned operands", i, pr[i].M, pr[i].N, K);
		ELF_REQUIRE(scale == 0.f || (pr[i].grad_bf16 && ((uintptr_t)pr[i].grad_bf16 % 8) == 0), "gemm_dw_group: a scaling pass needs the bf16 gradient buffers");
		tiles += (int64_t)(pr[i].M / 256) * (pr[i].N / dma::BN);
		flops += 2.0 * pr[i].M * pr[i].N * K;
	}
	// Whole tiles, one workgroup each, except in the launch's last round: when that round would fill at most half of the
	// chip, its tiles (the last ones of the last problems) are split along K so that proportionally shorter workgroups
	// fill it - at least 16 K slices each, and no more than 8 ways (the splits of a tile add with atomics, one after the
	// other: past that their adds cost more than the idle compute units).
	const int nk = K / dma::BKS;
	int splits = 1, tail = 0;
	if (const int rem = (int)(tiles % 256); rem != 0 && rem <= 128 && rem <= dma::TURN_TILES) {
		splits = 256 / rem < 8 ? 256 / rem : 8;
		while (splits > 1 && nk / splits < 16) splits--;
		if (splits > 1) tail = rem;
	}
	dma::GroupArgs ga{};
	ga.n = n;
	ga.compact = 1;
	for (int i = 0; i < n; i++)
		if ((pr[i].M / 256) * (pr[i].N / dma::BN) >= 256) ga.compact = 0;
	ga.tiles = (int)tiles, ga.tail = tail, ga.splits = splits;
	const uint32_t tag = tail ? next_turn_tag() : 0;
	uint32_t turn_base = tag * 977u;
	ga.turn_base = turn_base;
	const int64_t big = int64_t(160) << 20;
	int64_t before = 0;  // tiles of the problems ahead of this one
	int next = 0;
	for (int i = 0; i < n; i++) {
		const DwProblem& q = pr[i];
		const int ntiles = (q.M / 256) * (q.N / dma::BN);
		// this problem's share of the launch's last `tail` tiles
		const int64_t tail_from = tiles - tail;
		const int tail_i = before + ntiles <= tail_from ? 0 : (int)(before + ntiles - (tail_from > before ? tail_from : before));
		dma::Args& a = ga.a[i];
		a = dma::Args{(const bf16_t*)q.dY, (const bf16_t*)q.X, q.acc, nullptr, (bf16_t*)q.grad_bf16, q.lddy, q.ldx, q.N, 0, q.N, q.M, q.N, K, q.M / 256, q.N / dma::BN,
		              tail_i ? splits : 1, tail_i, 0, nullptr, 0, 0, 0, tail_i ? tag : 0, scale, turn_base};
		a.walk = ga.compact ? 2 : !((int64_t)q.M * K * 2 < big && (int64_t)q.N * K * 2 >= big);
		turn_base += (uint32_t)tail_i;
		ga.first[i] = ga.compact ? (int)before : next;
		ga.count[i] = ntiles + tail_i * (splits - 1);
		next += (ga.count[i] + 7) & ~7;
		before += ntiles;
	}
	if (ga.compact) next = 8 * (int)((tiles - tail + 7) / 8 + (tail + 7) / 8 * splits);
	{
		ProfScope prof(PROF_GEMM, flops, stream);
		using Sh = dma::Shape<8, 2>;
		constexpr int ring = Sh::NST * Sh::STAGE_BYTES + (Sh::LOADS_A > Sh::LOADS_B ? Sh::LOADS_A : Sh::LOADS_B) * 1024, epi = 8 * 32 * 136 * 4;
		constexpr int smem = ring > epi ? ring : epi;
		static bool attr_set = false;
		if (!attr_set) {
			ELF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dma::gemm_dw_group_kernel<EPI_F32_ACC>), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
			ELF_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dma::gemm_dw_group_kernel<EPI_F32_ACC_SCALE>), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
			attr_set = true;
		}
		if (scale != 0.f) ELF_LAUNCH(dma::gemm_dw_group_kernel<EPI_F32_ACC_SCALE>, dim3(next), dim3(512), smem, stream, ga);
		else ELF_LAUNCH(dma::gemm_dw_group_kernel<EPI_F32_ACC>, dim3(next), dim3(512), smem, stream, ga);
		ELF_CHECK_HIP(hipGetLastError());
	}
	// split tiles have no single epilogue that could scale them: a small kernel behind the launch does those
	if (scale != 0.f)
		for (int i = 0; i < n; i++)
			if (ga.a[i].tail_tiles > 0) {
				ELF_LAUNCH(dma::scale_tail_kernel, dim3(ga.a[i].tail_tiles * 8), dim3(256), 0, stream, ga.a[i]);
				ELF_CHECK_HIP(hipGetLastError());
			}
	return 0;
}

}  // namespace elf
