// Bandwidth-bound kernels of a transformer-block stage on gfx950: RMSNorm / LayerNorm,
// GELU, SwiGLU, RoPE, gradient scale.  All tensors are bf16 row-major [T, cols]; math is
// fp32 with one rounding on store.  Every lane moves 16 bytes per access (8 bf16) so that
// a wavefront reads 1 KiB contiguous; row reductions are wavefront butterflies (one wave
// per row, the row is held in registers so each input is read from HBM exactly once).
//
// These replace the ATen ops the reference stage runs through autograd
// (benchmarks/models/simple.py:44-52 GELU FFN, :444-445 LayerNorm, :460/:466 residual adds;
// elf/execution/block.py:518-527 scale_grads).  RMSNorm, RoPE and SwiGLU have no reference
// module; their definitions are the textbook ones stated next to each kernel.
#include <atomic>
#include <mutex>

#include "common.h"
#include "kernels.h"

namespace elf {

constexpr int ROWS_PER_BLOCK = 4;  // one wave per row, 4 waves per workgroup

struct Chunk {
	float v[8];
};

__device__ __forceinline__ Chunk load8(const bf16_t* p) {
	bf16x8 r = *reinterpret_cast<const bf16x8*>(p);
	Chunk c;
#pragma unroll
	for (int i = 0; i < 8; i++) c.v[i] = (float)r[i];
	return c;
}
__device__ __forceinline__ void store8(bf16_t* p, const Chunk& c) {
	bf16x8 r;
#pragma unroll
	for (int i = 0; i < 8; i++) r[i] = (bf16_t)c.v[i];
	*reinterpret_cast<bf16x8*>(p) = r;
}

// ------------------------------------------------------------------------------------------
// Norm forward.  RMS:  y = x * rsqrt(mean(x^2) + eps) * gamma
//                LN :  y = (x - mean) * rsqrt(var + eps) * gamma + beta   (biased variance)
// stats[row] = {mean (0 for RMS), rstd}.
// WPR = waves per row: 1 (four rows per workgroup, d <= 2048) or 4 (one row per workgroup).
// One output element of the norm from its row statistics: shared by the forward kernels and by the backward kernel that
// forms a dropped output again, so that both give the same bits (LN: one fused multiply-add for gamma and beta).
template <bool LN>
__device__ __forceinline__ float norm_out(float x, float mean, float rstd, float g, float b) {
	return LN ? __builtin_fmaf((x - mean) * rstd, g, b) : x * rstd * g;
}

template <int WPR>
__device__ __forceinline__ float row_sum(float v, float* red) {
	v = wave_sum(v);
	if constexpr (WPR > 1) {
		const int wave = threadIdx.x >> 6;
		__syncthreads();
		if ((threadIdx.x & 63) == 0) red[wave] = v;
		__syncthreads();
		v = red[0] + red[1] + red[2] + red[3];
	}
	return v;
}

template <int NCH, int WPR, bool LN>
__global__ __launch_bounds__(256) void norm_fwd_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ gamma,
                                                       const bf16_t* __restrict__ beta, bf16_t* __restrict__ y,
                                                       float2* __restrict__ stats, int T, int d, float eps) {
	__shared__ float red[4];
	const int tr = WPR == 1 ? (threadIdx.x & 63) : threadIdx.x;  // thread index within the row
	constexpr int TPR = 64 * WPR;
	const int row = WPR == 1 ? blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6) : blockIdx.x;
	if (row >= T) return;  // uniform per wave (WPR == 1) or per workgroup (WPR == 4)
	const int nchunks = d >> 3;
	const bf16_t* xr = x + (int64_t)row * d;
	Chunk c[NCH];
	float s = 0.f, ss = 0.f;
#pragma unroll
	for (int i = 0; i < NCH; i++) {
		const int ch = tr + i * TPR;
		if (ch < nchunks) {
			c[i] = load8(xr + ch * 8);
#pragma unroll
			for (int j = 0; j < 8; j++) {
				s += c[i].v[j];
				ss += c[i].v[j] * c[i].v[j];
			}
		}
	}
	float mean = 0.f, rstd;
	if (LN) {
		mean = row_sum<WPR>(s, red) / d;
		// second pass over registers for the variance (numerically safer than E[x^2]-mean^2)
		float var = 0.f;
#pragma unroll
		for (int i = 0; i < NCH; i++) {
			if (tr + i * TPR < nchunks) {
#pragma unroll
				for (int j = 0; j < 8; j++) {
					const float t = c[i].v[j] - mean;
					var += t * t;
				}
			}
		}
		rstd = rsqrtf(row_sum<WPR>(var, red) / d + eps);
	} else {
		rstd = rsqrtf(row_sum<WPR>(ss, red) / d + eps);
	}
	if (tr == 0) stats[row] = make_float2(mean, rstd);
	bf16_t* yr = y + (int64_t)row * d;
#pragma unroll
	for (int i = 0; i < NCH; i++) {
		const int ch = tr + i * TPR;
		if (ch < nchunks) {
			Chunk g = load8(gamma + ch * 8);
			Chunk o, b;
			if (LN) b = load8(beta + ch * 8);
#pragma unroll
			for (int j = 0; j < 8; j++) o.v[j] = norm_out<LN>(c[i].v[j], mean, rstd, g.v[j], LN ? b.v[j] : 0.f);
			store8(yr + ch * 8, o);
		}
	}
}

// Norm backward.  With xhat = (x - mean) * rstd, g = dy * gamma:
//   RMS: dx = rstd * (g - xhat * mean(g * xhat))
//   LN : dx = rstd * (g - mean(g) - xhat * mean(g * xhat))
// dx (+)= dres when a residual gradient bypasses the norm.  Per-workgroup partial sums of
// dgamma (= sum dy*xhat) and dbeta (= sum dy) go to part[blockIdx][2][d]; a second kernel
// folds them into the fp32 gradient accumulators.  YOUT: the norm's output y (a stash that dropped it after the forward)
// is written again as well, from the row the kernel holds anyway: the forward's arithmetic, the forward's bits.
template <int NCH, int WPR, bool LN, bool YOUT>
__global__ __launch_bounds__(256) void norm_bwd_kernel(const bf16_t* __restrict__ dy, const bf16_t* __restrict__ x,
                                                       const bf16_t* __restrict__ gamma,
                                                       const float2* __restrict__ stats,
                                                       const bf16_t* __restrict__ dres, bf16_t* __restrict__ dx,
                                                       float* __restrict__ part, int T, int d,
                                                       const bf16_t* __restrict__ beta, bf16_t* __restrict__ yout) {
	__shared__ float red[4];
	__shared__ float fold[WPR == 1 ? ROWS_PER_BLOCK : 1][WPR == 1 ? 64 * 8 : 1];
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int tr = WPR == 1 ? lane : threadIdx.x;
	constexpr int TPR = 64 * WPR;
	const int nchunks = d >> 3;
	Chunk g[NCH];
	float dg[NCH][8], db[NCH][8];
#pragma unroll
	for (int i = 0; i < NCH; i++) {
		const int ch = tr + i * TPR;
		if (ch < nchunks) g[i] = load8(gamma + ch * 8);
#pragma unroll
		for (int j = 0; j < 8; j++) dg[i][j] = db[i][j] = 0.f;
	}
	const int row_step = WPR == 1 ? gridDim.x * ROWS_PER_BLOCK : gridDim.x;
	// the next row's operands (dy, x, the residual gradient, the row statistics) are fetched while the current row is
	// reduced: a row costs two or three trips through the workgroup's reduction, during which nothing else would be in flight
	bf16x8 nx[NCH], ndy[NCH], nres[NCH];  // the row in flight
	float2 nst = make_float2(0.f, 0.f);
	auto fetch = [&](int r) {
		if (r < T) {
			nst = stats[r];
#pragma unroll
			for (int i = 0; i < NCH; i++) {
				const int ch = tr + i * TPR;
				if (ch < nchunks) {
					nx[i] = *reinterpret_cast<const bf16x8*>(x + (int64_t)r * d + ch * 8);
					ndy[i] = *reinterpret_cast<const bf16x8*>(dy + (int64_t)r * d + ch * 8);
					if (dres) nres[i] = *reinterpret_cast<const bf16x8*>(dres + (int64_t)r * d + ch * 8);
				}
			}
		}
	};
	int row = WPR == 1 ? blockIdx.x * ROWS_PER_BLOCK + wave : blockIdx.x;
	fetch(row);
	for (; row < T; row += row_step) {
		// the current row stays in its 16-bit form; xhat and dy * gamma are formed again for dx rather than kept as floats
		bf16x8 rx[NCH], rdy[NCH], rres[NCH];
		const float mean = nst.x, rstd = nst.y;
#pragma unroll
		for (int i = 0; i < NCH; i++) rx[i] = nx[i], rdy[i] = ndy[i], rres[i] = nres[i];
		fetch(row + row_step);
		float s1 = 0.f, s2 = 0.f;
#pragma unroll
		for (int i = 0; i < NCH; i++) {
			const int ch = tr + i * TPR;
			if (ch < nchunks) {
#pragma unroll
				for (int j = 0; j < 8; j++) {
					const float xhat = ((float)rx[i][j] - mean) * rstd;
					const float dyv = (float)rdy[i][j];
					dg[i][j] += dyv * xhat;
					if (LN) db[i][j] += dyv;
					const float gv = dyv * g[i].v[j];
					s1 += gv;
					s2 += gv * xhat;
				}
			}
		}
		const float m2 = row_sum<WPR>(s2, red) / d;
		const float m1 = LN ? row_sum<WPR>(s1, red) / d : 0.f;
		bf16_t* dxr = dx + (int64_t)row * d;
#pragma unroll
		for (int i = 0; i < NCH; i++) {
			const int ch = tr + i * TPR;
			if (ch < nchunks) {
				Chunk o;
#pragma unroll
				for (int j = 0; j < 8; j++) {
					const float xhat = ((float)rx[i][j] - mean) * rstd;
					const float gv = (float)rdy[i][j] * g[i].v[j];
					o.v[j] = rstd * (gv - m1 - xhat * m2);
					if (dres) o.v[j] += (float)rres[i][j];
				}
				store8(dxr + ch * 8, o);
				if constexpr (YOUT) {
					Chunk y, b;
					if (LN) b = load8(beta + ch * 8);
#pragma unroll
					for (int j = 0; j < 8; j++) y.v[j] = norm_out<LN>((float)rx[i][j], mean, rstd, g[i].v[j], LN ? b.v[j] : 0.f);
					store8(yout + (int64_t)row * d + ch * 8, y);
				}
			}
		}
	}
	float* pg = part + (int64_t)blockIdx.x * 2 * d;
	float* pb = pg + d;
	if constexpr (WPR > 1) {
		// every thread owns its columns outright
#pragma unroll
		for (int i = 0; i < NCH; i++) {
			const int ch = tr + i * TPR;
			if (ch < nchunks) {
#pragma unroll
				for (int j = 0; j < 8; j++) {
					pg[ch * 8 + j] = dg[i][j];
					if (LN) pb[ch * 8 + j] = db[i][j];
				}
			}
		}
	} else {
		// fold the 4 waves (4 different rows, same columns) through LDS, 512 columns at a time
#pragma unroll
		for (int i = 0; i < NCH; i++) {
			for (int which = 0; which < (LN ? 2 : 1); which++) {
				__syncthreads();
#pragma unroll
				for (int j = 0; j < 8; j++) fold[wave][lane * 8 + j] = which ? db[i][j] : dg[i][j];
				__syncthreads();
				for (int col = threadIdx.x; col < 512; col += 256) {
					const int ch = (col >> 3) + i * 64;
					if (ch < nchunks) {
						float s = 0.f;
#pragma unroll
						for (int w = 0; w < ROWS_PER_BLOCK; w++) s += fold[w][col];
						(which ? pb : pg)[ch * 8 + (col & 7)] = s;
					}
				}
			}
		}
	}
}

// main_grad[c] += sum_b part[b][which][c].  A workgroup owns 32 columns; its 32 row groups stride over the partial
// rows and are folded through LDS in a fixed order, and each column has one writer: the sums do not depend on
// the order in which workgroups run (bit-reproducible gamma / beta gradients).
__global__ __launch_bounds__(1024) void norm_bwd_finalize_kernel(const float* __restrict__ part, int nparts, int d,
                                                                 float* __restrict__ dgamma, float* __restrict__ dbeta) {
	__shared__ float red[2][32][33];
	const int cl = threadIdx.x & 31, rg = threadIdx.x >> 5;
	const int c = blockIdx.x * 32 + cl;
	float sg = 0.f, sb = 0.f;
	if (c < d) {
		// 16 loads in flight per lane: the kernel is a chain of dependent trips to memory otherwise
#pragma unroll 16
		for (int b = rg; b < nparts; b += 32) {
			sg += part[(int64_t)b * 2 * d + c];
			if (dbeta) sb += part[(int64_t)b * 2 * d + d + c];
		}
	}
	red[0][rg][cl] = sg;
	red[1][rg][cl] = sb;
	__syncthreads();
	if (rg == 0 && c < d) {
		float tg = 0.f, tb = 0.f;
#pragma unroll
		for (int r = 0; r < 32; r++) {
			tg += red[0][r][cl];
			tb += red[1][r][cl];
		}
		dgamma[c] += tg;
		if (dbeta) dbeta[c] += tb;
	}
}


// ------------------------------------------------------------------------------------------
// Narrow rows (d = 256, 512 or 768; the GPT-2-small width 768 is three 16-byte chunks per lane): half a
// wave per row, so that no lane idles in a partly filled chunk and a wave has two rows' loads in flight; reductions
// stay inside the half-wave (butterfly over 16 .. 1).  Forward: each wave takes PAIRS consecutive row pairs, all
// loads issued before the first reduction.
__device__ __forceinline__ float half_wave_sum(float v) {
#pragma unroll
	for (int o = 16; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
	return v;
}

template <int NCH, bool LN, int PAIRS>
__global__ __launch_bounds__(256) void norm_fwd_half_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ gamma,
                                                            const bf16_t* __restrict__ beta, bf16_t* __restrict__ y,
                                                            float2* __restrict__ stats, int T, float eps) {
	constexpr int d = NCH * 256;
	const int l32 = threadIdx.x & 31;
	const int row0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * (2 * PAIRS) + ((threadIdx.x >> 5) & 1);
	bf16x8 raw[PAIRS][NCH];
#pragma unroll
	for (int p = 0; p < PAIRS; p++) {
		const int row = row0 + 2 * p;
		if (row < T)
#pragma unroll
			for (int i = 0; i < NCH; i++) raw[p][i] = *reinterpret_cast<const bf16x8*>(x + (int64_t)row * d + (l32 + 32 * i) * 8);
	}
	Chunk g[NCH], b[NCH];
#pragma unroll
	for (int i = 0; i < NCH; i++) {
		g[i] = load8(gamma + (l32 + 32 * i) * 8);
		if (LN) b[i] = load8(beta + (l32 + 32 * i) * 8);
	}
#pragma unroll
	for (int p = 0; p < PAIRS; p++) {
		const int row = row0 + 2 * p;
		if (row >= T) continue;  // uniform per half-wave; the shuffles below stay inside it
		float c[NCH][8];
		float s = 0.f, ss = 0.f;
#pragma unroll
		for (int i = 0; i < NCH; i++)
#pragma unroll
			for (int j = 0; j < 8; j++) {
				c[i][j] = (float)raw[p][i][j];
				s += c[i][j];
				ss += c[i][j] * c[i][j];
			}
		float mean = 0.f, rstd;
		if (LN) {
			mean = half_wave_sum(s) / d;
			float var = 0.f;
#pragma unroll
			for (int i = 0; i < NCH; i++)
#pragma unroll
				for (int j = 0; j < 8; j++) {
					const float t = c[i][j] - mean;
					var += t * t;
				}
			rstd = rsqrtf(half_wave_sum(var) / d + eps);
		} else {
			rstd = rsqrtf(half_wave_sum(ss) / d + eps);
		}
		if (l32 == 0) stats[row] = make_float2(mean, rstd);
#pragma unroll
		for (int i = 0; i < NCH; i++) {
			Chunk o;
#pragma unroll
			for (int j = 0; j < 8; j++) o.v[j] = norm_out<LN>(c[i][j], mean, rstd, g[i].v[j], LN ? b[i].v[j] : 0.f);
			store8(y + (int64_t)row * d + (l32 + 32 * i) * 8, o);
		}
	}
}

// Backward for the same rows: a wave walks row pairs with the next pair's loads in flight while it reduces the current
// one; the eight rows a workgroup holds at a time are folded through LDS into one partial row per workgroup.
template <int NCH, bool LN>
__global__ __launch_bounds__(256) void norm_bwd_half_kernel(const bf16_t* __restrict__ dy, const bf16_t* __restrict__ x,
                                                            const bf16_t* __restrict__ gamma, const float2* __restrict__ stats,
                                                            const bf16_t* __restrict__ dres, bf16_t* __restrict__ dx,
                                                            float* __restrict__ part, int T) {
	constexpr int d = NCH * 256;
	__shared__ float fold[4][NCH * 256];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31;
	Chunk g[NCH];
	float dg[NCH][8], db[NCH][8];
#pragma unroll
	for (int i = 0; i < NCH; i++) {
		g[i] = load8(gamma + (l32 + 32 * i) * 8);
#pragma unroll
		for (int j = 0; j < 8; j++) dg[i][j] = db[i][j] = 0.f;
	}
	const int row_step = gridDim.x * 8;
	int row = blockIdx.x * 8 + wave * 2 + (lane >> 5);
	bf16x8 nx[NCH], ndy[NCH], nres[NCH];  // the row pair in flight
	float2 nst = make_float2(0.f, 0.f);
	auto fetch = [&](int r) {
		if (r < T) {
			nst = stats[r];
#pragma unroll
			for (int i = 0; i < NCH; i++) {
				nx[i] = *reinterpret_cast<const bf16x8*>(x + (int64_t)r * d + (l32 + 32 * i) * 8);
				ndy[i] = *reinterpret_cast<const bf16x8*>(dy + (int64_t)r * d + (l32 + 32 * i) * 8);
				if (dres) nres[i] = *reinterpret_cast<const bf16x8*>(dres + (int64_t)r * d + (l32 + 32 * i) * 8);
			}
		}
	};
	fetch(row);
	for (; row < T; row += row_step) {
		bf16x8 rx[NCH], rdy[NCH], rres[NCH];
		const float mean = nst.x, rstd = nst.y;
#pragma unroll
		for (int i = 0; i < NCH; i++) rx[i] = nx[i], rdy[i] = ndy[i], rres[i] = nres[i];
		fetch(row + row_step);  // the next pair's loads travel while this one is reduced and stored
		float s1 = 0.f, s2 = 0.f;
#pragma unroll
		for (int i = 0; i < NCH; i++)
#pragma unroll
			for (int j = 0; j < 8; j++) {
				const float xhat = ((float)rx[i][j] - mean) * rstd;
				const float dyv = (float)rdy[i][j];
				dg[i][j] += dyv * xhat;
				if (LN) db[i][j] += dyv;
				const float gv = dyv * g[i].v[j];
				s1 += gv;
				s2 += gv * xhat;
			}
		const float m2 = half_wave_sum(s2) / d;
		const float m1 = LN ? half_wave_sum(s1) / d : 0.f;
#pragma unroll
		for (int i = 0; i < NCH; i++) {
			Chunk o;
#pragma unroll
			for (int j = 0; j < 8; j++) {
				const float xhat = ((float)rx[i][j] - mean) * rstd;
				const float gv = (float)rdy[i][j] * g[i].v[j];
				o.v[j] = rstd * (gv - m1 - xhat * m2);
				if (dres) o.v[j] += (float)rres[i][j];
			}
			store8(dx + (int64_t)row * d + (l32 + 32 * i) * 8, o);
		}
	}
	// fold: the two rows of a wave by a shuffle, the four waves through LDS, in a fixed order
	float* pg = part + (int64_t)blockIdx.x * 2 * d;
	for (int which = 0; which < (LN ? 2 : 1); which++) {
		__syncthreads();
#pragma unroll
		for (int i = 0; i < NCH; i++)
#pragma unroll
			for (int j = 0; j < 8; j++) {
				float v = which ? db[i][j] : dg[i][j];
				v += __shfl_xor(v, 32, 64);
				if (lane < 32) fold[wave][(l32 + 32 * i) * 8 + j] = v;
			}
		__syncthreads();
		for (int col = threadIdx.x; col < d; col += 256) pg[which * d + col] = (fold[0][col] + fold[1][col]) + (fold[2][col] + fold[3][col]);
	}
}

// (at d = 1024 the backward's four chunks per lane of three tensors, current and next row, fill the register file and the
// full-wave kernel is faster)
static inline bool norm_half_rows(int d) { return d % 256 == 0 && d <= 768; }
// the full-wave backward kernel can write the norm's output again (see norm_bwd_kernel); the narrow-row one does not
bool norm_bwd_forms_output(int d) { return !norm_half_rows(d); }

static inline int norm_bwd_blocks(int T, int d) {
	if (norm_half_rows(d)) {
		// eight rows per workgroup at a time, one workgroup per compute unit: 256 partial rows for the fold kernel (with 512
		// the pair took 21 us at 8192 x 768, with 256 18 us, with 128 20 us)
		const int want = (T + 7) / 8;
		return want < 256 ? want : 256;
	}
	const int rows_per_block = d <= 2048 ? ROWS_PER_BLOCK : 1;
	const int want = (T + rows_per_block - 1) / rows_per_block;
	// fewer, longer workgroups for narrow rows and for the wide ones: the partial rows are overhead traffic that the fold
	// kernel reads back (d = 8192: 3.8 -> 4.1 TB/s with 512 instead of 1024; d = 4096 inside a stage's stream: 5.28 TB/s
	// with 512, 5.05 with 1024, 5.12 with 256, 4.7 with 384 or 2048 - two workgroups per compute unit, no ragged round)
	const int cap = (d <= 1024 || d >= 4096) ? 512 : 1024;
	return want < cap ? want : cap;
}

template <bool LN>
static int norm_fwd_dispatch(const void* x, const void* gamma, const void* beta, void* y, void* stats, int T, int d,
                             float eps, hipStream_t s) {
	const dim3 block(256);
	if (norm_half_rows(d)) {
		constexpr int PAIRS = 2;  // 16 rows per workgroup
		const dim3 grid((T + 16 - 1) / 16);
#define ELF_NORM_FWD_HALF(N) ELF_LAUNCH((norm_fwd_half_kernel<N, LN, PAIRS>), grid, block, 0, s, (const bf16_t*)x, (const bf16_t*)gamma, (const bf16_t*)beta, (bf16_t*)y, (float2*)stats, T, eps)
		switch (d / 256) {
			case 1: ELF_NORM_FWD_HALF(1); break;
			case 2: ELF_NORM_FWD_HALF(2); break;
			default: ELF_NORM_FWD_HALF(3); break;
		}
#undef ELF_NORM_FWD_HALF
		ELF_CHECK_HIP(hipGetLastError());
		return 0;
	}
#define ELF_NORM_FWD(N, W)                                                                                          \
	ELF_LAUNCH((norm_fwd_kernel<N, W, LN>), dim3(W == 1 ? (T + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK : T), block, 0, \
	                   s, (const bf16_t*)x, (const bf16_t*)gamma, (const bf16_t*)beta, (bf16_t*)y, (float2*)stats, T, d, eps)
	if (d <= 512) ELF_NORM_FWD(1, 1);
	else if (d <= 1024) ELF_NORM_FWD(2, 1);
	else if (d <= 2048) ELF_NORM_FWD(4, 1);
	else if (d <= 4096) ELF_NORM_FWD(2, 4);
	else ELF_NORM_FWD(4, 4);
#undef ELF_NORM_FWD
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

int norm_fwd(int kind, const void* x, const void* gamma, const void* beta, void* y, void* stats, int T, int d,
             float eps, hipStream_t s) {
	ELF_REQUIRE(T > 0 && d > 0 && d % 8 == 0 && d <= 8192, "norm_fwd: d must be a multiple of 8 and <= 8192 (d=%d)", d);
	ELF_REQUIRE(x && gamma && y && stats, "norm_fwd: null pointer");
	ProfScope prof(PROF_NORM_FWD, 4.0 * T * d, s);
	if (kind == NORM_LAYER) {
		ELF_REQUIRE(beta != nullptr, "norm_fwd: LayerNorm needs beta");
		return norm_fwd_dispatch<true>(x, gamma, beta, y, stats, T, d, eps, s);
	}
	return norm_fwd_dispatch<false>(x, gamma, beta, y, stats, T, d, eps, s);
}

int64_t norm_bwd_workspace_floats(int T, int d) { return (int64_t)norm_bwd_blocks(T, d) * 2 * d; }

template <bool LN>
static int norm_bwd_dispatch(const void* dy, const void* x, const void* gamma, const void* stats, const void* dres,
                             void* dx, float* part, int T, int d, hipStream_t s, const void* beta, void* yout) {
	const dim3 grid(norm_bwd_blocks(T, d)), block(256);
	if (norm_half_rows(d)) {
#define ELF_NORM_BWD_HALF(N) ELF_LAUNCH((norm_bwd_half_kernel<N, LN>), grid, block, 0, s, (const bf16_t*)dy, (const bf16_t*)x, (const bf16_t*)gamma, (const float2*)stats, (const bf16_t*)dres, (bf16_t*)dx, part, T)
		switch (d / 256) {
			case 1: ELF_NORM_BWD_HALF(1); break;
			case 2: ELF_NORM_BWD_HALF(2); break;
			default: ELF_NORM_BWD_HALF(3); break;
		}
#undef ELF_NORM_BWD_HALF
		ELF_CHECK_HIP(hipGetLastError());
		return 0;
	}
#define ELF_NORM_BWD_Y(N, W, Y)                                                                                  \
	ELF_LAUNCH((norm_bwd_kernel<N, W, LN, Y>), grid, block, 0, s, (const bf16_t*)dy, (const bf16_t*)x,     \
	                   (const bf16_t*)gamma, (const float2*)stats, (const bf16_t*)dres, (bf16_t*)dx, part, T, d, (const bf16_t*)beta, (bf16_t*)yout)
#define ELF_NORM_BWD(N, W)              \
	do {                                \
		if (yout) ELF_NORM_BWD_Y(N, W, true); \
		else ELF_NORM_BWD_Y(N, W, false);     \
	} while (0)
	if (d <= 512) ELF_NORM_BWD(1, 1);
	else if (d <= 1024) ELF_NORM_BWD(2, 1);
	else if (d <= 2048) ELF_NORM_BWD(4, 1);
	else if (d <= 4096) ELF_NORM_BWD(2, 4);
	else ELF_NORM_BWD(4, 4);
#undef ELF_NORM_BWD
#undef ELF_NORM_BWD_Y
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

static int norm_bwd_launch(int kind, const void* dy, const void* x, const void* gamma, const void* stats, const void* dres,
                           void* dx, float* dgamma, float* dbeta, float* workspace, int T, int d, hipStream_t s, const void* beta = nullptr,
                           void* yout = nullptr) {
	int rc;
	ELF_REQUIRE(!yout || (norm_bwd_forms_output(d) && (kind != NORM_LAYER || beta)), "norm_bwd: the output cannot be formed again at this width (d=%d)", d);
	if (kind == NORM_LAYER) {
		ELF_REQUIRE(dbeta != nullptr, "norm_bwd: LayerNorm needs dbeta");
		rc = norm_bwd_dispatch<true>(dy, x, gamma, stats, dres, dx, workspace, T, d, s, beta, yout);
	} else {
		rc = norm_bwd_dispatch<false>(dy, x, gamma, stats, dres, dx, workspace, T, d, s, beta, yout);
	}
	if (rc) return rc;
	const int nparts = norm_bwd_blocks(T, d);
	ELF_LAUNCH(norm_bwd_finalize_kernel, dim3((d + 31) / 32), dim3(1024), 0, s, workspace, nparts, d, dgamma,
	                   kind == NORM_LAYER ? dbeta : nullptr);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

int norm_bwd(int kind, const void* dy, const void* x, const void* gamma, const void* stats, const void* dres,
             void* dx, float* dgamma, float* dbeta, float* workspace, int T, int d, hipStream_t s, const void* beta, void* y_out) {
	ELF_REQUIRE(T > 0 && d > 0 && d % 8 == 0 && d <= 8192, "norm_bwd: d must be a multiple of 8 and <= 8192 (d=%d)", d);
	ELF_REQUIRE(dy && x && gamma && stats && dx && dgamma && workspace, "norm_bwd: null pointer");
	ProfScope prof(PROF_NORM_BWD, (dres ? 8.0 : 6.0) * T * d + (y_out ? 2.0 * T * d : 0.0), s);
	return norm_bwd_launch(kind, dy, x, gamma, stats, dres, dx, dgamma, dbeta, workspace, T, d, s, beta, y_out);
}

// Norm backward for callers that cannot allocate (code under HIP graph capture, tight serving loops): the
// per-workgroup partial sums of dgamma / dbeta go to an array that is part of the library's device image
// instead of a workspace argument.  Its size covers every shape norm_bwd accepts: at most 1024 partial rows
// of 2 x 8192 floats = 64 MiB, which every GPU the library runs on holds until the process ends.  The host
// sees `scratch` as a stand-in symbol only; its device address is looked up once per device.
constexpr int64_t NORM_BWD_SCRATCH_FLOATS = (int64_t)1024 * 2 * 8192;
static __device__ __align__(256) float scratch[NORM_BWD_SCRATCH_FLOATS];
constexpr int MAX_DEVICES = 64;
static std::atomic<float*> scratch_ptr[MAX_DEVICES] = {};  // written once per device under the mutex, read lock-free
static std::mutex scratch_mutex;

int norm_bwd_scratch_prepare() {
	int dev = -1;
	ELF_CHECK_HIP(hipGetDevice(&dev));
	ELF_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "norm_bwd_noalloc: device index %d out of range", dev);
	std::lock_guard<std::mutex> lock(scratch_mutex);
	if (!scratch_ptr[dev].load(std::memory_order_acquire)) {
		float* p = nullptr;
		ELF_CHECK_HIP(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
		ELF_REQUIRE(p != nullptr, "norm_bwd_noalloc: no device address for the scratch array");
		scratch_ptr[dev].store(p, std::memory_order_release);
	}
	return 0;
}

int norm_bwd_noalloc(int kind, const void* dy, const void* x, const void* gamma, const void* stats, const void* dres,
                     void* dx, float* dgamma, float* dbeta, int T, int d, hipStream_t s) {
	ELF_REQUIRE(T > 0 && d > 0 && d % 8 == 0 && d <= 8192, "norm_bwd_noalloc: d must be a multiple of 8 and <= 8192 (d=%d)", d);
	ELF_REQUIRE(dy && x && gamma && stats && dx && dgamma, "norm_bwd_noalloc: null pointer");
	ELF_REQUIRE(norm_bwd_workspace_floats(T, d) <= NORM_BWD_SCRATCH_FLOATS,
	            "norm_bwd_noalloc: T = %d, d = %d needs %lld floats of scratch, the built-in array holds %lld", T, d,
	            (long long)norm_bwd_workspace_floats(T, d), (long long)NORM_BWD_SCRATCH_FLOATS);
	int dev = -1;
	ELF_CHECK_HIP(hipGetDevice(&dev));
	ELF_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "norm_bwd_noalloc: device index %d out of range", dev);
	float* ptr = scratch_ptr[dev].load(std::memory_order_acquire);
	if (!ptr) {
		// first call on this device: the address lookup (no allocation; the array is part of the loaded code object)
		if (int rc = norm_bwd_scratch_prepare()) return rc;
		ptr = scratch_ptr[dev].load(std::memory_order_acquire);
	}
	// every workgroup writes its whole partial row before the fold reads it: nothing has to start at zero
	return norm_bwd_launch(kind, dy, x, gamma, stats, dres, dx, dgamma, dbeta, ptr, T, d, s);
}

// ------------------------------------------------------------------------------------------
// Activations.  GELU is the exact (erf) form of nn.GELU():  y = 0.5 x (1 + erf(x / sqrt 2)).
// SwiGLU: h = silu(g) * u with g = gu[:, :F], u = gu[:, F:].
__device__ __forceinline__ float gelu_grad_f(float x) {
	const float cdf = 0.5f * (1.f + erff(x * 0.70710678118654752f));
	const float pdf = 0.3989422804014327f * __expf(-0.5f * x * x);
	return cdf + x * pdf;
}

__global__ __launch_bounds__(256) void gelu_fwd_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ y, int64_t nchunks) {
	for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < nchunks; i += (int64_t)gridDim.x * blockDim.x) {
		Chunk c = load8(x + i * 8);
#pragma unroll
		for (int j = 0; j < 8; j++) c.v[j] = gelu_f(c.v[j]);
		store8(y + i * 8, c);
	}
}
__global__ __launch_bounds__(256) void gelu_bwd_kernel(const bf16_t* __restrict__ dy, const bf16_t* __restrict__ x,
                                                       bf16_t* __restrict__ dx, int64_t nchunks) {
	for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < nchunks; i += (int64_t)gridDim.x * blockDim.x) {
		Chunk c = load8(x + i * 8), g = load8(dy + i * 8);
#pragma unroll
		for (int j = 0; j < 8; j++) c.v[j] = g.v[j] * gelu_grad_f(c.v[j]);
		store8(dx + i * 8, c);
	}
}
// gu: [T, 2F]; h: [T, F]
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ h, int64_t T, int F) {
	const int cpr = F >> 3;
	const int64_t n = T * cpr;
	for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
		const int64_t row = i / cpr;
		const int c8 = (int)(i - row * cpr) * 8;
		Chunk g = load8(gu + row * 2 * F + c8), u = load8(gu + row * 2 * F + F + c8);
#pragma unroll
		for (int j = 0; j < 8; j++) g.v[j] = swiglu_f(g.v[j], u.v[j]);
		store8(h + row * F + c8, g);
	}
}
// dgu[:, :F] = dh * u * (sig + g sig (1 - sig));  dgu[:, F:] = dh * g * sig.  ACT: the activation silu(g) * u goes to
// `act` [T, F] as well (a stash that dropped it gets it back from the g and u read here anyway: the bits of swiglu_fwd).
template <bool ACT>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const bf16_t* __restrict__ dh, const bf16_t* __restrict__ gu,
                                                         bf16_t* __restrict__ dgu, bf16_t* __restrict__ act, int64_t T, int F) {
	const int cpr = F >> 3;
	const int64_t n = T * cpr;
	for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
		const int64_t row = i / cpr;
		const int c8 = (int)(i - row * cpr) * 8;
		Chunk g = load8(gu + row * 2 * F + c8), u = load8(gu + row * 2 * F + F + c8), d = load8(dh + row * F + c8);
		Chunk dg, du;
#pragma unroll
		for (int j = 0; j < 8; j++) swiglu_bwd_f(d.v[j], g.v[j], u.v[j], dg.v[j], du.v[j]);
		store8(dgu + row * 2 * F + c8, dg);
		store8(dgu + row * 2 * F + F + c8, du);
		if constexpr (ACT) {
#pragma unroll
			for (int j = 0; j < 8; j++) g.v[j] = swiglu_f(g.v[j], u.v[j]);
			store8(act + row * F + c8, g);
		}
	}
}

static inline int ew_grid(int64_t nchunks) {
	int64_t b = (nchunks + 255) / 256;
	return (int)(b < 256 * 16 ? (b < 1 ? 1 : b) : 256 * 16);
}

int gelu_fwd(const void* x, void* y, int64_t n, hipStream_t s) {
	ELF_REQUIRE(n > 0 && n % 8 == 0 && x && y, "gelu_fwd: n must be a positive multiple of 8");
	ProfScope prof(PROF_ACT_FWD, 4.0 * n, s);
	ELF_LAUNCH(gelu_fwd_kernel, dim3(ew_grid(n / 8)), dim3(256), 0, s, (const bf16_t*)x, (bf16_t*)y, n / 8);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}
int gelu_bwd(const void* dy, const void* x, void* dx, int64_t n, hipStream_t s) {
	ELF_REQUIRE(n > 0 && n % 8 == 0 && x && dy && dx, "gelu_bwd: n must be a positive multiple of 8");
	ProfScope prof(PROF_ACT_BWD, 6.0 * n, s);
	ELF_LAUNCH(gelu_bwd_kernel, dim3(ew_grid(n / 8)), dim3(256), 0, s, (const bf16_t*)dy, (const bf16_t*)x,
	                   (bf16_t*)dx, n / 8);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}
int swiglu_fwd(const void* gu, void* h, int64_t T, int F, hipStream_t s) {
	ELF_REQUIRE(T > 0 && F > 0 && F % 8 == 0 && gu && h, "swiglu_fwd: F must be a positive multiple of 8");
	ProfScope prof(PROF_ACT_FWD, 6.0 * T * F, s);
	ELF_LAUNCH(swiglu_fwd_kernel, dim3(ew_grid(T * (F / 8))), dim3(256), 0, s, (const bf16_t*)gu, (bf16_t*)h, T, F);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}
int swiglu_bwd(const void* dh, const void* gu, void* dgu, int64_t T, int F, hipStream_t s, void* act) {
	ELF_REQUIRE(T > 0 && F > 0 && F % 8 == 0 && gu && dh && dgu, "swiglu_bwd: F must be a positive multiple of 8");
	ProfScope prof(PROF_ACT_BWD, (act ? 12.0 : 10.0) * T * F, s);
	if (act) ELF_LAUNCH(swiglu_bwd_kernel<true>, dim3(ew_grid(T * (F / 8))), dim3(256), 0, s, (const bf16_t*)dh, (const bf16_t*)gu, (bf16_t*)dgu, (bf16_t*)act, T, F);
	else ELF_LAUNCH(swiglu_bwd_kernel<false>, dim3(ew_grid(T * (F / 8))), dim3(256), 0, s, (const bf16_t*)dh, (const bf16_t*)gu, (bf16_t*)dgu, (bf16_t*)nullptr, T, F);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

// ------------------------------------------------------------------------------------------
// Rotary embedding, half-split ("rotate_half") convention, applied in place to the first
// n_rot_heads heads of a packed [T, ld] projection buffer (q heads then k heads):
//   out[i]       = x[i] cos(a_i) - x[i+D/2] sin(a_i)
//   out[i + D/2] = x[i+D/2] cos(a_i) + x[i] sin(a_i),   a_i = pos * theta^(-2i/D), pos = t mod S.
// The backward is the same rotation with the sign of sin flipped.  cs is the fp32 table
// [S, D/2] of (cos, sin) pairs produced by rope_table().
__global__ void rope_table_kernel(float2* __restrict__ cs, int S, int half, double theta) {
	const int i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= S * half) return;
	const int pos = i / half, f = i % half;
	const double inv = pow(theta, -(double)f / (double)half);
	const double a = (double)pos * inv;
	cs[i] = make_float2((float)cos(a), (float)sin(a));
}
int rope_table(void* cs, int S, int D, double theta, hipStream_t s) {
	ELF_REQUIRE(cs && S > 0 && D > 0 && D % 16 == 0, "rope_table: head_dim must be a multiple of 16");
	const int n = S * (D / 2);
	ELF_LAUNCH(rope_table_kernel, dim3((n + 255) / 256), dim3(256), 0, s, (float2*)cs, S, D / 2, theta);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

__global__ __launch_bounds__(256) void rope_kernel(bf16_t* __restrict__ buf, const float2* __restrict__ cs, int64_t T, int S,
                                                   int ld, int n_heads, int D, float sign) {
	const int cph = D >> 4;  // 8-wide chunks per half head
	const int64_t n = T * n_heads * cph;
	for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
		const int c = (int)(i % cph);
		const int64_t th = i / cph;
		const int h = (int)(th % n_heads);
		const int64_t t = th / n_heads;
		const int pos = (int)(t % S);
		bf16_t* p = buf + t * ld + h * D + c * 8;
		Chunk a = load8(p), b = load8(p + D / 2);
		const float2* tab = cs + (int64_t)pos * (D / 2) + c * 8;
		Chunk oa, ob;
#pragma unroll
		for (int j = 0; j < 8; j++) {
			const float2 t2 = tab[j];
			rope_rot(a.v[j], b.v[j], t2.x, t2.y * sign, oa.v[j], ob.v[j]);
		}
		store8(p, oa);
		store8(p + D / 2, ob);
	}
}
int rope_apply(void* buf, const void* cs, int64_t T, int S, int ld, int n_heads, int D, int backward, hipStream_t s) {
	ELF_REQUIRE(buf && cs && T > 0 && S > 0 && T % S == 0, "rope: T must be a multiple of S");
	ELF_REQUIRE(D % 16 == 0 && ld % 8 == 0 && n_heads * D <= ld, "rope: bad head layout");
	const int64_t n = T * n_heads * (D / 16);
	ProfScope prof(PROF_ROPE, 4.0 * T * n_heads * D, s);
	ELF_LAUNCH(rope_kernel, dim3(ew_grid(n)), dim3(256), 0, s, (bf16_t*)buf, (const float2*)cs, T, S, ld, n_heads,
	                   D, backward ? -1.f : 1.f);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

// ------------------------------------------------------------------------------------------
// Gradient scale: the fp32 accumulator is multiplied by `scale` in place and its bf16
// rounding is written next to it (the parameter-dtype .grad the reference exposes).
__global__ __launch_bounds__(256) void scale_grads_kernel(float* __restrict__ acc, bf16_t* __restrict__ out, int64_t n4,
                                                          int64_t n, float scale) {
	for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
		f32x4 v = reinterpret_cast<f32x4*>(acc)[i];
		v *= scale;
		reinterpret_cast<f32x4*>(acc)[i] = v;
		if (out) {
			bf16x4 o;
#pragma unroll
			for (int j = 0; j < 4; j++) o[j] = (bf16_t)v[j];
			reinterpret_cast<bf16x4*>(out)[i] = o;
		}
	}
	// tail (n not a multiple of 4)
	if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
		const int64_t i = n4 * 4 + threadIdx.x;
		const float v = acc[i] * scale;
		acc[i] = v;
		if (out) out[i] = (bf16_t)v;
	}
}
int scale_grads(void* acc_f32, void* out_bf16, int64_t n, float scale, hipStream_t s) {
	ELF_REQUIRE(acc_f32 && n > 0, "scale_grads: empty");
	ELF_REQUIRE(((uintptr_t)acc_f32 % 16) == 0 && (!out_bf16 || ((uintptr_t)out_bf16 % 8) == 0), "scale_grads: misaligned");
	// buffers under a MiB (norm gains and biases) are launch-bound, not bandwidth-bound: they stay out of the bandwidth figure
	ProfScope prof(PROF_SCALE, (out_bf16 ? 10.0 : 8.0) * n, s, /*record=*/n >= (1 << 18));
	ELF_LAUNCH(scale_grads_kernel, dim3(ew_grid(n / 4 + 1)), dim3(256), 0, s, (float*)acc_f32, (bf16_t*)out_bf16,
	                   n / 4, n, scale);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

// out = a + b (residual add / gradient fan-in, elf/execution/block.py:651-655)
__global__ __launch_bounds__(256) void add_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ b,
                                                  bf16_t* __restrict__ o, int64_t nchunks) {
	for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < nchunks; i += (int64_t)gridDim.x * blockDim.x) {
		Chunk x = load8(a + i * 8), y = load8(b + i * 8);
#pragma unroll
		for (int j = 0; j < 8; j++) x.v[j] += y.v[j];
		store8(o + i * 8, x);
	}
}
int add_bf16(const void* a, const void* b, void* out, int64_t n, hipStream_t s) {
	ELF_REQUIRE(n > 0 && n % 8 == 0 && a && b && out, "add: n must be a positive multiple of 8");
	ProfScope prof(PROF_ADD, 6.0 * n, s);
	ELF_LAUNCH(add_kernel, dim3(ew_grid(n / 8)), dim3(256), 0, s, (const bf16_t*)a, (const bf16_t*)b, (bf16_t*)out, n / 8);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

// ------------------------------------------------------------------------------------------
// Bias gradient of a split linear layer (elf/zb_utils.py:247-252: go.sum(0) added to bias.grad in
// LinearDW.backward): out[c] += sum_t x[t, c] in fp32.  A workgroup owns 256 columns and one of gridDim.y
// slices of the rows; its 8 row groups are folded through LDS and the slice's sums go to part[slice][c].  A second
// kernel adds the slices in ascending order, one writer per column: equal bits from run to run.
__global__ __launch_bounds__(256) void colsum_kernel(const bf16_t* __restrict__ x, int64_t ld, float* __restrict__ part, int64_t T, int N) {
	__shared__ float red[8][256];
	const int cl = threadIdx.x & 31, rg = threadIdx.x >> 5;
	const int c0 = (blockIdx.x * 32 + cl) * 8;
	float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
	if (c0 < N) {
		for (int64_t t = (int64_t)blockIdx.y * 8 + rg; t < T; t += 8 * (int64_t)gridDim.y) {
			const Chunk c = load8(x + t * ld + c0);
#pragma unroll
			for (int j = 0; j < 8; j++) s[j] += c.v[j];
		}
	}
#pragma unroll
	for (int j = 0; j < 8; j++) red[rg][cl * 8 + j] = s[j];
	__syncthreads();
	const int c = blockIdx.x * 256 + threadIdx.x;
	if (c < N) {
		float t = 0.f;
#pragma unroll
		for (int r = 0; r < 8; r++) t += red[r][threadIdx.x];
		part[(int64_t)blockIdx.y * N + c] = t;
	}
}
__global__ __launch_bounds__(256) void colsum_fold_kernel(const float* __restrict__ part, int slices, int N, float* __restrict__ out) {
	const int c = blockIdx.x * 256 + threadIdx.x;
	if (c >= N) return;
	float t = 0.f;
#pragma unroll 8
	for (int sl = 0; sl < slices; sl++) t += part[(int64_t)sl * N + c];
	out[c] += t;
}
static inline int colsum_slices(int64_t T, int N) {
	const int col_blocks = (N + 255) / 256;
	int64_t slices = (1024 + col_blocks - 1) / col_blocks;  // about four workgroups per CU
	if (slices > 64) slices = 64;
	if (slices > (T + 7) / 8) slices = (T + 7) / 8;
	return (int)(slices < 1 ? 1 : slices);
}
int64_t colsum_workspace_floats(int64_t T, int N) { return T > 0 && N > 0 ? (int64_t)colsum_slices(T, N) * N : 0; }
int colsum_bf16(const void* x, int64_t ld, void* out_f32, int64_t T, int N, float* workspace, hipStream_t s) {
	ELF_REQUIRE(x && out_f32 && workspace && T > 0 && N > 0 && N % 8 == 0 && ld % 8 == 0 && ld >= N,
	            "colsum: null pointer, or N and the row stride are not multiples of 8 (T=%lld N=%d ld=%lld)", (long long)T, N, (long long)ld);
	const int col_blocks = (N + 255) / 256, slices = colsum_slices(T, N);
	ELF_LAUNCH(colsum_kernel, dim3(col_blocks, (unsigned)slices), dim3(256), 0, s, (const bf16_t*)x, ld, workspace, T, N);
	ELF_LAUNCH(colsum_fold_kernel, dim3(col_blocks), dim3(256), 0, s, (const float*)workspace, slices, N, (float*)out_f32);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

// ------------------------------------------------------------------------------------------
// Token embedding of a pipeline's first stage (benchmarks/models/simple.py:496, 502):
// out[t, :] = table[ids[t], :].  One 16-byte chunk per lane; rows of ids outside [0, V) give a
// zero row (the host cannot check ids without a device round trip).
__global__ __launch_bounds__(256) void embedding_fwd_kernel(const int64_t* __restrict__ ids, const bf16_t* __restrict__ table,
                                                            bf16_t* __restrict__ out, int64_t T, int d, int V) {
	const int cpr = d / 8;
	const int64_t n = T * cpr;
	for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
		const int64_t t = i / cpr;
		const int c = (int)(i - t * cpr) * 8;
		const int64_t id = ids[t];
		Chunk x;
		if (id >= 0 && id < V) {
			x = load8(table + id * d + c);
		} else {
#pragma unroll
			for (int j = 0; j < 8; j++) x.v[j] = 0.f;
		}
		store8(out + t * d + c, x);
	}
}
// dtable[ids[t], :] += dx[t, :] in fp32.  One workgroup of four waves per (token position, 512-column slice).  The
// workgroups of a token's first occurrence sum the rows of all its occurrences, each over its own column slice, and are
// the only writers of that table row: no atomics.  The positions behind the first occurrence are dealt to the four
// waves in runs of 64 (run k to wave k % 4); a wave adds its occurrences in ascending position, 16 row loads in flight
// at a time, and the four partial sums are folded in wave order: a fixed order of additions whatever the order in
// which waves run (bit-reproducible), and a token that fills the whole batch (padding) is summed by d / 128 waves
// instead of one.  The other workgroups find an earlier occurrence and leave (the ids are a few KiB and stay in cache).
__global__ __launch_bounds__(256) void embedding_bwd_kernel(const int64_t* __restrict__ ids, const bf16_t* __restrict__ dx,
                                                            float* __restrict__ dtable, int T, int d, int V) {
	__shared__ float part[4][512];
	const int t = blockIdx.x;
	const int64_t id = ids[t];
	if (id < 0 || id >= V) return;
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	{
		// an earlier occurrence?  The first 256 positions with one barrier (a frequent token is found there), then each wave
		// takes every fourth run of 128 positions without a barrier in between
		if (__syncthreads_or((int)threadIdx.x < t && ids[threadIdx.x] == id)) return;
		bool seen = false;
		for (int base = 256 + wave * 128; base < t && !seen; base += 512) {
			const int u = base + 2 * lane;
			const int64_t a = u < t ? ids[u] : -1, b = u + 1 < t ? ids[u + 1] : -1;
			seen = __ballot(a == id || b == id) != 0;
		}
		if (__syncthreads_or(seen)) return;
	}
	const int ch = blockIdx.y * 64 + lane;  // this lane's 8-column chunk
	const bool mine = ch < d / 8;
	float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
	for (int base = t + wave * 64; base < T; base += 256) {
		const int u = base + lane;
		unsigned long long bits = __ballot(u < T && ids[u] == id);
		while (bits) {
			constexpr int AHEAD = 16;
			Chunk x[AHEAD];
			int n = 0;
#pragma unroll
			for (int k = 0; k < AHEAD; k++) {
				if (bits) {
					const int64_t row = base + (__ffsll(bits) - 1);
					bits &= bits - 1;
					if (mine) x[k] = load8(dx + row * d + ch * 8);
					n = k + 1;
				}
			}
#pragma unroll
			for (int k = 0; k < AHEAD; k++)
				if (k < n && mine) {
#pragma unroll
					for (int j = 0; j < 8; j++) acc[j] += x[k].v[j];
				}
		}
	}
#pragma unroll
	for (int j = 0; j < 8; j++) part[wave][lane * 8 + j] = acc[j];
	__syncthreads();
	if (wave == 0 && mine) {
		float* g = dtable + id * d + ch * 8;
#pragma unroll
		for (int j = 0; j < 8; j++) {
			const float sum = ((part[0][lane * 8 + j] + part[1][lane * 8 + j]) + part[2][lane * 8 + j]) + part[3][lane * 8 + j];
			g[j] += sum;
		}
	}
}
int embedding_fwd(const void* ids, const void* table, void* out, int64_t T, int d, int V, hipStream_t s) {
	ELF_REQUIRE(ids && table && out && T > 0 && V > 0 && d > 0 && d % 8 == 0, "embedding_fwd: bad argument (d must be a multiple of 8)");
	ProfScope prof(PROF_EMBED, 4.0 * T * d, s);
	ELF_LAUNCH(embedding_fwd_kernel, dim3(ew_grid(T * (d / 8))), dim3(256), 0, s, (const int64_t*)ids, (const bf16_t*)table,
	                   (bf16_t*)out, T, d, V);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}
int embedding_bwd(const void* ids, const void* dx, void* dtable_f32, int64_t T, int d, int V, hipStream_t s) {
	ELF_REQUIRE(ids && dx && dtable_f32 && T > 0 && V > 0 && d > 0 && d % 8 == 0 && d <= 8192 && T < (int64_t(1) << 31),
	            "embedding_bwd: bad argument (d must be a multiple of 8 and at most 8192)");
	ProfScope prof(PROF_EMBED, 10.0 * T * d, s);
	ELF_LAUNCH(embedding_bwd_kernel, dim3((unsigned)T, (unsigned)((d / 8 + 63) / 64)), dim3(256), 0, s, (const int64_t*)ids, (const bf16_t*)dx, (float*)dtable_f32, (int)T, d, V);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

}  // namespace elf
