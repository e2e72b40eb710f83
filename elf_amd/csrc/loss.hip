// Cross-entropy of a pipeline's last stage over bf16 logits [rows, V] (row stride ld), computed in
// fp32 as the reference's loss function does after its upcast (benchmarks/models/simple.py:520-524,
// called from Engine.compute_loss, elf/execution/engine.py:374-410):
//     loss[r]      = logsumexp(x[r, :]) - x[r, target[r]]            (0 for target == ignore_index)
//     dlogits[r,c] = (softmax(x[r, :])[c] - (c == target[r])) * scale (0 for ignored rows and for
//                    the padding columns V <= c < ld_out)
// Forward and backward are one kernel — 4 bytes per logit of HBM traffic instead of the 10+ of a
// log-softmax / gather / scatter chain.  Short rows (up to 16384 columns) are read once into
// registers, reduced, and their gradient written from the same registers; longer rows are read
// twice by their workgroup, the second time out of cache.
#include "common.h"
#include "kernels.h"

namespace elf {

namespace {

constexpr float LOG2E_F = 1.4426950408889634f;

// 2^x as the bare hardware instruction: no denormal-range fix-up (results below 2^-126 flush to zero,
// which a softmax term that small may do).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

struct LossArgs {
	const bf16_t* x;
	int64_t ld;
	const int64_t* target;
	int64_t rows;
	int V;
	int64_t ignore_index;
	float scale;
	const float* dev_div;  // optional device scalar the gradient is divided by
	float* row_loss;       // optional
	bf16_t* dx;            // optional
	int64_t ld_out;
};

// Reductions over the G threads that share a row (G = 64: one wave; otherwise G / 64 waves of one
// workgroup, through LDS).
template <int G, bool MAX>
__device__ __forceinline__ float group_reduce(float v, float* red) {
	v = MAX ? wave_max(v) : wave_sum(v);
	if constexpr (G > 64) {
		constexpr int NW = G / 64;
		const int wave = threadIdx.x >> 6;
		__syncthreads();
		if ((threadIdx.x & 63) == 0) red[wave] = v;
		__syncthreads();
		v = red[0];
#pragma unroll
		for (int i = 1; i < NW; i++) v = MAX ? fmaxf(v, red[i]) : v + red[i];
	}
	return v;
}

__device__ __forceinline__ float grad_scale(const LossArgs& a) { return a.dev_div ? a.scale / *a.dev_div : a.scale; }

// Loss of one row from its statistics; NaN for a target outside [0, V) that is not ignore_index.
__device__ __forceinline__ float row_loss_of(const LossArgs& a, int64_t row, int64_t tgt, float m, float s) {
	if (tgt == a.ignore_index) return 0.f;
	if (tgt < 0 || tgt >= a.V) return __builtin_nanf("");
	return m + logf(s) - (float)a.x[row * a.ld + tgt];
}

// G threads per row, C 16-byte chunks (8 logits) per thread: rows of up to G * C * 8 columns.
template <int G, int C>
__global__ __launch_bounds__(G < 256 ? 256 : G) void cross_entropy_kernel(LossArgs a) {
	constexpr int BLOCK = G < 256 ? 256 : G;
	constexpr int ROWS = BLOCK / G;
	__shared__ float red[BLOCK / 64];
	const int lane = threadIdx.x % G;
	const int64_t row = (int64_t)blockIdx.x * ROWS + threadIdx.x / G;
	if (ROWS > 1 && row >= a.rows) return;  // whole waves leave together (G = 64 when ROWS > 1)
	const bf16_t* xr = a.x + row * a.ld;
	const int vchunks = (a.V + 7) / 8;

	bf16x8 reg[C];
	float m = -INFINITY;
#pragma unroll
	for (int j = 0; j < C; j++) {
		const int c = j * G + lane;
		if (c < vchunks) {
			reg[j] = *reinterpret_cast<const bf16x8*>(xr + (int64_t)c * 8);
#pragma unroll
			for (int i = 0; i < 8; i++)
				if (c * 8 + i < a.V) m = fmaxf(m, (float)reg[j][i]);
		}
	}
	m = group_reduce<G, true>(m, red);
	const float m2 = m * LOG2E_F;
	float s = 0.f;
#pragma unroll
	for (int j = 0; j < C; j++) {
		const int c = j * G + lane;
		if (c < vchunks) {
#pragma unroll
			for (int i = 0; i < 8; i++)
				if (c * 8 + i < a.V) s += fast_exp2((float)reg[j][i] * LOG2E_F - m2);
		}
	}
	s = group_reduce<G, false>(s, red);

	const int64_t tgt = a.target[row];
	if (a.row_loss && lane == 0) a.row_loss[row] = row_loss_of(a, row, tgt, m, s);
	if (!a.dx) return;
	const bool live = tgt != a.ignore_index;
	const float g = live ? grad_scale(a) : 0.f;
	const float gs = g / s;
	bf16_t* dr = a.dx + row * a.ld_out;
	const int ochunks = (int)(a.ld_out / 8);
#pragma unroll
	for (int j = 0; j < C; j++) {
		const int c = j * G + lane;
		if (c >= ochunks) continue;
		bf16x8 o;
#pragma unroll
		for (int i = 0; i < 8; i++) {
			const int col = c * 8 + i;
			float v = 0.f;
			if (c < vchunks && col < a.V) {
				v = fast_exp2((float)reg[j][i] * LOG2E_F - m2) * gs;
				if (col == tgt) v -= g;
			}
			o[i] = (bf16_t)v;
		}
		*reinterpret_cast<bf16x8*>(dr + (int64_t)c * 8) = o;
	}
}

// Longer rows: G threads per row (one workgroup), an online max / sum over one read of the row, then
// a second read (served by the cache hierarchy: the rows in flight on the chip are a few MiB) for the
// gradient.  The arithmetic is trimmed to what the two exponentials per logit leave room for: the
// running maximum only rescales the partial sum when it grows, column masks are confined to the last
// chunk of a row, the 1/sum * scale factor rides in the exponent, and the target column is fixed up
// by the one thread that holds it.
template <bool MASKED>
__device__ __forceinline__ void online_chunk(const bf16x8& r, int c, int V, float& m, float& s) {
	float x[8];
#pragma unroll
	for (int i = 0; i < 8; i++) x[i] = (MASKED && c * 8 + i >= V) ? -INFINITY : (float)r[i];
	const float cm = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7]))) * LOG2E_F;
	if (cm > m) {  // rare after the first chunks; s is 0 while m is -inf
		s *= fast_exp2(m - cm);
		m = cm;
	}
#pragma unroll
	for (int i = 0; i < 8; i++) s += fast_exp2(fmaf(x[i], LOG2E_F, -m));  // exp2(-inf) = 0 for masked columns
}

template <int G>
__global__ __launch_bounds__(G) void cross_entropy_stream_kernel(LossArgs a) {
	__shared__ float red[G / 64];
	const int lane = threadIdx.x;
	const int64_t row = blockIdx.x;
	const bf16_t* xr = a.x + row * a.ld;
	const int vchunks = (a.V + 7) / 8;
	const int full = a.V / 8;  // chunks with all 8 columns inside the row
	float m = -INFINITY, s = 0.f;  // m is in units of log2: max(x) * log2(e)
	int c = lane;
	for (; c + G < full; c += 2 * G) {  // two loads in flight per thread
		const bf16x8 r0 = *reinterpret_cast<const bf16x8*>(xr + (int64_t)c * 8);
		const bf16x8 r1 = *reinterpret_cast<const bf16x8*>(xr + (int64_t)(c + G) * 8);
		online_chunk<false>(r0, c, a.V, m, s);
		online_chunk<false>(r1, c + G, a.V, m, s);
	}
	for (; c < vchunks; c += G) {
		const bf16x8 r = *reinterpret_cast<const bf16x8*>(xr + (int64_t)c * 8);
		if (c < full) online_chunk<false>(r, c, a.V, m, s);
		else online_chunk<true>(r, c, a.V, m, s);
	}
	const float gm = group_reduce<G, true>(m, red);
	s = (m == -INFINITY) ? 0.f : s * fast_exp2(m - gm);
	s = group_reduce<G, false>(s, red);
	const float mx = gm * (1.f / LOG2E_F);  // back to natural units for the loss

	const int64_t tgt = a.target[row];
	if (a.row_loss && lane == 0) a.row_loss[row] = row_loss_of(a, row, tgt, mx, s);
	if (!a.dx) return;
	const float g = tgt != a.ignore_index ? grad_scale(a) : 0.f;
	bf16_t* dr = a.dx + row * a.ld_out;
	const int ochunks = (int)(a.ld_out / 8);
	if (g == 0.f) {  // ignored row (or a zero scale): the whole row of the gradient is zero
		bf16x8 z;
#pragma unroll
		for (int i = 0; i < 8; i++) z[i] = (bf16_t)0.f;
		for (int c2 = lane; c2 < ochunks; c2 += G) *reinterpret_cast<bf16x8*>(dr + (int64_t)c2 * 8) = z;
		return;
	}
	// softmax * |g| = exp2(x*log2e - (m + log2(s) - log2|g|)); the sign of g is applied after
	const float shift = gm + log2f(s) - log2f(fabsf(g));
	const float sign = g < 0.f ? -1.f : 1.f;
	const int tchunk = (tgt >= 0 && tgt < a.V) ? (int)(tgt >> 3) : -1;
	for (int c2 = lane; c2 < ochunks; c2 += G) {
		float v[8];
		if (c2 < full) {
			const bf16x8 r = *reinterpret_cast<const bf16x8*>(xr + (int64_t)c2 * 8);
#pragma unroll
			for (int i = 0; i < 8; i++) v[i] = fast_exp2((float)r[i] * LOG2E_F - shift) * sign;
		} else if (c2 < vchunks) {
			const bf16x8 r = *reinterpret_cast<const bf16x8*>(xr + (int64_t)c2 * 8);
#pragma unroll
			for (int i = 0; i < 8; i++) v[i] = c2 * 8 + i < a.V ? fast_exp2((float)r[i] * LOG2E_F - shift) * sign : 0.f;
		} else {
#pragma unroll
			for (int i = 0; i < 8; i++) v[i] = 0.f;
		}
		if (c2 == tchunk) {
#pragma unroll
			for (int i = 0; i < 8; i++)
				if (i == (int)(tgt & 7)) v[i] -= g;
		}
		bf16x8 o;
#pragma unroll
		for (int i = 0; i < 8; i++) o[i] = (bf16_t)v[i];
		*reinterpret_cast<bf16x8*>(dr + (int64_t)c2 * 8) = o;
	}
}

// out[0] = sum of row_loss (skipped when row_loss is null), out[1] = number of rows whose target is
// not ignore_index.  One workgroup, fixed summation order: the same inputs give the same bits.
__global__ __launch_bounds__(1024) void cross_entropy_reduce_kernel(const float* __restrict__ row_loss, const int64_t* __restrict__ target,
                                                                    int64_t rows, int64_t ignore_index, float* __restrict__ out) {
	__shared__ float red[16];
	float s = 0.f, n = 0.f;
	for (int64_t r = threadIdx.x; r < rows; r += 1024) {
		if (row_loss) s += row_loss[r];
		n += target[r] != ignore_index ? 1.f : 0.f;
	}
	s = group_reduce<1024, false>(s, red);
	n = group_reduce<1024, false>(n, red);
	if (threadIdx.x == 0) {
		if (row_loss) out[0] = s;
		out[1] = n;
	}
}

template <int G, int C>
void launch_rows(const LossArgs& a, hipStream_t s) {
	constexpr int BLOCK = G < 256 ? 256 : G;
	constexpr int ROWS = BLOCK / G;
	ELF_LAUNCH((cross_entropy_kernel<G, C>), dim3((unsigned)((a.rows + ROWS - 1) / ROWS)), dim3(BLOCK), 0, s, a);
}

}  // namespace

int cross_entropy(const void* logits, int64_t ld, const void* target, int64_t rows, int64_t V, int64_t ignore_index, float scale,
                  const void* dev_div, void* row_loss, void* dlogits, int64_t ld_out, hipStream_t s) {
	ELF_REQUIRE(logits && target && rows > 0 && V > 0 && V < (1ll << 30), "cross_entropy: bad argument");
	ELF_REQUIRE(rows < (1ll << 31), "cross_entropy: too many rows");
	ELF_REQUIRE(ld % 8 == 0 && ld >= V && ((uintptr_t)logits & 15) == 0,
	            "cross_entropy: logits rows must start on 16-byte boundaries (row stride %lld must be a multiple of 8 and >= V)", (long long)ld);
	ELF_REQUIRE(row_loss || dlogits, "cross_entropy: nothing to compute (no row_loss and no dlogits)");
	if (dlogits)
		ELF_REQUIRE(ld_out % 8 == 0 && ld_out >= V && ((uintptr_t)dlogits & 15) == 0,
		            "cross_entropy: gradient rows must start on 16-byte boundaries (row stride %lld must be a multiple of 8 and >= V)", (long long)ld_out);
	LossArgs a{(const bf16_t*)logits, ld, (const int64_t*)target, rows, (int)V, ignore_index, scale, (const float*)dev_div,
	           (float*)row_loss, (bf16_t*)dlogits, dlogits ? ld_out : 0};
	const int64_t width = dlogits && ld_out > V ? ld_out : V;
	ProfScope prof(PROF_LOSS, (dlogits ? 4.0 : 2.0) * rows * V, s);
	if (width <= 64 * 2 * 8) launch_rows<64, 2>(a, s);
	else if (width <= 64 * 8 * 8) launch_rows<64, 8>(a, s);
	else if (width <= 256 * 8 * 8) launch_rows<256, 8>(a, s);
	else if (width <= 65536) ELF_LAUNCH(cross_entropy_stream_kernel<256>, dim3((unsigned)rows), dim3(256), 0, s, a);
	else ELF_LAUNCH(cross_entropy_stream_kernel<1024>, dim3((unsigned)rows), dim3(1024), 0, s, a);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

int cross_entropy_reduce(const void* row_loss, const void* target, int64_t rows, int64_t ignore_index, void* out2, hipStream_t s) {
	ELF_REQUIRE(target && out2 && rows > 0, "cross_entropy_reduce: bad argument");
	ELF_LAUNCH(cross_entropy_reduce_kernel, dim3(1), dim3(1024), 0, s, (const float*)row_loss, (const int64_t*)target, rows,
	                   ignore_index, (float*)out2);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

}  // namespace elf
