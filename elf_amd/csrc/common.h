// Shared device/host helpers for the gfx950 stage kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

namespace elf {

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define ELF_LDS __attribute__((address_space(3)))

// Error plumbing: every C-ABI entry point returns 0 on success and a negative
// code on failure; the message is kept per host thread.
void set_error(const char* fmt, ...);
const char* get_error();

#define ELF_CHECK_HIP(expr)                                                             \
	do {                                                                                \
		hipError_t _e = (expr);                                                         \
		if (_e != hipSuccess) {                                                         \
			elf::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),      \
			               __FILE__, __LINE__);                                         \
			return -2;                                                                  \
		}                                                                               \
	} while (0)

#define ELF_REQUIRE(cond, ...)                \
	do {                                      \
		if (!(cond)) {                        \
			elf::set_error(__VA_ARGS__);      \
			return -1;                        \
		}                                     \
	} while (0)

__device__ __forceinline__ float bf2f(bf16_t v) { return (float)v; }
__device__ __forceinline__ bf16_t f2bf(float v) { return (bf16_t)v; }

// 64-lane butterfly reductions (wavefront = 64 on CDNA).
// MLP activations.  swiglu_f is shared by the activation kernel and the GEMM epilogue that fuses it, so
// that both give the same bits.  GELU is the exact (erf) form of nn.GELU(): 0.5 x (1 + erf(x / sqrt 2)).
__device__ __forceinline__ float gelu_f(float x) { return 0.5f * x * (1.f + erff(x * 0.70710678118654752f)); }
__device__ __forceinline__ float swiglu_f(float g, float u) {
	// hardware reciprocal (1 ulp): a correctly rounded division is ten more instructions per element, which
	// a GEMM epilogue cannot hide, and the result is rounded to bf16 anyway
	const float sig = __builtin_amdgcn_rcpf(1.f + __expf(-g));
	return g * sig * u;
}

// Gradient of silu(g) * u with respect to g and u for the incoming gradient d; shared by the activation
// backward kernel and the GEMM epilogue that fuses it, so that both give the same bits.
__device__ __forceinline__ void swiglu_bwd_f(float d, float g, float u, float& dg, float& du) {
	const float sig = 1.f / (1.f + __expf(-g));
	dg = d * u * sig * (1.f + g * (1.f - sig));
	du = d * g * sig;
}

// Half-split rotary rotation of one (x_i, x_{i+D/2}) pair by the angle whose (cos, sin) is (c, s); the backward
// passes -s.  Shared by the RoPE kernel and by the GEMM / attention epilogues that fuse it, so that all of them
// give the same bits: one rounded product and one fused multiply-add per output.
__device__ __forceinline__ void rope_rot(float lo, float hi, float c, float s, float& out_lo, float& out_hi) {
	out_lo = __builtin_fmaf(lo, c, -(hi * s));
	out_hi = __builtin_fmaf(hi, c, lo * s);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
	return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
	for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
	return v;
}

}  // namespace elf
