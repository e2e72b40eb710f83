// Direct global -> LDS loads (gfx950 global_load_lds_dwordx4) and explicit wait counters.
//
// The load is issued through inline assembly so that the compiler does not know it writes LDS:
// its own bookkeeping would otherwise force vmcnt(0) before every later LDS read and undo any
// prefetch distance.  The price is that ordering is the caller's job: wait_vmcnt<n>() (loads
// complete in order, n = how many younger loads may stay in flight) for the wave's own loads,
// then a workgroup barrier before lanes of other waves read the data.
#pragma once
#include "common.h"

namespace elf {

// 16 bytes per lane from (base + byte_off[lane]) to LDS at lds_byte_addr + lane * 16; base and
// lds_byte_addr are wave-uniform (scalar registers; the LDS address travels in M0).
__device__ __forceinline__ void dma16(const void* base, uint32_t byte_off, uint32_t lds_byte_addr) {
	asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_byte_addr), "v"(byte_off), "s"(base) : "memory", "m0");
}

// The same with the LDS address given as a wave-uniform base plus a compile-time byte offset: M0 is
// written by the add itself.
template <int IMM>
__device__ __forceinline__ void dma16_at(const void* base, uint32_t byte_off, uint32_t lds_base) {
	asm volatile("s_add_u32 m0, %0, %3\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(byte_off), "s"(base), "n"(IMM) : "memory", "m0", "scc");
}

// s_waitcnt with explicit fields (gfx9 layout: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]).
template <int VM, int LGKM = 15>
__device__ __forceinline__ void wait_counters() {
	__builtin_amdgcn_s_waitcnt((VM & 0xF) | (0x7 << 4) | ((LGKM & 0xF) << 8) | (((VM >> 4) & 3) << 14));
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
	wait_counters<N, 15>();
}

__device__ __forceinline__ uint32_t lds_addr(const void* p) {
	return (uint32_t)(uintptr_t)(const unsigned char ELF_LDS*)p;
}

}  // namespace elf
