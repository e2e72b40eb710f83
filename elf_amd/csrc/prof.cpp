// Live per-launch timing with HIP events on the launch stream (see ProfScope and launch_kernel in kernels.h): the
// events travel in the kernel dispatches themselves and read the kernels' own start and end timestamps.
#include <vector>

#include "common.h"
#include "kernels.h"

namespace elf {

struct ProfRec {
	int kind;
	double work;
	hipEvent_t e0, e1;
	bool started;  // a launch has taken the start event
};
static bool g_on = false;
static int g_one_in = 1;          // a launch carries events with probability 1 / g_one_in
static uint32_t g_pick = 1u;      // state of the generator that picks them (restarted by prof_enable: same picks every run)
static int64_t g_launches[PROF_COUNT];
static double g_work[PROF_COUNT];
static std::vector<ProfRec> g_recs;
static std::vector<hipEvent_t> g_free_events;
static thread_local ProfScope* t_scope = nullptr;

static hipEvent_t get_event() {
	if (!g_free_events.empty()) {
		hipEvent_t e = g_free_events.back();
		g_free_events.pop_back();
		return e;
	}
	hipEvent_t e = nullptr;
	// timing only: without the system-scope fence a recorded event neither writes the caches back nor invalidates
	// them, so bracketing a launch does not disturb the launches after it
	(void)hipEventCreateWithFlags(&e, hipEventDisableSystemFence);
	return e;
}

void prof_enable(int on) {
	for (auto& r : g_recs) {
		g_free_events.push_back(r.e0);
		g_free_events.push_back(r.e1);
	}
	g_recs.clear();
	g_on = on != 0;
	g_one_in = on > 1 ? on : 1;
	g_pick = 1u;
	for (int k = 0; k < PROF_COUNT; k++) {
		g_launches[k] = 0;
		g_work[k] = 0.0;
	}
}
bool prof_on() { return g_on; }

ProfScope::ProfScope(int kind, double work, hipStream_t s, bool record) : slot(-1), stream(s), outer(nullptr) {
	if (!g_on || !record) return;
	g_launches[kind]++;
	g_work[kind] += work;
	if (g_one_in > 1) {
		// an in-dispatch event pair costs the stream about 2 us per launch (a completion signal and two timestamps
		// for every dispatch instead of one signal per batch): timing a pseudo-random subset keeps the family
		// averages and most of the stream's speed
		g_pick = g_pick * 1664525u + 1013904223u;
		if ((g_pick >> 16) % (uint32_t)g_one_in != 0) return;
	}
	ProfRec r{kind, work, get_event(), get_event(), false};
	if (!r.e0 || !r.e1) return;
	slot = (int)g_recs.size();
	g_recs.push_back(r);
	outer = t_scope;
	t_scope = this;
}
ProfScope::~ProfScope() {
	if (slot >= 0) t_scope = outer;
}

bool prof_launch_events(hipEvent_t* start, hipEvent_t* stop) {
	if (!t_scope || t_scope->slot < 0 || t_scope->slot >= (int)g_recs.size()) return false;
	ProfRec& r = g_recs[t_scope->slot];
	*start = r.started ? nullptr : r.e0;
	*stop = r.e1;
	r.started = true;
	return true;
}

int prof_collect(int kind, double* total_ms, double* total_work) {
	int n = 0;
	double ms = 0, work = 0;
	for (auto& r : g_recs) {
		if (r.kind != kind || !r.started) continue;
		if (hipEventSynchronize(r.e1) != hipSuccess) continue;
		float t = 0;
		if (hipEventElapsedTime(&t, r.e0, r.e1) != hipSuccess) continue;
		ms += t;
		work += r.work;
		n++;
	}
	if (total_ms) *total_ms = ms;
	if (total_work) *total_work = work;
	return n;
}

int64_t prof_launches(int kind, double* total_work) {
	if (kind < 0 || kind >= PROF_COUNT) return 0;
	if (total_work) *total_work = g_work[kind];
	return g_launches[kind];
}

// ---------------------------------------------------------------------------------------------
// What this GPU's memory system sustains for the simplest access patterns: the yardstick the bandwidth-bound
// kernels are compared with.  mode 0: read n bytes (every lane sums 16-byte loads; one value per workgroup is
// written), 1: copy n bytes, 2: write n bytes, 3: read three streams of n bytes (src, src + n, src + 2 n) and write one
// (their XOR): the pattern of a normalisation backward (dy, x, residual gradient in; dx out).
// A workgroup takes contiguous chunks of 256 lanes x U x 16 bytes and strides over the buffer by the grid; V = 1 uses
// non-temporal stores.
template <int MODE, int U, int V>
__global__ __launch_bounds__(256) void hbm_probe_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n16) {
	const int64_t chunk = 256 * U;
	u32x4 acc = {0u, 0u, 0u, 0u};
	for (int64_t base = (int64_t)blockIdx.x * chunk; base < n16; base += (int64_t)gridDim.x * chunk) {
		u32x4 v[U];
#pragma unroll
		for (int u = 0; u < U; u++) {
			const int64_t i = base + u * 256 + threadIdx.x;
			if constexpr (MODE == 2) v[u] = u32x4{(uint32_t)i, 1u, 2u, 3u};
			else if constexpr (MODE == 3) v[u] = i < n16 ? src[i] ^ src[i + n16] ^ src[i + 2 * n16] : u32x4{0u, 0u, 0u, 0u};
			else v[u] = i < n16 ? src[i] : u32x4{0u, 0u, 0u, 0u};
		}
#pragma unroll
		for (int u = 0; u < U; u++) {
			const int64_t i = base + u * 256 + threadIdx.x;
			if constexpr (MODE == 0) acc += v[u];
			else if (i < n16) {
				if constexpr (V == 1) __builtin_nontemporal_store(v[u], dst + i);
				else dst[i] = v[u];
			}
		}
	}
	if constexpr (MODE == 0) dst[(int64_t)blockIdx.x * 256 + threadIdx.x] = acc;  // keeps the loads alive
}

int hbm_probe(int mode, const void* src, void* dst, int64_t bytes, hipStream_t s) {
	ELF_REQUIRE(mode >= 0 && mode <= 3 && dst && (mode == 2 || src) && bytes >= 16 && bytes % 16 == 0, "hbm_probe: bad argument");
	ELF_REQUIRE(((uintptr_t)src % 16) == 0 && ((uintptr_t)dst % 16) == 0, "hbm_probe: buffers must be 16-byte aligned");
	const int64_t n16 = bytes / 16;
	const dim3 block(256);
	// the best of unroll 4 / 8, 1024 / 2048 / 8192 workgroups and plain / non-temporal stores for each pattern at 1 GiB
	if (mode == 0) ELF_LAUNCH((hbm_probe_kernel<0, 4, 0>), dim3(1024), block, 0, s, (const u32x4*)src, (u32x4*)dst, n16);
	else if (mode == 1) ELF_LAUNCH((hbm_probe_kernel<1, 4, 1>), dim3(8192), block, 0, s, (const u32x4*)src, (u32x4*)dst, n16);
	else if (mode == 3) ELF_LAUNCH((hbm_probe_kernel<3, 4, 1>), dim3(8192), block, 0, s, (const u32x4*)src, (u32x4*)dst, n16);
	else ELF_LAUNCH((hbm_probe_kernel<2, 8, 0>), dim3(8192), block, 0, s, (const u32x4*)src, (u32x4*)dst, n16);
	ELF_CHECK_HIP(hipGetLastError());
	return 0;
}

}  // namespace elf
