// Live per-launch timing with HIP events on the launch stream (see ProfScope in kernels.h).
#include <vector>

#include "common.h"
#include "kernels.h"

namespace elf {

struct ProfRec {
	int kind;
	double work;
	hipEvent_t e0, e1;
};
static bool g_on = false;
static std::vector<ProfRec> g_recs;
static std::vector<hipEvent_t> g_free_events;

static hipEvent_t get_event() {
	if (!g_free_events.empty()) {
		hipEvent_t e = g_free_events.back();
		g_free_events.pop_back();
		return e;
	}
	hipEvent_t e = nullptr;
	(void)hipEventCreate(&e);
	return e;
}

void prof_enable(int on) {
	for (auto& r : g_recs) {
		g_free_events.push_back(r.e0);
		g_free_events.push_back(r.e1);
	}
	g_recs.clear();
	g_on = on != 0;
}
bool prof_on() { return g_on; }

ProfScope::ProfScope(int kind, double work, hipStream_t s) : slot(-1), stream(s) {
	if (!g_on) return;
	ProfRec r{kind, work, get_event(), get_event()};
	if (!r.e0 || !r.e1) return;
	(void)hipEventRecord(r.e0, s);
	slot = (int)g_recs.size();
	g_recs.push_back(r);
}
ProfScope::~ProfScope() {
	if (slot >= 0) (void)hipEventRecord(g_recs[slot].e1, stream);
}

int prof_collect(int kind, double* total_ms, double* total_work) {
	int n = 0;
	double ms = 0, work = 0;
	for (auto& r : g_recs) {
		if (r.kind != kind) continue;
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

}  // namespace elf
