#include "pools.h"
#include "common.h"
#include <stdlib.h>

namespace elf {

// ---------------------------------------------------------------------------------------------
size_t DevicePool::round_up(size_t b) {
	const size_t gran = b >= (size_t(1) << 20) ? (size_t(2) << 20) : 512;
	return (b + gran - 1) / gran * gran;
}

DevicePool::~DevicePool() {
	poll_pending(true);
	trim();
}

void DevicePool::poll_pending(bool block) {
	for (size_t i = 0; i < pending_.size();) {
		hipError_t e = block ? hipEventSynchronize(pending_[i].ev) : hipEventQuery(pending_[i].ev);
		if (e == hipSuccess) {
			free(pending_[i].p);
			pending_[i] = pending_.back();
			pending_.pop_back();
		} else {
			(void)hipGetLastError();  // hipErrorNotReady is not sticky, but clear it anyway
			i++;
		}
	}
}

void* DevicePool::alloc(size_t bytes) {
	if (bytes == 0) bytes = 1;
	const size_t sz = round_up(bytes);
	if (!pending_.empty()) poll_pending(false);
	auto it = free_.find(sz);
	void* p = nullptr;
	if (it != free_.end() && !it->second.empty()) {
		p = it->second.back();
		it->second.pop_back();
	} else {
		hipError_t e = hipMalloc(&p, sz);
		if (e != hipSuccess) {
			// give cached and in-flight blocks back to the driver and retry once
			(void)hipGetLastError();
			poll_pending(true);
			trim();
			e = hipMalloc(&p, sz);
			if (e != hipSuccess) {
				(void)hipGetLastError();
				set_error("device pool: hipMalloc of %zu bytes failed: %s (live %zu, reserved %zu)", sz,
				          hipGetErrorString(e), live_, reserved_);
				return nullptr;
			}
		}
		reserved_ += sz;
		size_of_[p] = sz;
	}
	live_ += sz;
	if (live_ > peak_) peak_ = live_;
	return p;
}

void DevicePool::free(void* p) {
	if (!p) return;
	auto it = size_of_.find(p);
	if (it == size_of_.end()) return;
	live_ -= it->second;
	free_[it->second].push_back(p);
}

void DevicePool::free_after(void* p, hipEvent_t ev) {
	if (!p) return;
	pending_.push_back({p, ev});
}

void DevicePool::trim() {
	for (auto& kv : free_) {
		for (void* p : kv.second) {
			reserved_ -= kv.first;
			size_of_.erase(p);
			(void)hipFree(p);
		}
		kv.second.clear();
	}
}

// ---------------------------------------------------------------------------------------------
PinnedPool::PinnedPool(bool host_backing) : host_backing_(host_backing) {}

PinnedPool::~PinnedPool() {
	for (auto& p : parents_) {
		if (host_backing_) ::free(p.base);
		else (void)hipHostFree(p.base);
	}
}

static int64_t next_pow2(int64_t n) {
	int64_t b = 1;
	while (b < n) b <<= 1;
	return b;
}

int PinnedPool::alloc_parent(int elem_size, int dtype_key, int64_t min_elems) {
	Parent p;
	p.elem_size = elem_size;
	p.dtype_key = dtype_key;
	p.elems = next_pow2(min_elems);
	void* base = nullptr;
	const size_t bytes = (size_t)p.elems * elem_size;
	if (host_backing_) {
		base = ::malloc(bytes);
	} else {
		if (hipHostMalloc(&base, bytes, hipHostMallocDefault) != hipSuccess) {
			(void)hipGetLastError();
			base = nullptr;
		}
	}
	if (!base) {
		set_error("pinned pool: cannot allocate a %zu-byte parent chunk", bytes);
		return -1;
	}
	p.base = (char*)base;
	p.free_list.push_back({0, p.elems});
	parents_.push_back(p);
	return (int)parents_.size() - 1;
}

bool PinnedPool::allocate(int64_t elems, int elem_size, int dtype_key, Block* out) {
	const int64_t req = elems < 1 ? 1 : elems;
	int pi = -1;
	size_t si = 0;
	for (size_t i = 0; i < parents_.size() && pi < 0; i++) {
		if (parents_[i].dtype_key != dtype_key) continue;
		auto& fl = parents_[i].free_list;
		for (size_t j = 0; j < fl.size(); j++) {
			if (fl[j].second >= req) {
				pi = (int)i;
				si = j;
				break;
			}
		}
	}
	if (pi < 0) {
		pi = alloc_parent(elem_size, dtype_key, req);
		if (pi < 0) return false;
		si = 0;
	}
	Parent& p = parents_[pi];
	const int64_t off = p.free_list[si].first;
	const int64_t left = p.free_list[si].second - req;
	if (left == 0) p.free_list.erase(p.free_list.begin() + si);
	else p.free_list[si] = {off + req, left};
	Block b;
	b.ptr = p.base + (size_t)off * elem_size;
	b.parent = pi;
	b.offset = off;
	b.length = req;
	live_[b.ptr] = b;
	if (out) *out = b;
	return true;
}

bool PinnedPool::fits(int64_t elems, int dtype_key) const {
	const int64_t req = elems < 1 ? 1 : elems;
	for (const auto& p : parents_) {
		if (p.dtype_key != dtype_key) continue;
		for (const auto& seg : p.free_list)
			if (seg.second >= req) return true;
	}
	return false;
}

void PinnedPool::insert_free(Parent& p, int64_t off, int64_t len) {
	auto& fl = p.free_list;
	size_t i = 0;
	while (i < fl.size() && fl[i].first <= off) i++;
	fl.insert(fl.begin() + i, {off, len});
	std::vector<std::pair<int64_t, int64_t>> merged;
	for (auto& s : fl) {
		if (!merged.empty() && merged.back().first + merged.back().second == s.first) merged.back().second += s.second;
		else merged.push_back(s);
	}
	fl.swap(merged);
}

bool PinnedPool::free(void* ptr) {
	auto it = live_.find(ptr);
	if (it == live_.end()) return false;
	const Block b = it->second;
	live_.erase(it);
	insert_free(parents_[b.parent], b.offset, b.length);
	return true;
}

bool PinnedPool::reserve(int64_t bytes, int elem_size, int dtype_key) {
	const int64_t elems = (bytes + elem_size - 1) / elem_size;
	return alloc_parent(elem_size, dtype_key, elems) >= 0;
}

int64_t PinnedPool::size_bytes() const {
	int64_t s = 0;
	for (auto& p : parents_) s += p.elems * p.elem_size;
	return s;
}

}  // namespace elf
