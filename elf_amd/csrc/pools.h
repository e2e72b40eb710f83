// Memory pools owned by a stage: a size-bucketed device cache (activation / gradient stashes and
// temporaries) and the pinned-host arena used by activation offload.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <map>
#include <unordered_map>
#include <utility>
#include <vector>

namespace elf {

// Device cache.  All users enqueue on one stream, so a buffer returned with free() may be handed
// out again immediately: the new user's kernels are ordered after the old user's on that stream.
// Buffers still being read by a side stream are returned with free_after(event).
class DevicePool {
   public:
	~DevicePool();
	void* alloc(size_t bytes);  // nullptr on failure (message in get_error())
	void free(void* p);
	// event ownership stays with the caller, who must call drain() before destroying the event
	void free_after(void* p, hipEvent_t ev);
	void poll() { if (!pending_.empty()) poll_pending(false); }  // return blocks whose event has fired
	void drain() { poll_pending(true); }                         // wait for every pending event
	void trim();                              // release every cached block to the driver
	size_t live_bytes() const { return live_; }
	size_t peak_bytes() const { return peak_; }
	size_t reserved_bytes() const { return reserved_; }
	void reset_peak() { peak_ = live_; }

   private:
	static size_t round_up(size_t b);
	void poll_pending(bool block);
	std::unordered_map<size_t, std::vector<void*>> free_;
	std::unordered_map<void*, size_t> size_of_;
	struct Pending {
		void* p;
		hipEvent_t ev;
	};
	std::vector<Pending> pending_;
	size_t live_ = 0, peak_ = 0, reserved_ = 0;
};

// Pinned-host arena with the placement policy of the reference's PinnedHostTensorPool
// (elf/execution/offload.py:14-158): per dtype, a list of parent chunks whose length is
// the next power of two of the request that created them; allocation is first fit over parents
// in creation order and over each parent's free list in offset order, carving from the start of
// the segment; free re-inserts the segment in offset order and merges adjacent segments.
class PinnedPool {
   public:
	typedef void* (*AllocFn)(size_t);
	typedef void (*FreeFn)(void*);
	// host_backing = true uses malloc/free instead of hipHostMalloc (policy tests without a GPU)
	explicit PinnedPool(bool host_backing = false);
	~PinnedPool();
	struct Block {
		void* ptr = nullptr;
		int parent = -1;      // index of the parent chunk (creation order, over all element sizes)
		int64_t offset = 0;   // in elements
		int64_t length = 0;   // in elements
	};
	bool allocate(int64_t elems, int elem_size, int dtype_key, Block* out);
	bool fits(int64_t elems, int dtype_key) const;  // whether allocate() would find room without a new parent chunk
	bool free(void* ptr);            // false if ptr is not a live block of this pool
	bool reserve(int64_t bytes, int elem_size, int dtype_key);
	int64_t size_bytes() const;      // sum of parent chunk sizes
	int n_parents() const { return (int)parents_.size(); }
	int n_free_segments(int parent) const { return (int)parents_[parent].free_list.size(); }
	std::pair<int64_t, int64_t> free_segment(int parent, int i) const { return parents_[parent].free_list[i]; }

   private:
	struct Parent {
		char* base;
		int elem_size;
		int dtype_key;
		int64_t elems;
		std::vector<std::pair<int64_t, int64_t>> free_list;  // (offset, length), sorted by offset
	};
	int alloc_parent(int elem_size, int dtype_key, int64_t min_elems);
	void insert_free(Parent& p, int64_t off, int64_t len);
	std::vector<Parent> parents_;
	std::map<void*, Block> live_;
	bool host_backing_;
};

}  // namespace elf
