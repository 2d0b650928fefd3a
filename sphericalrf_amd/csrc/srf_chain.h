// Ordered offsets across the items of a compositing launch (device only): every item publishes the number of samples
// it keeps, and an item's offset is the sum over all items before it, found by a decoupled look-back.
#pragma once
#include "srf_wave.h"
#include "srf_device.h"

namespace srf {

// Ordered offsets across items (an item: the rays of a group that a streaming workgroup takes at a time, see
// fused::items_of_group).  Every item publishes the number of samples it keeps; an
// item's offset is the sum over all items before it.  Items are bundled into segments of 64:
// inside a segment an item adds up its predecessors' counts with one 64-wide read; a
// segment's total is accumulated as its items publish (complete once all 64 have), and the sum
// over earlier segments is found by a decoupled look-back over segment entries (the totals of
// complete segments, back to the nearest segment for which somebody has left the sum of everything
// up to and including it).  With a few thousand items in flight both steps usually finish in one
// memory round trip, where a single-level look-back would have to walk back over every item in flight.
constexpr uint32_t PREPARE_WAVES = 16;   // groups per workgroup of k_chain_prepare
// Segment totals lie this many 8-byte words apart: every item in flight adds to one of a few neighbouring segments' totals, and
// additions to one stretch of memory take turns
constexpr uint32_t SEG_STRIDE = 32;
struct ChainScratch {
	unsigned long long* item_status;    // per item:    flag << 32 | count (flag 1; 3 = gave up)
	unsigned long long* seg_status;     // per segment of 64 items: items published so far << 32 | sum of their counts
	unsigned long long* seg_prefix;     // per segment: flag << 32 | count (flag 2: everything up to and including the segment, 3 = an item gave up)
	uint32_t* initial;                  // value of the compacted counter before the launch
	uint32_t* error;                    // device word: set when an item gave up
	uint32_t* slow_count;               // number of entries of slow_items
	uint32_t* n_items;                  // number of items
	uint32_t* group_words;              // per group: how many items it makes (fused::group_items_word)
	unsigned long long* group_cuts;     // per group that makes several: at which rays its items begin (fused::plan_cuts)
	uint32_t* prepare_sums;             // per workgroup of k_chain_prepare: how many items its groups make
	U2* items;                          // the items in ray order (fused::items_of_group)
	uint32_t* slow_items;               // items of groups that the streaming path does not take (see k_chain_prepare)
	uint32_t* side;                     // per ray of such a group: samples consumed (forward kernel), then compacted offset (streaming kernel)
	U2* saved_records;                  // per ray of such a group: its record on entry, which the commit overwrites (NULL: a group is worked on by one workgroup)
	uint32_t* host_error;               // like error, in host memory the device can write (may be NULL)
	uint32_t spin_limit;                // polls an item makes before it gives up
	uint32_t max_parts;                 // items a group may be cut into (what the scratch has room for)
	// the wave-per-item kernel's words (these three are zero between calls: its last workgroup to leave clears them)
	uint32_t* ticket;                   // rounds of items handed out so far
	uint32_t* disorder;                 // set when the call's rays are not laid out in increasing order
	uint32_t* exits;                    // workgroups that have left
	uint32_t* stride;                   // stride of the sample windows
	void* item_desc;                    // per item: its rays and samples (wv::ItemDesc)
	void* args_copy;                    // the call's fused::Args and this structure, in device memory
	void* scratch_copy;
};

constexpr uint32_t LOOKBACK_SLEEP = 2;
constexpr uint32_t CHAIN_FAILED = 0xffffffffu;   // prefix of a group whose look-back gave up; also what the compacted counter reads then

__device__ inline unsigned long long status_load(const unsigned long long* p) {
	return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void status_store(unsigned long long* p, uint32_t flag, uint32_t value) {
	__hip_atomic_store(p, ((unsigned long long)flag << 32) | value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// a segment's prefix word only ever goes up: nothing (0) -> prefix (flag 2) -> an item gave up (flag 3), whoever writes last
__device__ inline void status_raise(unsigned long long* p, uint32_t flag, uint32_t value) {
	(void)__hip_atomic_fetch_max(p, ((unsigned long long)flag << 32) | value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// An item's count, visible to every item after it (one lane): its own status word, and its share of its segment's running total.
__device__ inline void chain_publish(const ChainScratch& S, uint32_t i, uint32_t total) {
	if (lane_id() == 0) {
		status_store(&S.item_status[i], 1u, total);
		(void)__hip_atomic_fetch_add(&S.seg_status[(size_t)(i / WAVE) * SEG_STRIDE], (1ull << 32) | total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	}
}

// Exclusive prefix of item i over the items before it, by the 64 lanes of one wave.  An item only waits for
// lower-numbered items.  Both levels are read in the same round trip (each lane loads one item entry of its own
// segment and the entries of one earlier segment); a round is repeated until nothing it needs is missing.  The first round's
// loads can be requested long before their values are needed (chain_peek), so that the round trip overlaps other work; the words
// only ever move from "missing" to "there", so an early value is either final or asks for another round.  Everything an item
// needs is put there when its predecessors publish their counts, never when they resolve their own prefixes, so an item waits only
// for a workgroup that has fallen behind by the time that passes between an item's count and its look-back.
// Every wait is bounded: past the limit, or when a predecessor has given up, the item gives up too: it marks its own
// entries so that its successors stop at once, raises the error words and returns CHAIN_FAILED.
struct ChainPeek { unsigned long long vg, vs, vp; uint32_t initial; };

// initial: *S.initial, for a caller that has read it already
__device__ inline ChainPeek chain_peek(const ChainScratch& S, uint32_t i, uint32_t initial) {
	const uint32_t lane = lane_id();
	const uint32_t seg = i / WAVE, j = i % WAVE;
	ChainPeek p;
	p.initial = initial;
	p.vg = 1ull << 32;
	if (j != 0 && lane < j) p.vg = status_load(&S.item_status[seg * WAVE + lane]);
	p.vs = 0ull;
	p.vp = (2ull << 32) | p.initial;                  // before the first segment: the counter's value before the launch
	const int64_t idx = (int64_t)seg - 1 - (int64_t)lane;
	if (idx >= 0) { p.vs = status_load(&S.seg_status[(size_t)idx * SEG_STRIDE]); p.vp = status_load(&S.seg_prefix[idx]); }
	return p;
}

__device__ inline ChainPeek chain_peek(const ChainScratch& S, uint32_t i) { return chain_peek(S, i, *S.initial); }

__device__ inline uint32_t chain_resolve(const ChainScratch& S, uint32_t i, uint32_t total, const ChainPeek& peek) {
	const uint32_t lane = lane_id();
	const uint32_t seg = i / WAVE, j = i % WAVE;
	const uint32_t initial = peek.initial;
	uint32_t spins = 0, within = 0, before = 0;
	bool have_within = j == 0, have_before = false, failed = false, first = true;
	int64_t hi = (int64_t)seg - 1;
	for (;;) {
		unsigned long long vg = 1ull << 32, vs = 0ull, vp = (2ull << 32) | initial;
		if (first) {
			vg = peek.vg; vs = peek.vs; vp = peek.vp;
		} else {
			if (!have_within && lane < j) vg = status_load(&S.item_status[seg * WAVE + lane]);
			const int64_t idx = hi - (int64_t)lane;
			if (!have_before && idx >= 0) { vs = status_load(&S.seg_status[(size_t)idx * SEG_STRIDE]); vp = status_load(&S.seg_prefix[idx]); }
		}
		first = false;
		const uint32_t gflag = (uint32_t)(vg >> 32), pflag = (uint32_t)(vp >> 32);
		if (__ballot(gflag == 3u) != 0ull) { failed = true; break; }
		if (!have_within && __ballot(gflag == 0u) == 0ull) {
			within = wave_sum_fast(lane < j ? (uint32_t)vg : 0u);
			have_within = true;
		}
		if (!have_before) {
			// a segment's entry: its inclusive prefix (left by whoever has resolved past it), else its total once all of its items have published
			const bool complete = (uint32_t)(vs >> 32) == WAVE;
			const unsigned long long has_prefix = __ballot(pflag == 2u);
			const unsigned long long missing = __ballot(pflag != 2u && pflag != 3u && !complete);
			const unsigned long long poisoned = __ballot(pflag == 3u);
			const uint32_t first_prefix = has_prefix ? (uint32_t)__builtin_ctzll(has_prefix) : 64u;
			const uint32_t first_missing = missing ? (uint32_t)__builtin_ctzll(missing) : 64u;
			const uint32_t first_poisoned = poisoned ? (uint32_t)__builtin_ctzll(poisoned) : 64u;
			if (first_poisoned < first_prefix && first_poisoned < first_missing) { failed = true; break; }
			if (first_prefix < first_missing) {
				before += wave_sum_fast(lane < first_prefix ? (uint32_t)vs : (lane == first_prefix ? (uint32_t)vp : 0u));
				have_before = true;
			} else if (first_missing == 64u) { before += wave_sum_fast((uint32_t)vs); hi -= 64; continue; }   // 64 totals, no prefix yet: look further back
		}
		if (have_before && have_within) break;
		if (++spins > S.spin_limit) { failed = true; break; }
		__builtin_amdgcn_s_sleep(LOOKBACK_SLEEP);
	}
	if (failed) {
		if (lane == 0) {
			status_store(&S.item_status[i], 3u, 0u);
			status_raise(&S.seg_prefix[seg], 3u, 0u);
			atomicExch(S.error, 1u);
			if (S.host_error) __hip_atomic_store(S.host_error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
		}
		return CHAIN_FAILED;
	}
	// shortcuts for later look-backs: the prefix up to the end of the segment before this one, and up to the end of this one
	if (lane == 0) {
		if (j == 0 && seg != 0) status_raise(&S.seg_prefix[seg - 1], 2u, before);
		if (j == WAVE - 1) status_raise(&S.seg_prefix[seg], 2u, before + within + total);
	}
	return before + within;
}

} // namespace srf
