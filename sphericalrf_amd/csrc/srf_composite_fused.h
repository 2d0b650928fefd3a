// Single-launch training compositing (forward, loss, ordered compaction, backward).
//
// A group is RAYS consecutive rays.  Because a sampler that assigns offsets in ray
// order lays the samples of consecutive rays out back to back, the group's samples form
// one contiguous range, which is streamed through the group in windows of WIN samples:
//
//   phase A  (thread <-> sample)  coalesced loads of rgb-sigma and dt; alpha = 1 - exp(-sigma dt);
//                                 {alpha, colour} of every sample goes to LDS
//   count    (lane   <-> ray)     the transmittance part of the reference's loop alone (termination test,
//                                 T *= (1 - alpha)): how many samples the ray consumes.  The group's total
//                                 is published to the other groups as soon as it is known.
//   chain    (lane   <-> ray)     the reference's loop over those samples in order: weight = alpha * T,
//                                 colour sum, T *= (1 - alpha); the transmittance after each sample and
//                                 the colour sum including it replace the sample's LDS record
//   finish   (lane   <-> ray)     background, target, loss, gradient of the loss; the group's
//                                 compacted count is chained to its predecessors' (decoupled
//                                 look-back over groups) to get ordered offsets
//   phase C  (thread <-> sample)  gradients from the exact per-sample T and colour prefix,
//                                 stored at the compacted position
//
// Only the chain is sequential, and it carries nine arithmetic operations per sample with the
// exponentials, conversions and gradient arithmetic left to the sample-parallel phases; every
// value a sample's gradient depends on is produced by the same operations in the same order
// as a one-thread-per-ray loop, so the results are bit-identical to it.
//
// Groups whose rays are not laid out back to back in increasing order (arbitrary caller
// supplied offsets) take a per-ray path with the same arithmetic.  Groups whose samples do not
// fit one window run the forward phases over all windows first and then a second sweep that
// recomputes them and emits gradients.
//
// The phases are host/device functions of (thread id, shared block state, per-thread state) so
// that a host build can run a group phase by phase in plain loops.
#pragma once
#include "srf_bodies.h"

#if defined(__HIP_DEVICE_COMPILE__)
// a value that is the same in every lane of the wave (read from LDS, say), moved to where the compiler knows it is
#define SRF_UNIFORM_U32(x) ((uint32_t)__builtin_amdgcn_readfirstlane((int)(x)))
#define SRF_LDS_ADD(p, v) atomicAdd((p), (v))
#define SRF_LDS_AND(p, v) atomicAnd((p), (v))
// keeps the instruction scheduler from interleaving the unrolled per-slot bodies, which would
// multiply the live temporaries by the slot count and cost occupancy
#define SRF_SLOT_FENCE() __builtin_amdgcn_sched_barrier(0)
#else
#define SRF_UNIFORM_U32(x) ((uint32_t)(x))
#define SRF_LDS_ADD(p, v) (*(p) += (v))
#define SRF_LDS_AND(p, v) (*(p) &= (v))
#define SRF_SLOT_FENCE() ((void)0)
#endif

namespace srf {
namespace fused {

constexpr uint32_t RAYS = 64;        // rays per group: one lane of a wavefront per ray during count, chain and finish
constexpr uint32_t RAYS_HI = 8, RAYS_LO = 8;
static_assert(RAYS_HI * RAYS_LO == RAYS, "group shape");

// how many threads share the sample-parallel phases of a group and how many samples each of them holds in registers
// FENCE_SLOTS: keep the scheduler from interleaving the per-slot bodies (a kernel with a tight register budget)
template <uint32_t THREADS_, uint32_t SLOTS_, bool FENCE_SLOTS_>
struct Geometry {
	static constexpr uint32_t THREADS = THREADS_;
	static constexpr uint32_t SLOTS = SLOTS_;
	static constexpr uint32_t WIN = THREADS_ * SLOTS_;   // samples per window
	static constexpr bool FENCE_SLOTS = FENCE_SLOTS_;
};
// a whole workgroup of four waves on the samples, windows of 1792: the kernel for groups of any length
using WideGeometry = Geometry<256, 7, true>;
// six waves on the samples (two more walk the rays and plan meanwhile), windows of 1920: the streaming kernel
using StreamGeometry = Geometry<384, 5, false>;

constexpr uint32_t GAP_SLACK = 1024; // a group whose sample range exceeds its sample count by more takes the per-ray path
constexpr uint32_t CHAIN_UNROLL = 8;
constexpr uint32_t COUNT_UNROLL = 8;
constexpr uint32_t NPLAN = 4;        // plans kept at once by a kernel that has three items under way and plans a fourth

// M_LANE_LO / M_LANE_HI: the rays (lanes) of the group that this plan covers; M_GROUP: which group; M_ITEM: the number
// of the item that the plan is for (NO_ITEM: none, the plan is a placeholder), set by kernels that number their items
enum { M_S0 = 0, M_TOTAL, M_SUM, M_CONTIG, M_LANE_LO, M_LANE_HI, M_GROUP, M_ITEM, M_N };
constexpr uint32_t NO_ITEM = 0xffffffffu;

// per ray, read by phase C
struct alignas(16) RayOut {
	float g[3];         // d loss / d colour
	uint32_t obase;     // compacted offset of the ray minus the position of its first sample in the group: a kept sample at position s lands at obase + s
	float c[3];         // composited colour
	uint32_t s_end;     // position in the group after the ray's last kept sample (kept: after the compacted-capacity clamp)
};

// where a group's rays lie in the sample buffer
struct Plan {
	uint32_t rabs[RAYS];        // absolute first-sample index per ray
	uint32_t rbase[RAYS + 1];   // first-sample index relative to the group's first sample
	uint32_t rn[RAYS];          // samples of the ray on input
	uint32_t misc[M_N];
};
template <class G>
SRF_HD bool plan_fits_one_window(const Plan& pl) { return pl.misc[M_CONTIG] != 0 && pl.misc[M_TOTAL] <= G::WIN; }

// Where a kernel with windows of G::WIN samples cuts a planned group into items: bit r of the result is set when an item
// starts at ray r.  Greedy from the front: an item takes rays for as long as the stretch from its first ray's first sample to
// the next ray's first sample (the group's end after the last ray) fits one window.  0 when the kernel cannot take the group:
// rays not laid out back to back, a single ray longer than a window, more than max_parts items.
constexpr uint32_t MAX_PARTS = RAYS;     // at worst every ray is an item of its own
template <class G>
SRF_HD uint64_t plan_cuts(const Plan& pl, uint32_t max_parts) {
	if (pl.misc[M_CONTIG] == 0) return 0ull;
	const uint32_t total = pl.misc[M_TOTAL];
	if (total <= G::WIN) return 1ull;
	uint64_t cuts = 1ull;
	uint32_t parts = 1, lo = 0;
	for (uint32_t r = 1; r <= RAYS; ++r) {
		const uint32_t end = r < RAYS ? pl.rbase[r] : total;      // where ray r - 1 and the gap after it end
		if (end - pl.rbase[lo] <= G::WIN) continue;
		if (r - 1 == lo) return 0ull;                              // ray lo alone does not fit
		lo = r - 1;
		cuts |= 1ull << lo;
		if (++parts > max_parts || end - pl.rbase[lo] > G::WIN) return 0ull;
	}
	return cuts;
}

// Where the kernel for the listed groups cuts a group whose rays lie back to back: as plan_cuts, except that a ray longer than
// a window is a part of its own (that kernel takes a part through as many windows as it needs).
template <class G>
SRF_HD uint64_t plan_cuts_any_length(const Plan& pl) {
	const uint32_t total = pl.misc[M_TOTAL];
	uint64_t cuts = 1ull;
	uint32_t lo = 0;
	for (;;) {
		uint32_t r = lo;      // the first ray from lo on that ends beyond the window beginning with ray lo
		while (r < RAYS && (r + 1 < RAYS ? pl.rbase[r + 1] : total) - pl.rbase[lo] <= G::WIN) ++r;
		if (r == lo) ++r;     // ray lo alone is longer than a window
		if (r >= RAYS) return cuts;
		lo = r;
		cuts |= 1ull << lo;
	}
}

// The plan of rays [lo, hi) of a planned group, one lane per ray: the other rays own nothing in it.
SRF_HD void plan_part_lane(uint32_t lane, const Plan& group, uint32_t lo, uint32_t hi, uint32_t g, Plan& part) {
	const uint32_t start = group.rbase[lo];
	const uint32_t end = hi < RAYS ? group.rbase[hi] : group.misc[M_TOTAL];
	const uint32_t total = end - start;
	const bool mine = lane >= lo && lane < hi;
	part.rabs[lane] = group.rabs[lane];
	part.rn[lane] = mine ? group.rn[lane] : 0u;
	part.rbase[lane] = lane < lo ? 0u : (lane < hi ? group.rbase[lane] - start : total);
	if (lane == 0) {
		part.rbase[RAYS] = total;
		part.misc[M_S0] = group.misc[M_S0] + start;
		part.misc[M_TOTAL] = total;
		part.misc[M_SUM] = 0;
		part.misc[M_CONTIG] = 1;
		part.misc[M_LANE_LO] = lo;
		part.misc[M_LANE_HI] = hi;
		part.misc[M_GROUP] = g;
	}
}

// An item is what a streaming workgroup takes at a time: rays [lo, hi) of one group.  A group is one item, or several when
// it is cut (plan_cuts), and the items of all groups, in ray order, are the units of the ordered-offset chain.
//   x  group
//   y  lo | hi << 8 | listed << 16   (listed: the streaming path does not take the group, see plan_cuts == 0)
// What k_chain_prepare leaves per group for the pass that numbers the items: items | listed << 16 (and the cuts themselves
// when there are several).
SRF_HD uint32_t group_items_word(uint64_t cuts) { return cuts ? (uint32_t)__builtin_popcountll(cuts) : (1u | 1u << 16); }
SRF_HD U2 make_item(uint32_t g, uint32_t lo, uint32_t hi, bool listed) {
	U2 item;
	item.x = g;
	item.y = lo | (hi << 8) | (listed ? 1u << 16 : 0u);
	return item;
}
// the items of a group in ray order, written to out[0 .. n): the whole group when it is listed or not cut
SRF_HD uint32_t items_of_group(uint32_t g, uint32_t word, uint64_t cuts, U2* out) {
	const uint32_t n = word & 0xffu;
	const bool listed = (word & (1u << 16)) != 0u;
	if (listed || n <= 1u) { out[0] = make_item(g, 0u, RAYS, listed); return 1u; }
	for (uint32_t k = 0; k < n; ++k) {
		const uint32_t lo = (uint32_t)__builtin_ctzll(cuts);
		cuts &= cuts - 1ull;
		out[k] = make_item(g, lo, cuts ? (uint32_t)__builtin_ctzll(cuts) : RAYS, false);
	}
	return n;
}
SRF_HD uint32_t item_lo(U2 item) { return item.y & 0xffu; }
SRF_HD uint32_t item_hi(U2 item) { return (item.y >> 8) & 0xffu; }
SRF_HD bool item_listed(U2 item) { return (item.y >> 16) != 0; }

constexpr uint32_t NO_OWNER = 0xffu;

// one window of samples in LDS
//   S      phase A: {alpha, r, g, b}; after the chain: {T before the sample, colour sum r, g, b including it}
//   owner  which ray's chain consumed the sample (NO_OWNER: none), written by the chain, read by phase C
constexpr uint32_t CHAIN_LOOKAHEAD = 8;   // records the ray loops may read past a ray's last sample (they are not used)
template <class G>
struct Window {
	Float4 S[G::WIN + CHAIN_LOOKAHEAD];
	uint8_t owner[G::WIN];
};

// per-ray results of a group in LDS
struct RayLds {
	RayOut out[RAYS];
	uint32_t rnf[RAYS];         // samples consumed by the forward pass (early termination)
	float loss[RAYS];           // loss of the ray, parked until the clamp is known
	Float4 carry[RAYS];         // transmittance and colour sum the chain left (for a kernel whose chain and finish run on different waves)
};

template <class G, bool HALF_IN>
struct SlotState {
	uint32_t raw[G::SLOTS][HALF_IN ? 2 : 4];
	float dt[G::SLOTS];
	float alpha[G::SLOTS];
};

struct RayCarry { float T, Cr, Cg, Cb; uint32_t k; uint32_t numsteps; uint32_t done; };

struct Args {
	LossConst K;
	uint32_t n_active;
	const float* rays_rgba;
	uint32_t* ray_coord_indices;
	const float* dt_arr;
	const float* coords;
	float* compacted_coords;
	const void* net;
	void* dloss;
	float* loss_output;
	float* rgb_ray_out;
	float mean_density;
};

template <bool HALF_IN>
SRF_HD void unpack_raw(const uint32_t* raw, float v[4]) {
	if constexpr (HALF_IN) {
		v[0] = half_bits_to_float((uint16_t)(raw[0] & 0xffffu)); v[1] = half_bits_to_float((uint16_t)(raw[0] >> 16));
		v[2] = half_bits_to_float((uint16_t)(raw[1] & 0xffffu)); v[3] = half_bits_to_float((uint16_t)(raw[1] >> 16));
	} else {
		v[0] = srf_u2f(raw[0]); v[1] = srf_u2f(raw[1]); v[2] = srf_u2f(raw[2]); v[3] = srf_u2f(raw[3]);
	}
}

// ---- set-up: one lane per ray ------------------------------------------------------------
// The ray's record and its target colour are fetched together, before anything depends on them
// (records of rays past the active count are read too, and ignored: the buffers hold K.n_rays entries).
SRF_HD void load_ray(uint32_t lane, uint32_t ray0, const Args& A, Plan& pl, Float4* target_rgba) {
	const uint32_t i = ray0 + lane;
	uint32_t n = 0, b = 0;
	*target_rgba = mk4(0.f, 0.f, 0.f, 0.f);
	if (i < A.K.n_rays) {
		const U2 rec = *(const U2*)(A.ray_coord_indices + 2 * (size_t)i);
		*target_rgba = *(const Float4*)(A.rays_rgba + 4 * (size_t)i);
		if (i < A.n_active) { n = rec.x; b = rec.y; }
	}
	pl.rn[lane] = n;
	pl.rabs[lane] = b;
}

// layout check and relative offsets, one lane per ray; misc[M_SUM] = 0 and misc[M_CONTIG] = 1 beforehand
SRF_HD void plan_lane(uint32_t lane, uint32_t ray0, const Args& A, Plan& pl) {
	const uint32_t n_here = A.n_active > ray0 ? (A.n_active - ray0 < RAYS ? A.n_active - ray0 : RAYS) : 0;
	const uint32_t s0 = n_here ? pl.rabs[0] : 0;
	if (lane < n_here) {
		const uint64_t prev_end = lane ? (uint64_t)pl.rabs[lane - 1] + pl.rn[lane - 1] : (uint64_t)s0;
		if ((uint64_t)pl.rabs[lane] < prev_end) SRF_LDS_AND(&pl.misc[M_CONTIG], 0u);
		pl.rbase[lane] = pl.rabs[lane] - s0;
		SRF_LDS_ADD(&pl.misc[M_SUM], pl.rn[lane]);
	}
	if (lane == 0) {
		const uint64_t end = n_here ? (uint64_t)pl.rabs[n_here - 1] + pl.rn[n_here - 1] : 0;
		pl.misc[M_S0] = s0;
		pl.misc[M_TOTAL] = (uint32_t)end - s0;      // modulo 2^32: in the plan of a part of the group the first ray's offset cancels
		if (!(end >= s0 && end - s0 <= 0xffffffffull)) SRF_LDS_AND(&pl.misc[M_CONTIG], 0u);
	}
}

// after plan_lane of every lane: rays past the end own nothing; big gaps disqualify the group
SRF_HD void plan_finish_lane(uint32_t lane, uint32_t ray0, const Args& A, Plan& pl) {
	const uint32_t n_here = A.n_active > ray0 ? (A.n_active - ray0 < RAYS ? A.n_active - ray0 : RAYS) : 0;
	const uint32_t total = pl.misc[M_TOTAL];
	if (lane >= n_here) pl.rbase[lane] = total;
	if (lane == 0) {
		pl.rbase[RAYS] = total;
		if ((uint64_t)total > (uint64_t)pl.misc[M_SUM] + GAP_SLACK) pl.misc[M_CONTIG] = 0;
		pl.misc[M_LANE_LO] = 0; pl.misc[M_LANE_HI] = RAYS;
		pl.misc[M_GROUP] = ray0 / RAYS;
	}
}

SRF_HD void reset_carry(uint32_t lane, const Plan& pl, RayCarry& c) {
	c.T = 1.f; c.Cr = 0.f; c.Cg = 0.f; c.Cb = 0.f; c.k = 0; c.numsteps = pl.rn[lane]; c.done = 0;
}

// ---- phase A: thread <-> sample ----------------------------------------------------------
// loads: every slot inside the group's range is fetched, whether or not a ray owns it (holes left by
// dropped rays lie between valid samples, inside the buffer), so the loads wait for nothing but the plan
template <class G, bool HALF_IN>
SRF_HD void phase_a_load(uint32_t tid, uint32_t win, const Args& A, const Plan& pl, SlotState<G, HALF_IN>& st) {
	const uint32_t total = pl.misc[M_TOTAL], s0 = pl.misc[M_S0];
	const uint32_t in_window = total - win * G::WIN < G::WIN ? total - win * G::WIN : G::WIN;
	const uint32_t n_slots = (in_window + G::THREADS - 1) / G::THREADS;     // the same for every thread: unused slot rows are skipped outright
	#pragma unroll
	for (uint32_t j = 0; j < G::SLOTS; ++j) {
		const uint32_t srel = win * G::WIN + tid + j * G::THREADS;
		if (j < n_slots && srel < total) {
			const size_t s = (size_t)s0 + srel;
			if constexpr (HALF_IN) {
				const U2 p = *(const U2*)((const uint32_t*)A.net + s * 2);
				st.raw[j][0] = p.x; st.raw[j][1] = p.y;
			} else {
				const U4 p = *(const U4*)((const uint32_t*)A.net + s * 4);
				st.raw[j][0] = p.x; st.raw[j][1] = p.y; st.raw[j][2] = p.z; st.raw[j][3] = p.w;
			}
			st.dt[j] = A.dt_arr[s * A.K.dt_stride];
		}
	}
}

// The same loads for a plan that fits one window, with the addresses built from one base per array and a 32-bit offset
// per thread.  A slot past the range re-reads the range's last sample instead of being skipped (its values are not used):
// nothing here depends on the lane, so the registers need no merging with their old contents.
template <class G, bool HALF_IN>
SRF_HD void phase_a_load_single(uint32_t tid, const Args& A, const Plan& pl, SlotState<G, HALF_IN>& st) {
	const uint32_t total = SRF_UNIFORM_U32(pl.misc[M_TOTAL]), s0 = SRF_UNIFORM_U32(pl.misc[M_S0]);
	if (total == 0) return;
	const uint32_t n_slots = (total + G::THREADS - 1) / G::THREADS;
	const uint32_t* net = (const uint32_t*)A.net + (size_t)s0 * (HALF_IN ? 2 : 4);
	const float* dt = A.dt_arr + (size_t)s0 * A.K.dt_stride;
	#pragma unroll
	for (uint32_t j = 0; j < G::SLOTS; ++j) {
		if (j < n_slots) {
			const uint32_t q = tid + j * G::THREADS;
			const uint32_t srel = q < total ? q : total - 1;
			if constexpr (HALF_IN) {
				const U2 p = *(const U2*)(net + srel * 2u);
				st.raw[j][0] = p.x; st.raw[j][1] = p.y;
			} else {
				const U4 p = *(const U4*)(net + srel * 4u);
				st.raw[j][0] = p.x; st.raw[j][1] = p.y; st.raw[j][2] = p.z; st.raw[j][3] = p.w;
			}
			st.dt[j] = dt[(size_t)srel * A.K.dt_stride];
		}
	}
}

// activations and alpha of every slot in the range; {alpha, colour} goes to LDS.  Which ray a sample belongs to
// does not matter here (a slot in a hole between rays gets a meaningless record that no chain reads); the chain
// marks the samples it consumes and phase C works from those marks.
// PLAIN: both activations are "None", known at compile time (the arithmetic is the same, the switches are gone)
template <class G, bool HALF_IN, bool PLAIN = false>
SRF_HD void phase_a_compute(uint32_t tid, uint32_t win, const Args& A, Window<G>& w, const Plan& pl, SlotState<G, HALF_IN>& st) {
	const int rgb_act = PLAIN ? (int)SRF_ACT_NONE : A.K.rgb_act, density_act = PLAIN ? (int)SRF_ACT_NONE : A.K.density_act;
	const uint32_t total = pl.misc[M_TOTAL];
	const uint32_t in_window = total - win * G::WIN < G::WIN ? total - win * G::WIN : G::WIN;
	const uint32_t n_slots = (in_window + G::THREADS - 1) / G::THREADS;
	#pragma unroll
	for (uint32_t j = 0; j < G::SLOTS; ++j) {
		if (G::FENCE_SLOTS) SRF_SLOT_FENCE();
		const uint32_t q = tid + j * G::THREADS;
		const uint32_t srel = win * G::WIN + q;
		if (j < n_slots && srel < total) {
			float v[4];
			unpack_raw<HALF_IN>(st.raw[j], v);
			const float density = act_density(v[3], density_act);
			const float alpha = 1.f - srf_expf(-density * st.dt[j]);
			st.alpha[j] = alpha;
			w.S[q] = mk4(alpha, act_rgb(v[0], rgb_act), act_rgb(v[1], rgb_act), act_rgb(v[2], rgb_act));
			w.owner[q] = (uint8_t)NO_OWNER;
		}
	}
}

template <class G, bool HALF_IN, bool PLAIN = false>
SRF_HD void phase_a(uint32_t tid, uint32_t win, const Args& A, Window<G>& w, const Plan& pl, SlotState<G, HALF_IN>& st) {
	phase_a_load<G, HALF_IN>(tid, win, A, pl, st);
	phase_a_compute<G, HALF_IN, PLAIN>(tid, win, A, w, pl, st);
}

// ---- count: lane <-> ray (the transmittance half of ray_marcher.cu:63-79) -------------------
// How many samples the reference's loop consumes before the transmittance falls below the threshold: the same
// T *= (1 - alpha) sequence the chain runs, without the colours.  For groups that fit one window.
// Every lane runs n_max steps (the largest count among the lanes that run together) without branching: a lane keeps
// multiplying after its ray has ended or terminated, which changes nothing, and latches the first step at which the
// reference's test `T < threshold` (made before a sample is consumed) holds.  Reads past the ray's end are clamped to the
// window's padding.
template <class G>
SRF_HD uint32_t count_lane(uint32_t lane, uint32_t n_max, const Args& A, const Window<G>& w, const Plan& pl) {
	const Float4* S = w.S;
	const uint32_t last = G::WIN + CHAIN_LOOKAHEAD - 1;
	const uint32_t base = pl.rbase[lane];
	uint32_t cnt = pl.rn[lane];
	float T = 1.f;
	const float thr = A.K.thr;
	for (uint32_t k = 0; k < n_max; k += COUNT_UNROLL) {
		float a[COUNT_UNROLL];
		#pragma unroll
		for (uint32_t u = 0; u < COUNT_UNROLL; ++u) a[u] = S[base + k + u < last ? base + k + u : last].x;
		// only the products depend on one another: the first step at which the test holds is the smallest such step
		uint32_t first = 0xffffffffu;
		#pragma unroll
		for (uint32_t u = 0; u < COUNT_UNROLL; ++u) {
			const uint32_t here = T < thr ? k + u : 0xffffffffu;
			first = here < first ? here : first;
			T *= (1.f - a[u]);
		}
		cnt = first < cnt ? first : cnt;
	}
	return cnt;
}

// ---- chain with the count known: lane <-> ray (ray_marcher.cu:63-79, :171-182) -------------------
// The reference's loop over the n_fwd samples count_lane found: no termination test is left in it.  Every lane runs
// n_max steps (the largest n_fwd among the lanes that run together); steps past a lane's n_fwd change nothing.
// The steps [k_lo, k_hi) of that loop (k_lo a multiple of CHAIN_UNROLL; the lane's ray is carried in c from one stretch to the next).
// MARK_OWNER = false: the samples' owner marks are written elsewhere (mark_owners)
template <class G, bool MARK_OWNER = true>
SRF_HD void chain_counted_steps(uint32_t lane, uint32_t n_fwd, uint32_t k_lo, uint32_t k_hi, Window<G>& w, const Plan& pl, RayCarry& c) {
	const uint32_t base = pl.rbase[lane];
	const uint32_t last = G::WIN + CHAIN_LOOKAHEAD - 1;
	float T = c.T, r = c.Cr, g = c.Cg, b = c.Cb;
	for (uint32_t k = k_lo; k < k_hi; k += CHAIN_UNROLL) {
		Float4 v[CHAIN_UNROLL];
		#pragma unroll
		for (uint32_t u = 0; u < CHAIN_UNROLL; ++u) v[u] = w.S[base + k + u < last ? base + k + u : last];
		// A step past the ray's count runs on an all-zero record (what was read there may be anything, not-a-number included), which
		// leaves T (times 1) and the colour sums (plus 0) as they are, so the stretch needs no branches; written so that only T's
		// products and each colour's sums depend on one another.
		float a[CHAIN_UNROLL], Tb[CHAIN_UNROLL], wgt[CHAIN_UNROLL];
		Float4 out[CHAIN_UNROLL];
		#pragma unroll
		for (uint32_t u = 0; u < CHAIN_UNROLL; ++u) {
			if (!(k + u < n_fwd)) v[u] = mk4(0.f, 0.f, 0.f, 0.f);
			a[u] = v[u].x;
		}
		#pragma unroll
		for (uint32_t u = 0; u < CHAIN_UNROLL; ++u) { Tb[u] = T; wgt[u] = a[u] * T; T *= (1.f - a[u]); }
		#pragma unroll
		for (uint32_t u = 0; u < CHAIN_UNROLL; ++u) {
			r += wgt[u] * v[u].y; g += wgt[u] * v[u].z; b += wgt[u] * v[u].w;
			out[u] = mk4(Tb[u], r, g, b);
		}
		#pragma unroll
		for (uint32_t u = 0; u < CHAIN_UNROLL; ++u) {
			if (k + u < n_fwd) {
				w.S[base + k + u] = out[u];
				if (MARK_OWNER) w.owner[base + k + u] = (uint8_t)lane;
			}
		}
	}
	c.T = T; c.Cr = r; c.Cg = g; c.Cb = b;
}
SRF_HD void chain_counted_begin(RayCarry& c) { c.T = 1.f; c.Cr = 0.f; c.Cg = 0.f; c.Cb = 0.f; }
SRF_HD void chain_counted_end(uint32_t lane, uint32_t n_fwd, RayLds& rl, const Plan& pl, RayCarry& c) {
	c.k = n_fwd; c.numsteps = pl.rn[lane]; c.done = 0;
	rl.rnf[lane] = n_fwd;
	rl.carry[lane] = mk4(c.T, c.Cr, c.Cg, c.Cb);
}
template <class G, bool MARK_OWNER = true>
SRF_HD void chain_counted(uint32_t lane, uint32_t n_fwd, uint32_t n_max, Window<G>& w, RayLds& rl, const Plan& pl, RayCarry& c) {
	chain_counted_begin(c);
	chain_counted_steps<G, MARK_OWNER>(lane, n_fwd, 0, n_max, w, pl, c);
	chain_counted_end(lane, n_fwd, rl, pl, c);
}

// Owner marks of a one-window plan, lane <-> ray: every sample in a ray's range is marked with the ray, whether or not the
// chain will consume it (phase C tells by the ray's count); n_max: the largest range among the lanes that run together.
// After phase A, which marks every sample as nobody's.
template <class G>
SRF_HD void mark_owners(uint32_t lane, uint32_t n_max, Window<G>& w, const Plan& pl) {
	const uint32_t base = pl.rbase[lane], n = pl.rn[lane];
	for (uint32_t k = 0; k < n_max; ++k) if (k < n) w.owner[base + k] = (uint8_t)lane;
}

// where chain_counted left the lane's ray, read back by another wave
SRF_HD void carry_from_lds(uint32_t lane, const RayLds& rl, const Plan& pl, RayCarry& c) {
	const Float4 v = rl.carry[lane];
	c.T = v.x; c.Cr = v.y; c.Cg = v.z; c.Cb = v.w;
	c.k = rl.rnf[lane]; c.numsteps = pl.rn[lane]; c.done = 0;
}

// ---- chain over one window of a longer group: lane <-> ray (ray_marcher.cu:63-79; the same loop again at :171-182) ----
// Walks the ray's samples inside this window in order: early-termination test, weight,
// colour sum, transmittance; leaves {T before the sample, colour sum including it} in place.
template <class G>
SRF_HD void chain(uint32_t lane, uint32_t win, const Args& A, Window<G>& w, RayLds& rl, const Plan& pl, RayCarry& c) {
	const uint32_t base = pl.rbase[lane];
	const uint32_t win_lo = win * G::WIN;
	// samples of this ray that lie in the window: k in [c.k, k_end)
	uint32_t k_end = c.numsteps;
	if (base + k_end > win_lo + G::WIN) k_end = win_lo + G::WIN > base ? win_lo + G::WIN - base : 0;
	float T = c.T, r = c.Cr, g = c.Cg, b = c.Cb;
	uint32_t k = c.k;
	bool stop = c.done != 0;     // a ray that terminated in an earlier window stays where it stopped
	while (k < k_end && !stop) {
		Float4 v[CHAIN_UNROLL];
		#pragma unroll
		for (uint32_t u = 0; u < CHAIN_UNROLL; ++u) {
			const uint32_t kk = k + u < k_end ? k + u : k_end - 1;     // clamped: stays inside the ray
			v[u] = w.S[base + kk - win_lo];
		}
		#pragma unroll
		for (uint32_t u = 0; u < CHAIN_UNROLL; ++u) {
			if (stop || k >= k_end) break;
			if (T < A.K.thr) { stop = true; break; }
			const float alpha = v[u].x;
			const float weight = alpha * T;
			r += weight * v[u].y; g += weight * v[u].z; b += weight * v[u].w;
			w.S[base + k - win_lo] = mk4(T, r, g, b);
			T *= (1.f - alpha);
			w.owner[base + k - win_lo] = (uint8_t)lane;
			++k;
		}
	}
	c.T = T; c.Cr = r; c.Cg = g; c.Cb = b;
	c.k = k;
	c.done = stop ? 1u : 0u;
	rl.rnf[lane] = k;
}

// ---- finish: lane <-> ray (ray_marcher.cu:81-109, 128-133) -------------------------------
SRF_HD void finish_ray(uint32_t lane, uint32_t ray0, const Args& A, RayLds& rl, RayCarry& c, Float4 target_rgba, uint32_t lane_lo = 0, uint32_t lane_hi = RAYS) {
	const uint32_t i = ray0 + lane;
	if (i >= A.n_active || lane < lane_lo || lane >= lane_hi) { rl.rnf[lane] = 0; return; }
	float target[3], bg[3];
	target_and_background(A.K, target_rgba, target, bg);
	float r = c.Cr, g = c.Cg, b = c.Cb;
	if (c.k == c.numsteps) { r += c.T * bg[0]; g += c.T * bg[1]; b += c.T * bg[2]; }
	RayOut& o = rl.out[lane];
	o.c[0] = r; o.c[1] = g; o.c[2] = b;
	float lo[3];
	loss_channel(A.K.loss_type, target[0], r, &lo[0], &o.g[0]);
	loss_channel(A.K.loss_type, target[1], g, &lo[1], &o.g[1]);
	loss_channel(A.K.loss_type, target[2], b, &lo[2], &o.g[2]);
	rl.loss[lane] = (((lo[0] + lo[1]) + lo[2]) / 3.0f) / (float)A.K.n_rays;
	rl.rnf[lane] = c.k;
	if (A.rgb_ray_out) { A.rgb_ray_out[3 * (size_t)i] = r; A.rgb_ray_out[3 * (size_t)i + 1] = g; A.rgb_ray_out[3 * (size_t)i + 2] = b; }
}

// after the ordered offset of the ray is known (ray_marcher.cu:116-131)
// write_loss = false: the ray's loss is written later, by commit_loss (a kernel whose finish may still be running on another wave)
SRF_HD void commit_ray(uint32_t lane, uint32_t ray0, uint32_t cbase, const Args& A, RayLds& rl, const Plan& pl, uint32_t lane_lo = 0, uint32_t lane_hi = RAYS, bool write_loss = true) {
	const uint32_t i = ray0 + lane;
	RayOut& o = rl.out[lane];
	const uint32_t first = pl.rbase[lane];
	o.obase = cbase - first;
	if (i >= A.n_active || lane < lane_lo || lane >= lane_hi) { o.s_end = first; return; }
	uint32_t n = rl.rnf[lane];
	const uint32_t room = A.K.n_max_compacted - (A.K.n_max_compacted < cbase ? A.K.n_max_compacted : cbase);
	n = room < n ? room : n;
	o.s_end = first + n;
	A.ray_coord_indices[2 * (size_t)i] = n;
	A.ray_coord_indices[2 * (size_t)i + 1] = cbase;
	if (write_loss && n != 0 && A.loss_output) A.loss_output[i] = rl.loss[lane];
}

SRF_HD void commit_loss(uint32_t lane, uint32_t ray0, const Args& A, const RayLds& rl, const Plan& pl, uint32_t lane_lo = 0, uint32_t lane_hi = RAYS) {
	const uint32_t i = ray0 + lane;
	if (i >= A.n_active || lane < lane_lo || lane >= lane_hi) return;
	if (rl.out[lane].s_end != pl.rbase[lane] && A.loss_output) A.loss_output[i] = rl.loss[lane];
}

// ---- phase C: thread <-> sample (ray_marcher.cu:171-201) ---------------------------------
// COPY_COORDS = false: the kept samples' coordinates are moved elsewhere (coords_copy_single)
template <class G, bool HALF_IN, bool HALF_OUT, bool PLAIN = false, bool COPY_COORDS = true>
SRF_HD void phase_c(uint32_t tid, uint32_t win, const Args& A, const Window<G>& w, const RayLds& rl, const Plan& pl, SlotState<G, HALF_IN>& st) {
	const int rgb_act = PLAIN ? (int)SRF_ACT_NONE : A.K.rgb_act, density_act = PLAIN ? (int)SRF_ACT_NONE : A.K.density_act;
	const float l2_reg = rgb_act == SRF_ACT_EXPONENTIAL ? 1e-4f : 0.0f;
	const float l1_reg_density = (A.K.use_grid && (A.mean_density < A.K.min_optical_thickness)) ? 1e-4f : 0.0f;
	const uint32_t total = pl.misc[M_TOTAL];
	const uint32_t in_window = total - win * G::WIN < G::WIN ? total - win * G::WIN : G::WIN;
	const uint32_t n_slots = (in_window + G::THREADS - 1) / G::THREADS;
	#pragma unroll
	for (uint32_t j = 0; j < G::SLOTS; ++j) {
		if (G::FENCE_SLOTS) SRF_SLOT_FENCE();
		if (j >= n_slots) continue;
		const uint32_t q = tid + j * G::THREADS;
		if (win * G::WIN + q >= total) continue;
		const uint32_t r = w.owner[q];
		if (r >= RAYS) continue;
		const uint32_t srel = win * G::WIN + q;                  // position in the group
		const Float4 og = *(const Float4*)&rl.out[r].g[0];      // g.xyz, obase
		const Float4 oc = *(const Float4*)&rl.out[r].c[0];      // c.xyz, s_end
		if (srel >= srf_f2u(oc.w)) continue;
		const Float4 after = w.S[q];                             // T before the sample, colour sum including it
		const float T_before = after.x;
		float v[4];
		unpack_raw<HALF_IN>(st.raw[j], v);
		const float cr = act_rgb(v[0], rgb_act), cg = act_rgb(v[1], rgb_act), cb = act_rgb(v[2], rgb_act);
		const float weight = st.alpha[j] * T_before;
		const float T = T_before * (1.f - st.alpha[j]);          // the chain's own update (ray_marcher.cu:181)
		const float d0 = A.K.loss_scale * ((weight * og.x) * act_rgb_derivative(v[0], rgb_act) + srf_max_zero(l2_reg * v[0]));
		const float d1 = A.K.loss_scale * ((weight * og.y) * act_rgb_derivative(v[1], rgb_act) + srf_max_zero(l2_reg * v[1]));
		const float d2 = A.K.loss_scale * ((weight * og.z) * act_rgb_derivative(v[2], rgb_act) + srf_max_zero(l2_reg * v[2]));
		const float sx = oc.x - after.y, sy = oc.y - after.z, sz = oc.z - after.w;
		const float dd = act_density_derivative(v[3], density_act);
		const float dotv = (og.x * (T * cr - sx) + og.y * (T * cg - sy)) + og.z * (T * cb - sz);
		const float dmlp = dd * (st.dt[j] * dotv);
		const float d3 = A.K.loss_scale * dmlp + (v[3] < 0 ? -l1_reg_density : 0.0f);
		const size_t o = (size_t)(uint32_t)(srf_f2u(og.w) + srel);
		// One vector store per sample when the records are 4 wide (the reference's padded_output_width).  The general
		// case goes through volatile pointers only to keep the compiler from folding both cases into scalar stores.
		if (HALF_OUT) {
			const uint32_t lo = (uint32_t)float_to_half_bits(d0) | ((uint32_t)float_to_half_bits(d1) << 16);
			const uint32_t hi = (uint32_t)float_to_half_bits(d2) | ((uint32_t)float_to_half_bits(d3) << 16);
			if (A.K.out_width == 4) {
				U2 v; v.x = lo; v.y = hi;
				*((U2*)A.dloss + o) = v;
			} else {
				volatile uint16_t* p = (volatile uint16_t*)A.dloss + o * A.K.out_width;
				p[0] = (uint16_t)(lo & 0xffffu); p[1] = (uint16_t)(lo >> 16); p[2] = (uint16_t)(hi & 0xffffu); p[3] = (uint16_t)(hi >> 16);
			}
		} else if (A.K.out_width == 4) {
			*((Float4*)A.dloss + o) = mk4(d0, d1, d2, d3);
		} else {
			volatile float* p = (volatile float*)A.dloss + o * A.K.out_width;
			p[0] = d0; p[1] = d1; p[2] = d2; p[3] = d3;
		}
		if (COPY_COORDS && A.compacted_coords) {
			const size_t s = (size_t)pl.misc[M_S0] + (size_t)win * G::WIN + q;
			float cc[7];
			for (int c = 0; c < 7; ++c) cc[c] = A.coords[7 * s + c];
			for (int c = 0; c < 7; ++c) A.compacted_coords[7 * o + c] = cc[c];
		}
	}
}

// ---- coordinates of the kept samples of a one-window plan: lane <-> sample (ray_marcher.cu:196-199) ----
// By the 64 lanes of one wave, COORDS_DEPTH rows of 64 samples at a time so that several rows' loads are under way together.
constexpr uint32_t COORDS_DEPTH = 8;
template <class G>
SRF_HD void coords_copy_rows(uint32_t lane, uint32_t q0, const Args& A, const Window<G>& w, const RayLds& rl, const Plan& pl) {
	const uint32_t total = pl.misc[M_TOTAL];
	const float* src = A.coords + 7 * (size_t)pl.misc[M_S0];
	float cc[COORDS_DEPTH][7];
	size_t o[COORDS_DEPTH];
	bool ok[COORDS_DEPTH];
	#pragma unroll
	for (uint32_t u = 0; u < COORDS_DEPTH; ++u) {
		const uint32_t q = q0 + u * RAYS + lane;
		ok[u] = false; o[u] = 0;
		if (q < total) {
			const uint32_t r = w.owner[q];
			if (r < RAYS) {
				if (q < rl.out[r].s_end) {
					ok[u] = true;
					o[u] = (size_t)(uint32_t)(rl.out[r].obase + q);
					for (int c = 0; c < 7; ++c) cc[u][c] = src[7 * q + c];
				}
			}
		}
	}
	#pragma unroll
	for (uint32_t u = 0; u < COORDS_DEPTH; ++u) {
		if (ok[u]) for (int c = 0; c < 7; ++c) A.compacted_coords[7 * o[u] + c] = cc[u][c];
	}
}
template <class G>
SRF_HD void coords_copy_single(uint32_t lane, const Args& A, const Window<G>& w, const RayLds& rl, const Plan& pl) {
	if (!A.compacted_coords) return;
	const uint32_t total = SRF_UNIFORM_U32(pl.misc[M_TOTAL]);
	for (uint32_t q0 = 0; q0 < total; q0 += COORDS_DEPTH * RAYS) coords_copy_rows<G>(lane, q0, A, w, rl, pl);
}

} // namespace fused
} // namespace srf
