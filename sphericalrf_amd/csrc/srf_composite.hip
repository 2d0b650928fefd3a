// RayMarcher: front-to-back alpha compositing with loss and gradients (training),
// chunked compositing (rendering), and the orchestrator's small kernels
// (ordered ray compaction, shading, batch roll-over).
#include "srf_internal.h"
#include <mutex>
#include "srf_bodies.h"
#include "srf_composite_fused.h"
#include "srf_chain.h"
#include <stdlib.h>

namespace srf {

template <bool HALF_IN>
__global__ void __launch_bounds__(128) k_loss_forward(LossConst K, const float* __restrict__ rays_rgba, const uint32_t* __restrict__ n_rays_counter,
                                                      const uint32_t* __restrict__ ray_coord_indices, const float* __restrict__ dt_arr,
                                                      const void* __restrict__ net, FwdRay* __restrict__ fwd, uint32_t* __restrict__ n_out,
                                                      float* __restrict__ rgb_ray_out) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < K.n_rays) loss_forward_body<HALF_IN>(i, K, rays_rgba, *n_rays_counter, ray_coord_indices, dt_arr, net, fwd + i, n_out + i, rgb_ray_out);
}

template <bool HALF_IN, bool HALF_OUT>
__global__ void __launch_bounds__(128) k_loss_backward(LossConst K, const uint32_t* __restrict__ n_rays_counter, uint32_t* __restrict__ ray_coord_indices,
                                                       const float* __restrict__ dt_arr, const float* __restrict__ coords, float* __restrict__ compacted_coords,
                                                       const void* __restrict__ net, void* __restrict__ dloss, float* __restrict__ loss_output,
                                                       const float* __restrict__ mean_density_ptr, const FwdRay* __restrict__ fwd,
                                                       const uint32_t* __restrict__ n_fwd, const uint32_t* __restrict__ cbase_arr,
                                                       float* __restrict__ reg_buffer) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < K.n_rays) loss_backward_body<HALF_IN, HALF_OUT>(i, K, *n_rays_counter, ray_coord_indices, dt_arr, coords, compacted_coords, net, dloss, loss_output,
	                                                        mean_density_ptr ? *mean_density_ptr : 0.f, fwd[i], n_fwd[i], cbase_arr[i], reg_buffer);
}

// round: the frame loop's words on the device, in place of the three numbers of A that change from round to round (or NULL)
template <bool HALF_IN>
__global__ void __launch_bounds__(128) k_volume_rendering(Params P, srf_render_args A, float thr, srf_ray_payload* __restrict__ payloads,
                                                          float* __restrict__ rgba, const float* __restrict__ coords, const void* __restrict__ net,
                                                          const RoundWords* __restrict__ round) {
	if (round) { A.n_rays = round->n_alive; A.n_steps = round->n_steps; A.i_steps_offset = round->offset; }
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < A.n_rays) volume_rendering_body<HALF_IN>(i, P, A, thr, payloads, rgba, coords, net);
}

// ------------------------------------------------------------------------------------
// Single-launch compositing (phases in srf_composite_fused.h)
// ------------------------------------------------------------------------------------
// bytes of device scratch the chain needs for n_rays rays whose groups are cut into at most max_parts items each, and where
// its parts lie (save_records: with room for a copy of the listed groups' ray records, see k_slow_groups)
struct ChainLayout { size_t off_seg, off_prefix, off_misc, off_words, off_cuts, off_sums, off_items, off_list, off_side, off_saved, bytes; };
SRF_HD constexpr ChainLayout chain_layout(uint32_t n_rays, uint32_t max_parts, bool save_records) {
	const size_t n_groups = ((size_t)n_rays + fused::RAYS - 1) / fused::RAYS;
	const size_t n_items = (size_t)max_parts * n_groups;
	ChainLayout L = {};
	L.off_seg = (n_items * 8 + 255) / 256 * 256;
	L.off_prefix = (L.off_seg + (n_items + 63) / 64 * 8 * SEG_STRIDE + 255) / 256 * 256;
	L.off_misc = (L.off_prefix + (n_items + 63) / 64 * 8 + 255) / 256 * 256;
	L.off_words = L.off_misc + 512;
	L.off_cuts = (L.off_words + n_groups * 4 + 255) / 256 * 256;
	L.off_sums = (L.off_cuts + n_groups * 8 + 255) / 256 * 256;
	L.off_items = (L.off_sums + (n_groups / PREPARE_WAVES + 1) * 4 + 255) / 256 * 256;
	L.off_list = (L.off_items + n_items * 8 + 255) / 256 * 256;
	L.off_side = (L.off_list + n_groups * 4 + 255) / 256 * 256;
	L.off_saved = (L.off_side + n_groups * fused::RAYS * 4 + 255) / 256 * 256;
	L.bytes = L.off_saved + (save_records ? n_groups * fused::RAYS * 8 : 0);
	return L;
}
static ChainScratch chain_scratch_at(void* base, uint32_t n_rays, uint32_t max_parts, bool save_records, uint32_t* host_error, uint32_t spin_limit) {
	const ChainLayout L = chain_layout(n_rays, max_parts, save_records);
	ChainScratch S;
	S.item_status = (unsigned long long*)base;
	S.seg_status = (unsigned long long*)((char*)base + L.off_seg);
	S.seg_prefix = (unsigned long long*)((char*)base + L.off_prefix);
	S.initial = (uint32_t*)((char*)base + L.off_misc);
	S.error = S.initial + 1;
	S.slow_count = S.initial + 2;
	S.n_items = S.initial + 3;
	S.group_words = (uint32_t*)((char*)base + L.off_words);
	S.group_cuts = (unsigned long long*)((char*)base + L.off_cuts);
	S.prepare_sums = (uint32_t*)((char*)base + L.off_sums);
	S.items = (U2*)((char*)base + L.off_items);
	S.slow_items = (uint32_t*)((char*)base + L.off_list);
	S.side = (uint32_t*)((char*)base + L.off_side);
	S.saved_records = save_records ? (U2*)((char*)base + L.off_saved) : nullptr;
	S.host_error = host_error;
	S.spin_limit = spin_limit;
	S.max_parts = max_parts;
	return S;
}
// Items a group may be cut into: any number where the scratch is allocated to fit; the scratch that is part of the library's
// image (see g_noalloc_scratch) has room for eight, and groups that need more take the path of the listed ones there.
constexpr uint32_t STREAM_MAX_PARTS = fused::MAX_PARTS;
constexpr uint32_t NOALLOC_MAX_PARTS = 8;

// Ordering point between the phases of a group (see srf_composite_fused.h): a workgroup barrier.
__device__ __forceinline__ void group_sync() { __syncthreads(); }

// ---- groups that do not fit the streaming path ------------------------------------------------
// The streaming kernel takes groups whose rays are laid out back to back and whose samples fit one of its windows.  The
// others (arbitrary caller-supplied offsets; more samples than one window) are rare and are kept out of its code:
//   k_chain_prepare      plans every group and notes how many items it makes
//   k_chain_items        numbers the items in ray order, clears their words of the chain and lists those of groups that the streaming path does not take
//   k_slow_groups (fwd)  forward pass of the listed groups; leaves the number of samples every one of their rays consumes
//   k_composite_stream   for a listed group only chains those counts to its neighbours' and leaves the rays' compacted offsets
//   k_slow_groups (bwd)  forward pass again, then commit and gradients at those offsets
// Rays not laid out back to back are composited one lane per ray; groups with a ray longer than a window run the window
// phases over all windows.

// Records of one group into a plan, by the 64 lanes of one wave: what fused::plan_lane and fused::plan_finish_lane
// compute lane by lane through LDS, with the wave's own reductions instead (64 lanes adding to one LDS word take turns).
// The streaming kernel plans an item of a cut group while the items before it may already have committed, which overwrites
// their rays' records (count and offset after compaction).  Offsets relative to the group's first sample are therefore kept
// modulo 2^32: in plan_part_lane the first ray's offset cancels, so a part's plan depends on the records of its own rays and
// of the ray after them only, and that ray's item commits after this one has been planned (it waits for this one's count).
// Whether the rays lie back to back is decided once, before anything is overwritten (k_chain_prepare), and travels with the item.
__device__ __forceinline__ void plan_from_records(uint32_t lane, uint32_t g, U2 rec, const fused::Args& A, fused::Plan& pl) {
	using namespace fused;
	const uint32_t ray0 = g * RAYS;
	const uint32_t n_here = A.n_active > ray0 ? (A.n_active - ray0 < RAYS ? A.n_active - ray0 : RAYS) : 0;
	const uint32_t rn = rec.x, rabs = rec.y;             // (0, 0) past the active count
	const uint32_t s0 = n_here ? lane_value_u32(rabs, 0) : 0u;
	const uint32_t prev_rabs = lane_below_u32(rabs), prev_rn = lane_below_u32(rn);
	const uint64_t prev_end = lane ? (uint64_t)prev_rabs + prev_rn : (uint64_t)s0;
	const bool mine = lane < n_here;
	const bool out_of_order = mine && (uint64_t)rabs < prev_end;
	const uint32_t sum = wave_sum_fast(mine ? rn : 0u);
	const uint32_t last = n_here ? n_here - 1 : 0u;
	const uint64_t end = n_here ? (uint64_t)lane_value_u32(rabs, last) + lane_value_u32(rn, last) : 0ull;
	const uint32_t total = (uint32_t)end - s0;
	const bool fits = end >= s0 && end - s0 <= 0xffffffffull;
	const bool contiguous = __ballot(out_of_order) == 0ull && fits && !((uint64_t)total > (uint64_t)sum + GAP_SLACK);
	pl.rn[lane] = rn;
	pl.rabs[lane] = rabs;
	pl.rbase[lane] = mine ? rabs - s0 : total;
	if (lane == 0) {
		pl.rbase[RAYS] = total;
		pl.misc[M_S0] = s0; pl.misc[M_TOTAL] = total; pl.misc[M_SUM] = sum; pl.misc[M_CONTIG] = contiguous ? 1u : 0u;
		pl.misc[M_LANE_LO] = 0; pl.misc[M_LANE_HI] = RAYS; pl.misc[M_GROUP] = g;
	}
	__builtin_amdgcn_wave_barrier();
}

__device__ __forceinline__ U2 load_record(uint32_t g, uint32_t lane, const fused::Args& A) {
	U2 rec; rec.x = 0; rec.y = 0;
	const uint32_t i = g * fused::RAYS + lane;
	if (i < A.n_active) rec = *(const U2*)(A.ray_coord_indices + 2 * (size_t)i);
	return rec;
}

// fused::plan_cuts by the 64 lanes of the wave that wrote the plan: lane r holds where ray r begins and ends, one ballot finds
// the first ray that does not fit with the rays from `lo` on (the ends only grow), so a group costs one round per item.
__device__ __forceinline__ uint64_t plan_cuts_wave(uint32_t lane, const fused::Plan& pl, uint32_t win, uint32_t max_parts) {
	using namespace fused;
	if (pl.misc[M_CONTIG] == 0) return 0ull;
	if (pl.misc[M_TOTAL] <= win) return 1ull;
	const uint32_t start = pl.rbase[lane], end = pl.rbase[lane + 1];      // rbase[RAYS]: the group's end
	uint64_t cuts = 1ull;
	uint32_t parts = 1, lo = 0;
	for (;;) {
		const uint32_t lo_base = lane_value_u32(start, lo);
		const uint64_t beyond = __ballot(end - lo_base > win) & ~((1ull << lo) - 1ull);
		if (beyond == 0ull) return cuts;
		const uint32_t r = (uint32_t)__builtin_ctzll(beyond);
		if (r == lo) return 0ull;                      // ray lo alone does not fit
		lo = r;
		cuts |= 1ull << lo;
		if (++parts > max_parts) return 0ull;
	}
}

// One wave per group, PREPARE_WAVES groups per workgroup; a workgroup also leaves the number of items its groups make.
__global__ void __launch_bounds__(PREPARE_WAVES * WAVE) k_chain_prepare(fused::Args A, const uint32_t* __restrict__ n_rays_counter, ChainScratch S,
                                                                       const uint32_t* __restrict__ counter) {
	using namespace fused;
	__shared__ Plan plans[PREPARE_WAVES];
	__shared__ uint32_t n_items_of_wave[PREPARE_WAVES];
	const uint32_t wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
	const uint32_t g = blockIdx.x * PREPARE_WAVES + wave;
	if (blockIdx.x == 0 && threadIdx.x == 0) { *S.initial = *counter; *S.error = 0u; *S.slow_count = 0u; }
	const uint32_t counter_now = *n_rays_counter;
	A.n_active = counter_now < A.K.n_rays ? counter_now : A.K.n_rays;
	uint32_t word = 0;
	if (g < div_up(A.n_active, RAYS)) {
		Plan& pl = plans[wave];
		plan_from_records(lane, g, load_record(g, lane, A), A, pl);
		const uint64_t cuts = plan_cuts_wave(lane, pl, StreamGeometry::WIN, S.max_parts);
		word = group_items_word(cuts);
		if (lane == 0) {
			S.group_words[g] = word;
			if ((word & 0xffu) > 1u) S.group_cuts[g] = cuts;
		}
	}
	if (lane == 0) n_items_of_wave[wave] = word & 0xffu;
	__syncthreads();
	if (threadIdx.x == 0) {
		uint32_t n = 0;
		for (uint32_t k = 0; k < PREPARE_WAVES; ++k) n += n_items_of_wave[k];
		S.prepare_sums[blockIdx.x] = n;
	}
}

// Numbers the items: an exclusive scan of the groups' item counts.  A workgroup takes ITEMS_THREADS consecutive groups (one
// per thread); what lies before them it adds up from the sums that k_chain_prepare's workgroups left.
constexpr uint32_t ITEMS_THREADS = 1024;
static_assert(ITEMS_THREADS % PREPARE_WAVES == 0, "an items workgroup starts where a prepare workgroup starts");
__global__ void __launch_bounds__(ITEMS_THREADS) k_chain_items(uint32_t n_rays_max, const uint32_t* __restrict__ n_rays_counter, ChainScratch S) {
	using namespace fused;
	__shared__ uint32_t wave_total[ITEMS_THREADS / WAVE], wave_before[ITEMS_THREADS / WAVE];
	const uint32_t tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
	const uint32_t counter_now = *n_rays_counter;
	const uint32_t n_groups = div_up(counter_now < n_rays_max ? counter_now : n_rays_max, RAYS);
	const uint32_t g_first = blockIdx.x * ITEMS_THREADS;
	if (g_first >= n_groups && !(n_groups == 0 && blockIdx.x == 0)) return;
	const uint32_t g = g_first + tid;
	const uint32_t word = g < n_groups ? S.group_words[g] : 0u;
	uint32_t before = 0;
	for (uint32_t k = tid; k < g_first / PREPARE_WAVES; k += ITEMS_THREADS) before += S.prepare_sums[k];
	const uint32_t n = word & 0xffu;
	const uint32_t incl = wave_inclusive_scan_fast(n);
	const uint32_t before_w = wave_sum_fast(before);
	if (lane == WAVE - 1) { wave_total[wave] = incl; wave_before[wave] = before_w; }
	__syncthreads();
	uint32_t base = 0, all = 0;
	for (uint32_t k = 0; k < ITEMS_THREADS / WAVE; ++k) { const uint32_t t = wave_total[k]; base += wave_before[k] + (k < wave ? t : 0u); all += wave_before[k] + t; }
	if (n != 0) {
		const uint32_t first = base + incl - n;
		items_of_group(g, word, n > 1u ? S.group_cuts[g] : 1ull, S.items + first);
		if ((word & (1u << 16)) != 0u) S.slow_items[atomicAdd(S.slow_count, 1u)] = first;
		// the chain's words of these items, and of the segments of 64 items that begin with one of them
		for (uint32_t i = first; i < first + n; ++i) {
			S.item_status[i] = 0ull;
			if (i % WAVE == 0) { S.seg_status[(size_t)(i / WAVE) * SEG_STRIDE] = 0ull; S.seg_prefix[i / WAVE] = 0ull; }
		}
	}
	if (tid == 0 && g_first + ITEMS_THREADS >= n_groups) *S.n_items = all;     // the workgroup with the last group
}

struct SlowShared {
	fused::Window<fused::WideGeometry> w;
	fused::RayLds rl;
	fused::Plan plan;       // the group
	fused::Plan part;       // the rays of it that are under way
};

// Where a listed group whose rays lie back to back is cut into parts: like plan_cuts_wave, but a ray longer than a window
// is a part of its own.  A part's rays go through the windows together and one after another part's, so that a group of long
// rays does not walk them one behind the other; the parts of a group are dealt to `slots` units of work, which different
// workgroups take.
__device__ __forceinline__ uint64_t slow_cuts_wave(uint32_t lane, const fused::Plan& pl, uint32_t win) {
	using namespace fused;
	const uint32_t start = pl.rbase[lane], end = pl.rbase[lane + 1];
	uint64_t cuts = 1ull;
	uint32_t lo = 0;
	for (;;) {
		const uint32_t lo_base = lane_value_u32(start, lo);
		const uint64_t beyond = __ballot(end - lo_base > win) & ~((1ull << lo) - 1ull);
		if (beyond == 0ull) return cuts;
		uint32_t r = (uint32_t)__builtin_ctzll(beyond);
		if (r == lo) ++r;                              // ray lo alone is longer than a window
		if (r >= RAYS) return cuts;
		lo = r;
		cuts |= 1ull << lo;
	}
}

constexpr uint32_t SLOW_PART_SLOTS = 16;      // workgroups that share a listed group (see k_slow_groups)
constexpr uint32_t SLOW_WORKGROUPS = 2048;

template <bool HALF_IN, bool HALF_OUT, bool BACKWARD>
__global__ void __launch_bounds__(fused::WideGeometry::THREADS) k_slow_groups(fused::Args A, const uint32_t* __restrict__ n_rays_counter, const float* __restrict__ mean_density_ptr, ChainScratch S, uint32_t slots) {
	using namespace fused;
	using G = WideGeometry;
	__shared__ SlowShared sh;
	const uint32_t tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
	const uint32_t n_listed = *S.slow_count;
	// a unit of work: the parts of one listed group whose number is `slot` modulo `slots`
	const uint64_t n_units = (uint64_t)n_listed * slots;
	if (blockIdx.x >= n_units) return;
	const uint32_t counter_now = *n_rays_counter;
	A.mean_density = mean_density_ptr ? *mean_density_ptr : 0.f;
	A.n_active = counter_now < A.K.n_rays ? counter_now : A.K.n_rays;
	if (!BACKWARD) A.rgb_ray_out = nullptr;      // written once, by the second forward pass
	for (uint64_t unit = blockIdx.x; unit < n_units; unit += gridDim.x) {
		const uint32_t k = (uint32_t)(unit / slots), slot = (uint32_t)(unit % slots);
		const uint32_t g = S.items[S.slow_items[k]].x;
		const uint32_t ray0 = g * RAYS;
		if (wave == 0) {
			// The commit of the backward launch overwrites a ray's record, and the workgroups that share a group do not wait for
			// one another: they plan from the copy that the forward launch left.
			U2 rec;
			if (BACKWARD && S.saved_records) rec = S.saved_records[(size_t)ray0 + lane];
			else {
				rec = load_record(g, lane, A);
				if (S.saved_records && slot == 0) S.saved_records[(size_t)ray0 + lane] = rec;
			}
			plan_from_records(lane, g, rec, A, sh.plan);
		}
		group_sync();
		if (sh.plan.misc[M_CONTIG] != 0) {
			uint64_t cuts = slow_cuts_wave(lane, sh.plan, G::WIN);      // (the same in every wave)
			for (uint32_t part_number = 0; cuts != 0ull; ++part_number) {
				const uint32_t lo = (uint32_t)__builtin_ctzll(cuts);
				cuts &= cuts - 1ull;
				const uint32_t hi = cuts ? (uint32_t)__builtin_ctzll(cuts) : RAYS;
				if (part_number % slots != slot) continue;
				const Plan& pl = sh.part;
				if (wave == 0) plan_part_lane(lane, sh.plan, lo, hi, g, sh.part);
				group_sync();
				const bool live = wave == 0 && ray0 + lane < A.n_active && lane >= lo && lane < hi;
				const uint32_t n_win = (pl.misc[M_TOTAL] + G::WIN - 1) / G::WIN;
				SlotState<G, HALF_IN> st;
				RayCarry c;
				Float4 target = mk4(0.f, 0.f, 0.f, 0.f);
				if (live) target = *(const Float4*)(A.rays_rgba + 4 * (size_t)(ray0 + lane));
				if (wave == 0) reset_carry(lane, pl, c);
				for (uint32_t win = 0; win < n_win; ++win) {
					phase_a<G, HALF_IN>(tid, win, A, sh.w, pl, st);
					group_sync();
					if (wave == 0) chain<G>(lane, win, A, sh.w, sh.rl, pl, c);
					group_sync();
				}
				if (wave == 0) finish_ray(lane, ray0, A, sh.rl, c, target, lo, hi);
				if (!BACKWARD) {
					if (live) S.side[ray0 + lane] = sh.rl.rnf[lane];
				} else {
					if (wave == 0) commit_ray(lane, ray0, live ? S.side[ray0 + lane] : 0u, A, sh.rl, pl, lo, hi);
					group_sync();
					if (wave == 0) reset_carry(lane, pl, c);
					for (uint32_t win = 0; win < n_win; ++win) {
						phase_a<G, HALF_IN>(tid, win, A, sh.w, pl, st);
						group_sync();
						if (wave == 0) chain<G>(lane, win, A, sh.w, sh.rl, pl, c);
						group_sync();
						phase_c<G, HALF_IN, HALF_OUT>(tid, win, A, sh.w, sh.rl, pl, st);
						group_sync();
					}
				}
				group_sync();
			}
		} else if (wave == 0 && slot == 0) {
			const bool live = ray0 + lane < A.n_active;
			uint32_t n = 0;
			FwdRay fw;
			loss_forward_body<HALF_IN>(ray0 + lane, A.K, A.rays_rgba, A.n_active, A.ray_coord_indices, A.dt_arr, A.net, &fw, &n, A.rgb_ray_out);
			if (!BACKWARD) {
				if (live) S.side[ray0 + lane] = n;
			} else if (live) {
				loss_backward_body<HALF_IN, HALF_OUT>(ray0 + lane, A.K, A.n_active, A.ray_coord_indices, A.dt_arr, A.coords, A.compacted_coords, A.net, A.dloss, A.loss_output,
				                                      A.mean_density, fw, n, S.side[ray0 + lane], nullptr);
			}
		}
		group_sync();
	}
}

// ---- the streaming kernel ---------------------------------------------------------------------
// Workgroups are persistent: workgroup b works on items b, b + gridDim.x, b + 2 gridDim.x, ...  (Handing the items out
// in the order in which workgroups become free would need a counter that every item increments, and the device serialises
// those increments at a rate below the rate of items; consecutive items on one workgroup would make each workgroup wait
// for its neighbour's last item.)  A workgroup's first wave walks
// rays (one lane per ray: count, chain, finish, ordered offsets), its second wave plans, its other waves work on samples
// (phases A and C), and three items are under way at any time, in two LDS windows:
//
//                 first half of iteration j                      second half of iteration j
//   ray wave      look-back and commit of item j                 count of item j + 1 (its total is published), then its chain
//   plan wave     finish of item j (colours, loss, its gradient) plan of item j + 3; records further ahead requested; losses of
//                                                                item j written; coordinates of item j's kept samples moved
//   sample waves  phase A of item j + 1 (other window)           samples of item j + 2 requested; phase C of item j
//
// so every load has at least half an iteration to arrive before it is used, and an item's total is published a chain and
// a barrier before its own look-back needs its predecessors' totals: a workgroup has to fall that far behind the others
// before they wait for it.  The ray wave is the one sequential stream of a workgroup, so it runs at raised
// priority.  An item waits for every lower-numbered item's total.  Lower-numbered items belong to workgroups that are
// resident at the same time (the grid is sized to what the device holds at once); waits are bounded all the same.
// Two workgroups per CU (two windows take most of their 80 KB of LDS each).
#define SRF_STREAM_OCCUPANCY __attribute__((amdgpu_waves_per_eu(4, 4)))
constexpr uint32_t STREAM_WORKGROUPS_PER_CU = 2;
// Eight waves per workgroup: the hardware deals a workgroup's waves round the four SIMDs, so two such workgroups fill every
// SIMD evenly (a workgroup of, say, six waves may not find room next to another although the totals fit, and the items of a
// workgroup that is not resident are waited for in vain).
constexpr uint32_t STREAM_THREADS = 2 * WAVE + fused::StreamGeometry::THREADS;
static_assert(STREAM_THREADS == 8 * WAVE, "workgroup shape");

struct StreamShared {
	fused::Window<fused::StreamGeometry> win[2];
	fused::RayLds rl;
	fused::Plan plan[fused::NPLAN];     // ring: the plans of the three items under way and of the one after them
	fused::Plan group_plan;             // plan wave: the group whose rays the item being planned belongs to
};

// Build flag SRF_KERNEL_TIMING: lane 0 of the ray wave and of the first sample wave add up the cycles they spend in
// the parts of an iteration, into counters after the chain's misc words.
#ifdef SRF_KERNEL_TIMING
#define SRF_T(k) do { if (lane == 0 && wave <= 2) { const unsigned long long now_ = clock64(); t_acc_[k] += now_ - t_prev_; t_prev_ = now_; } } while (0)
#else
#define SRF_T(k) ((void)0)
#endif

template <bool HALF_IN, bool HALF_OUT, bool PLAIN>
__global__ void __launch_bounds__(STREAM_THREADS) SRF_STREAM_OCCUPANCY k_composite_stream(fused::Args A, const uint32_t* __restrict__ n_rays_counter, const float* __restrict__ mean_density_ptr,
                                                                     ChainScratch S, uint32_t* __restrict__ compacted_counter) {
	using namespace fused;
	using G = StreamGeometry;
	static_assert(RAYS == WAVE, "one lane per ray");
	static_assert(NPLAN == 4, "three items under way, one being planned");
	__shared__ StreamShared sh;
	const uint32_t tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
	const uint32_t st_id = tid - 2 * WAVE;                   // index among the sample threads (waves 2-7)
	const bool ray_wave = wave == 0, plan_wave = wave == 1;
	const uint32_t counter_now = *n_rays_counter;
	A.mean_density = mean_density_ptr ? *mean_density_ptr : 0.f;
	A.n_active = counter_now < A.K.n_rays ? counter_now : A.K.n_rays;   // rays past the active count belong to no item: they are left untouched
	const uint32_t n_items = SRF_UNIFORM_U32(*S.n_items);
	if (blockIdx.x >= n_items) return;
	const uint32_t initial = SRF_UNIFORM_U32(*S.initial);     // (in a scalar register: looked at in the loop, it is not waited for again there)

#ifdef SRF_KERNEL_TIMING
	unsigned long long t_acc_[12] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
	unsigned long long t_prev_ = clock64();
	unsigned long long n_it_ = 0;
	bool t_on_ = false;
#endif
	SlotState<G, HALF_IN> set_c, set_a, set_l;     // samples of the item in phase C / in phase A / being loaded
	// ray wave, about the item it commits in the next first half
	uint32_t n_cur = 0, incl_cur = 0;               // count of its ray, scanned over the wave
	uint32_t total_cur = 0;                         // samples it keeps
	ChainPeek peek;
	peek.vg = 0ull; peek.vs = 0ull; peek.vp = 0ull; peek.initial = 0u;
	RayCarry carry;
	carry.T = 1.f; carry.Cr = 0.f; carry.Cg = 0.f; carry.Cb = 0.f; carry.k = 0; carry.numsteps = 0; carry.done = 0;
	// plan wave: the numbers of the workgroup's items, in the order it takes them ...
	uint32_t handed = 0;
	auto next_number = [&]() -> uint32_t {
		const uint64_t i = (uint64_t)blockIdx.x + (uint64_t)handed * gridDim.x;
		if (i >= n_items) return NO_ITEM;
		++handed;
		return (uint32_t)i;
	};
	// ... the item it plans next (number, record, its group's ray records: requested an iteration earlier) and the item after that,
	// and the target colours of the rays it finishes next
	Float4 target = mk4(0.f, 0.f, 0.f, 0.f);
	uint32_t number_p = NO_ITEM, number_q = NO_ITEM;
	U2 item_p, item_q, rec_p;
	item_p.x = 0; item_p.y = 0; item_q = item_p; rec_p = item_p;
	auto load_item = [&](uint32_t number) { U2 item; item.x = 0; item.y = 0; if (number != NO_ITEM) item = S.items[number]; return item; };
	auto plan_next = [&](Plan& out) {                // turns item_p into a plan and moves the requests one item on
		const U2 item = item_p, rec = rec_p;
		const uint32_t number = number_p;
		if (number != NO_ITEM) {
			const uint32_t g = item.x;
#ifdef SRF_KERNEL_TIMING
			{ U2 r_ = rec; asm volatile("" : "+v"(r_.x), "+v"(r_.y)); if (lane == 0 && wave == 1 && t_on_) { const unsigned long long now_ = clock64(); t_acc_[5] += now_ - t_prev_; t_prev_ = now_; } }
#endif
			plan_from_records(lane, g, rec, A, sh.group_plan);
#ifdef SRF_KERNEL_TIMING
			if (lane == 0 && wave == 1 && t_on_) { const unsigned long long now_ = clock64(); t_acc_[6] += now_ - t_prev_; t_prev_ = now_; }
#endif
			plan_part_lane(lane, sh.group_plan, item_lo(item), item_hi(item), g, out);
#ifdef SRF_KERNEL_TIMING
			if (lane == 0 && wave == 1 && t_on_) { const unsigned long long now_ = clock64(); t_acc_[7] += now_ - t_prev_; t_prev_ = now_; }
#endif
		}
		if (lane == 0) {
			out.misc[M_ITEM] = number;
			if (number != NO_ITEM && item_listed(item)) out.misc[M_CONTIG] = 0;     // only its offsets pass through here
		}
		item_p = item_q; number_p = number_q;
		rec_p = load_record(item_p.x, lane, A);     // (no item: group 0's, unused)
		number_q = next_number();
		item_q = load_item(number_q);
	};
	if (plan_wave) {
		number_p = next_number(); item_p = load_item(number_p);
		number_q = next_number(); item_q = load_item(number_q);
		rec_p = load_record(item_p.x, lane, A);
		plan_next(sh.plan[0]);
	}
	group_sync();
	if (ray_wave) __builtin_amdgcn_s_setprio(3);

	// the workgroup's item `it` is finished and gets its phase C in iteration `it`; its items it + 1 and it + 2 are under way behind it
	for (int it = -2;; ++it) {
		const Plan& pl = sh.plan[(uint32_t)(it + 4) % NPLAN];
		const Plan& pl1 = sh.plan[(uint32_t)(it + 5) % NPLAN];
		const Plan& pl2 = sh.plan[(uint32_t)(it + 6) % NPLAN];
		Plan& pl3 = sh.plan[(uint32_t)(it + 7) % NPLAN];
		Window<G>& w = sh.win[(uint32_t)(it + 4) % 2];
		Window<G>& w1 = sh.win[(uint32_t)(it + 5) % 2];
		// numbers of the items (plans of items it and it + 1 were written an iteration or more ago)
		const uint32_t i_0 = it >= 0 ? SRF_UNIFORM_U32(pl.misc[M_ITEM]) : NO_ITEM, i_1 = it + 1 >= 0 ? SRF_UNIFORM_U32(pl1.misc[M_ITEM]) : NO_ITEM;
		const bool has0 = i_0 != NO_ITEM, has1 = i_1 != NO_ITEM;
		const bool fast = has0 && pl.misc[M_CONTIG] != 0;
		const bool fast1 = has1 && pl1.misc[M_CONTIG] != 0;
		const uint32_t ray0 = has0 ? pl.misc[M_GROUP] * RAYS : 0u, lo = has0 ? pl.misc[M_LANE_LO] : 0u, hi = has0 ? pl.misc[M_LANE_HI] : 0u;
#ifdef SRF_KERNEL_TIMING
		if (lane == 0 && wave <= 2) { ++n_it_; t_prev_ = clock64(); t_on_ = true; }
#endif
		// ---- first half
		if (ray_wave) {
			// The counter that covers memory operations cannot tell loads from stores, which complete in no fixed order, so once a
			// store is under way every wait for a load becomes a wait for everything.  The status words requested in the previous
			// second half are therefore waited for here, before this half's first store, while everything under way is old.
			if (has0) asm volatile("" : "+v"(peek.vg), "+v"(peek.vs), "+v"(peek.vp), "+v"(peek.initial));
			if (has0) {
				const uint32_t prefix = chain_resolve(S, i_0, total_cur, peek);
				SRF_T(6);
				const uint32_t cbase = prefix == CHAIN_FAILED ? CHAIN_FAILED : prefix + incl_cur - n_cur;
				if (fast) commit_ray(lane, ray0, cbase, A, sh.rl, pl, lo, hi, false);
				else if (ray0 + lane < A.n_active) S.side[ray0 + lane] = cbase;
				if (i_0 == n_items - 1 && lane == 0) *compacted_counter = prefix == CHAIN_FAILED ? CHAIN_FAILED : prefix + total_cur;
			}
		} else if (plan_wave) {
			if (fast) {
				carry_from_lds(lane, sh.rl, pl, carry);
				finish_ray(lane, ray0, A, sh.rl, carry, target, lo, hi);
			}
		} else {
#ifdef SRF_KERNEL_TIMING
			asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
			SRF_T(4);
#endif
			if (fast1) phase_a_compute<G, HALF_IN, PLAIN>(st_id, 0, A, w1, pl1, set_a);
			SRF_T(5);
		}
		SRF_T(0);
		group_sync();
		SRF_T(1);
		const bool has2 = SRF_UNIFORM_U32(pl2.misc[M_ITEM]) != NO_ITEM;      // written in the previous second half (or before the loop)
		// ---- second half
		if (ray_wave) {
			if (has1) {
				const uint32_t ray1 = pl1.misc[M_GROUP] * RAYS, lo1 = pl1.misc[M_LANE_LO], hi1 = pl1.misc[M_LANE_HI];
				if (fast1) n_cur = count_lane<G>(lane, wave_max_fast(pl1.rn[lane]), A, w1, pl1);
				else n_cur = (ray1 + lane < A.n_active && lane >= lo1 && lane < hi1) ? S.side[ray1 + lane] : 0u;
				incl_cur = wave_inclusive_scan_fast(n_cur);
				total_cur = lane_value_u32(incl_cur, WAVE - 1);
				chain_publish(S, i_1, total_cur);
				SRF_T(7);
				if (fast1) chain_counted<G, false>(lane, n_cur, wave_max_fast(n_cur), w1, sh.rl, pl1, carry);
				peek = chain_peek(S, i_1, initial);                            // needed in the next first half; the items before this one have published by now unless their workgroups lag
				SRF_T(4);
			}
		} else if (plan_wave) {
			// the plan first: it waits for records requested an iteration ago, and that wait must not include anything younger (see above)
			plan_next(pl3);
			if (fast1) mark_owners<G>(lane, wave_max_fast(pl1.rn[lane]), w1, pl1);     // which ray each sample of item it + 1 belongs to, for its phase C
			SRF_T(4);
			if (has1) {
				const uint32_t ray1 = pl1.misc[M_GROUP] * RAYS;
				if (ray1 + lane < A.n_active) target = *(const Float4*)(A.rays_rgba + 4 * (size_t)(ray1 + lane));
			}
			if (fast) commit_loss(lane, ray0, A, sh.rl, pl, lo, hi);
			if (fast) coords_copy_single<G>(lane, A, w, sh.rl, pl);
		} else {
			if (has2 && pl2.misc[M_CONTIG] != 0) phase_a_load_single<G, HALF_IN>(st_id, A, pl2, set_l);
			SRF_T(7);
			if (fast) phase_c<G, HALF_IN, HALF_OUT, PLAIN, false>(st_id, 0, A, w, sh.rl, pl, set_c);
			SRF_T(8);
		}
		SRF_T(2);
		group_sync();
		SRF_T(3);
		if (!has1 && !has2 && it + 1 >= 0) break;
		set_c = set_a;
		set_a = set_l;
	}
#ifdef SRF_KERNEL_TIMING
	if (lane == 0 && wave <= 2) {
		unsigned long long* out = (unsigned long long*)(S.initial + 16) + wave * 12;
		for (int k = 0; k < 11; ++k) atomicAdd(out + k, t_acc_[k]);
		atomicAdd(out + 11, n_it_);
	}
#endif
}

// testbed.cu:423-446 — compaction of the live rays into dst and of the finished, visible ones into the final buffers.
// The reference hands positions out with one atomicAdd a ray, in whatever order the threads arrive; here the order is the
// source order (every later stage then sees the same arrays run after run): blocks of 1024 rays count their two classes with
// wave ballots (k_compact_count), and the moving kernel gives every block the sum of the counts before it (a block reads the
// at most few thousand counts itself), every wavefront its offset inside the block, and every lane its rank from the ballot.
constexpr uint32_t COMPACT_BLOCK = 1024;
struct Payload40 { uint32_t w[10]; };

// 1: alive, 2: finished with visible alpha, 0: dropped
__device__ __forceinline__ uint32_t compact_class(uint32_t i, uint32_t n, const srf_ray_payload* __restrict__ payloads, const float* __restrict__ rgba) {
	if (i >= n) return 0u;
	if (payloads[i].alive != 0) return 1u;
	return rgba[4 * (size_t)i + 3] > 0.001f ? 2u : 0u;
}

// counts[b] = {alive, finished} of block b; block 0 also notes the counters' values on entry, which are where this call's output starts
// the number of rays a paced compaction looks at: those alive after the last round, none once the loop has run out of iterations
__device__ __forceinline__ uint32_t paced_n(const RoundWords* __restrict__ in) { return in->next_offset < FRAME_MARCH_ITER ? in->n_alive : 0u; }

__global__ void __launch_bounds__(COMPACT_BLOCK) k_compact_count(uint32_t n, const srf_ray_payload* __restrict__ payloads, const float* __restrict__ rgba,
                                                                 U2* __restrict__ counts, const uint32_t* __restrict__ n_alive_counter,
                                                                 const uint32_t* __restrict__ n_final_counter, uint32_t* __restrict__ initial, bool alive_from_zero,
                                                                 const RoundWords* __restrict__ paced_in) {
	__shared__ uint32_t part[2][COMPACT_BLOCK / 64];
	if (paced_in) {
		n = paced_n(paced_in);
		if (blockIdx.x * COMPACT_BLOCK >= n && blockIdx.x != 0) return;      // (uniform over the block)
	}
	const uint32_t i = blockIdx.x * COMPACT_BLOCK + threadIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
	const uint32_t c = compact_class(i, n, payloads, rgba);
	const uint32_t na = (uint32_t)__popcll(__ballot(c == 1u)), nf = (uint32_t)__popcll(__ballot(c == 2u));
	if (lane == 0) { part[0][wave] = na; part[1][wave] = nf; }
	__syncthreads();
	if (threadIdx.x == 0) {
		uint32_t a = 0, f = 0;
		for (uint32_t k = 0; k < COMPACT_BLOCK / 64; ++k) { a += part[0][k]; f += part[1][k]; }
		U2 v; v.x = a; v.y = f;
		counts[blockIdx.x] = v;
		if (blockIdx.x == 0) { initial[0] = alive_from_zero || paced_in ? 0u : *n_alive_counter; initial[1] = *n_final_counter; }
	}
}

__global__ void __launch_bounds__(COMPACT_BLOCK) k_compact_move(uint32_t n, const srf_ray_payload* __restrict__ src_p, const float* __restrict__ src_c,
                                                                srf_ray_payload* __restrict__ dst_p, float* __restrict__ dst_c,
                                                                srf_ray_payload* __restrict__ fin_p, float* __restrict__ fin_c,
                                                                const U2* __restrict__ counts, const uint32_t* __restrict__ initial,
                                                                uint32_t* __restrict__ n_alive_counter, uint32_t* __restrict__ n_final_counter,
                                                                unsigned long long* __restrict__ host_word, uint32_t stamp,
                                                                const RoundWords* __restrict__ paced_in, RoundWords* __restrict__ paced_out, uint32_t n_pixels) {
	__shared__ uint32_t part[2][COMPACT_BLOCK / 64];
	__shared__ uint32_t before[2][COMPACT_BLOCK / 64];
	__shared__ uint32_t block_base[2];
	uint32_t last_block = gridDim.x - 1;
	if (paced_in) {
		n = paced_n(paced_in);
		last_block = n ? (n - 1u) / COMPACT_BLOCK : 0u;
		if (blockIdx.x > last_block) return;      // (uniform over the block)
	}
	const uint32_t i = blockIdx.x * COMPACT_BLOCK + threadIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
	// what the blocks before this one hold
	uint32_t a = 0, f = 0;
	for (uint32_t k = threadIdx.x; k < blockIdx.x; k += COMPACT_BLOCK) { const U2 v = counts[k]; a += v.x; f += v.y; }
	a = wave_sum_fast(a); f = wave_sum_fast(f);
	const uint32_t c = compact_class(i, n, src_p, src_c);
	const uint64_t m_alive = __ballot(c == 1u), m_fin = __ballot(c == 2u);
	if (lane == 0) { before[0][wave] = a; before[1][wave] = f; part[0][wave] = (uint32_t)__popcll(m_alive); part[1][wave] = (uint32_t)__popcll(m_fin); }
	__syncthreads();
	if (threadIdx.x < 2) {
		uint32_t sum = initial[threadIdx.x];
		for (uint32_t k = 0; k < COMPACT_BLOCK / 64; ++k) sum += before[threadIdx.x][k];
		block_base[threadIdx.x] = sum;
		// the wavefronts' offsets inside the block, in place of their counts
		uint32_t run = 0;
		for (uint32_t k = 0; k < COMPACT_BLOCK / 64; ++k) { const uint32_t v = part[threadIdx.x][k]; part[threadIdx.x][k] = run; run += v; }
		if (blockIdx.x == last_block) {
			if (!paced_in) *(threadIdx.x == 0 ? n_alive_counter : n_final_counter) = sum + run;
			else if (threadIdx.x == 1) *n_final_counter = sum + run;
			else {
				// the round's words (Testbed::render_frame's host arithmetic, testbed.cu:526-547, :596)
				RoundWords w;
				w.n_alive = sum + run;
				uint32_t steps = w.n_alive ? n_pixels / w.n_alive : 0u;
				steps = steps < FRAME_MIN_STEPS ? FRAME_MIN_STEPS : (steps > FRAME_MAX_STEPS ? FRAME_MAX_STEPS : steps);
				w.n_steps = w.n_alive ? steps : 0u;
				w.offset = paced_in->next_offset;
				w.n_elements = w.n_alive * w.n_steps;
				w.next_offset = w.offset + w.n_steps;
				w.rounds = paced_in->rounds + (w.n_alive ? 1u : 0u);
				w.pad[0] = w.pad[1] = 0u;
				*paced_out = w;
			}
			// for a host that waits for the number of live rays: the count with the call's stamp above it, in one store to host memory
			if (threadIdx.x == 0 && host_word) __hip_atomic_store(host_word, ((unsigned long long)stamp << 32) | (sum + run), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
		}
	}
	__syncthreads();
	const uint64_t below = (1ull << lane) - 1ull;
	if (c == 1u) {
		const uint32_t k = block_base[0] + part[0][wave] + (uint32_t)__popcll(m_alive & below);
		((Payload40*)dst_p)[k] = ((const Payload40*)src_p)[i];
		*(Float4*)(dst_c + 4 * (size_t)k) = *(const Float4*)(src_c + 4 * (size_t)i);
	} else if (c == 2u) {
		const uint32_t k = block_base[1] + part[1][wave] + (uint32_t)__popcll(m_fin & below);
		((Payload40*)fin_p)[k] = ((const Payload40*)src_p)[i];
		*(Float4*)(fin_c + 4 * (size_t)k) = *(const Float4*)(src_c + 4 * (size_t)i);
	}
}

__global__ void __launch_bounds__(256) k_shade(uint32_t n, const float* __restrict__ rgba, const srf_ray_payload* __restrict__ payloads,
                                               float* __restrict__ frame, int render_mode, int train_in_linear, const uint32_t* __restrict__ n_dev) {
	if (n_dev) n = *n_dev;
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n) shade_body(i, rgba, payloads, frame, render_mode, train_in_linear);
}

// tcnn::fill_rollover: bytes past the valid prefix repeat it cyclically
__global__ void __launch_bounds__(256) k_fill_rollover(uint32_t n_out_words, const uint32_t* __restrict__ n_in_ptr, uint32_t stride_words, uint32_t* __restrict__ buf) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	const uint32_t n_in_words = *n_in_ptr * stride_words;
	if (i < n_in_words || i >= n_out_words || n_in_words == 0) return;
	buf[i] = buf[i % n_in_words];
}

// tcnn::fill_rollover_and_rescale: the same, with the copied value scaled by n_in / n_out
template <bool HALF>
__global__ void __launch_bounds__(256) k_fill_rollover_rescale(uint32_t n_elements, uint32_t stride, const uint32_t* __restrict__ n_in_ptr, void* __restrict__ buf) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	const uint32_t n_in = *n_in_ptr;
	if (i < n_in * stride || i >= n_elements * stride || n_in == 0) return;
	const float v = net_load<HALF>(buf, i % (n_in * stride));
	net_store<HALF>(buf, i, v * (float)n_in / (float)n_elements);
}

// The chain of a streaming launch gave up (see chain_resolve): the outputs of that call are invalid.  Reported once, by the
// first call that notices; from then on the marcher composites with the three-launch implementation, which has no waits
// between workgroups.
static int check_chain_error(srf_marcher* m) {
	if (m->host_error && *m->host_error) {
		*m->host_error = 0u;
		m->degraded += 1;
		SRF_FAIL(SRF_ERR_HIP, "compositing: in an earlier call a workgroup gave up waiting for its predecessors' sample counts; that call's compacted "
		                      "offsets and gradients are invalid (its compacted counter reads 0xffffffff). This marcher now uses %s.",
		         m->degraded == 1 && !m->force_waves ? "the wave-per-item kernel" : "the three-launch implementation");
	}
	return SRF_OK;
}

// Workgroups of the streaming kernel that the device holds at once: the kernel's groups wait for one another, so its grid
// must not exceed that.  Asked of the runtime once per kernel variant.
template <bool HI, bool HO, bool PL>
static int stream_resident_workgroups(uint32_t* out) {
	constexpr int MAX_DEVICES = 64;
	static uint32_t per_device[MAX_DEVICES];      // per variant and device (racing first calls both write the same value)
	int dev = 0;
	SRF_HIP(hipGetDevice(&dev));
	SRF_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "compositing: device index %d out of range", dev);
	uint32_t cached = per_device[dev];
	if (!cached) {
		hipDeviceProp_t prop; int per_cu = 0;
		SRF_HIP(hipGetDeviceProperties(&prop, dev));
		SRF_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)k_composite_stream<HI, HO, PL>, (int)STREAM_THREADS, 0));
		if (per_cu < 1) SRF_FAIL(SRF_ERR_HIP, "compositing: the streaming kernel does not fit this device");
		if (per_cu > (int)STREAM_WORKGROUPS_PER_CU) per_cu = (int)STREAM_WORKGROUPS_PER_CU;
		cached = (uint32_t)prop.multiProcessorCount * (uint32_t)per_cu;
		per_device[dev] = cached;
	}
	*out = cached;
	return SRF_OK;
}

static int launch_stream(const srf_loss_args* a, const LossConst& K, ChainScratch S, const float* rays_rgba, const uint32_t* n_rays_counter,
                         uint32_t* ray_coord_indices, const float* dt, const float* coords, float* compacted_coords, uint32_t* n_compacted_coords_counter,
                         const void* network_output, void* dloss_doutput, float* loss_output, const float* density_grid_mean, float* rgb_ray_out, hipStream_t st) {
	const uint32_t n_groups = div_up(a->n_rays, fused::RAYS);
	fused::Args A;
	A.K = K;
	A.n_active = 0;
	A.rays_rgba = rays_rgba; A.ray_coord_indices = ray_coord_indices; A.dt_arr = dt; A.coords = coords; A.compacted_coords = compacted_coords;
	A.net = network_output; A.dloss = dloss_doutput; A.loss_output = loss_output; A.rgb_ray_out = rgb_ray_out; A.mean_density = 0.f;
	const bool hin = a->network_output_dtype == SRF_DTYPE_F16, hout = a->dloss_dtype == SRF_DTYPE_F16;
	const bool plain = a->rgb_activation == SRF_ACT_NONE && a->density_activation == SRF_ACT_NONE;
	uint32_t resident = 0;
	int rc;
#define SRF_RESIDENT(HI, HO, PL) rc = stream_resident_workgroups<HI, HO, PL>(&resident)
#define SRF_RESIDENT_IO(PL) do { if (hin && hout) SRF_RESIDENT(true, true, PL); else if (hin) SRF_RESIDENT(true, false, PL); else if (hout) SRF_RESIDENT(false, true, PL); else SRF_RESIDENT(false, false, PL); } while (0)
	if (plain) SRF_RESIDENT_IO(true); else SRF_RESIDENT_IO(false);
#undef SRF_RESIDENT_IO
#undef SRF_RESIDENT
	if (rc != SRF_OK) return rc;
	const dim3 grid(n_groups < resident ? n_groups : resident), block(STREAM_THREADS), slow_block(fused::WideGeometry::THREADS), slow_grid(n_groups < SLOW_WORKGROUPS ? n_groups : SLOW_WORKGROUPS);   // listed groups are few as a rule
	const uint32_t slow_slots = S.saved_records ? SLOW_PART_SLOTS : 1u;       // without the copy of their records a group is one workgroup's
	hipLaunchKernelGGL(k_chain_prepare, dim3(div_up(n_groups, PREPARE_WAVES)), dim3(PREPARE_WAVES * WAVE), 0, st, A, n_rays_counter, S, (const uint32_t*)n_compacted_coords_counter);
	hipLaunchKernelGGL(k_chain_items, dim3(div_up(n_groups, ITEMS_THREADS)), dim3(ITEMS_THREADS), 0, st, a->n_rays, n_rays_counter, S);
	SRF_LAUNCH_CHECK();
	if (hin) hipLaunchKernelGGL((k_slow_groups<true, false, false>), slow_grid, slow_block, 0, st, A, n_rays_counter, density_grid_mean, S, slow_slots);
	else     hipLaunchKernelGGL((k_slow_groups<false, false, false>), slow_grid, slow_block, 0, st, A, n_rays_counter, density_grid_mean, S, slow_slots);
	SRF_LAUNCH_CHECK();
#define SRF_STREAM(HI, HO, PL) hipLaunchKernelGGL((k_composite_stream<HI, HO, PL>), grid, block, 0, st, A, n_rays_counter, density_grid_mean, S, n_compacted_coords_counter)
#define SRF_STREAM_IO(PL) do { if (hin && hout) SRF_STREAM(true, true, PL); else if (hin) SRF_STREAM(true, false, PL); else if (hout) SRF_STREAM(false, true, PL); else SRF_STREAM(false, false, PL); } while (0)
	if (plain) SRF_STREAM_IO(true); else SRF_STREAM_IO(false);
#undef SRF_STREAM_IO
#undef SRF_STREAM
	SRF_LAUNCH_CHECK();
#define SRF_SLOW_BWD(HI, HO) hipLaunchKernelGGL((k_slow_groups<HI, HO, true>), slow_grid, slow_block, 0, st, A, n_rays_counter, density_grid_mean, S, slow_slots)
	if (hin && hout) SRF_SLOW_BWD(true, true); else if (hin) SRF_SLOW_BWD(true, false); else if (hout) SRF_SLOW_BWD(false, true); else SRF_SLOW_BWD(false, false);
#undef SRF_SLOW_BWD
	SRF_LAUNCH_CHECK();
#ifdef SRF_KERNEL_TIMING
	{
		unsigned long long h[36];
		SRF_HIP(hipStreamSynchronize(st));
		SRF_HIP(hipMemcpy(h, S.initial + 16, sizeof(h), hipMemcpyDeviceToHost));
		SRF_HIP(hipMemset(S.initial + 16, 0, sizeof(h)));
		static const char* names[3][9] = {{"commit", "barrier", "-", "barrier", "chain", "-", "resolve", "count+publish", "-"},
		                                  {"finish", "barrier", "rest", "barrier", "plan-tail", "rec-wait", "from-records", "part", "-"},
		                                  {"-", "barrier", "-", "barrier", "wait-loads", "phaseA", "-", "issue-loads", "phaseC"}};
		for (int role = 0; role < 3; ++role) {
			const double n = (double)h[role * 12 + 11];
			if (n == 0) continue;
			fprintf(stderr, "stream timing, %s (%.0f iterations), mean cycles:", role == 0 ? "ray wave" : role == 1 ? "plan wave" : "sample wave", n);
			for (int k = 0; k < 9; ++k) fprintf(stderr, " %s %.0f", names[role][k], h[role * 12 + k] / n);
			fprintf(stderr, "\n");
		}
	}
#endif
	return SRF_OK;
}

// srf_compact_rays; alive_from_zero: the live rays are numbered from 0 whatever the counter holds (the frame loop's case: it
// would otherwise clear the counter with a launch of its own before every round)
int compact_rays(srf_marcher* m, uint32_t n, const srf_ray_payload* src_payloads, const float* src_rgba,
                 srf_ray_payload* dst_payloads, float* dst_rgba, srf_ray_payload* final_payloads, float* final_rgba,
                 uint32_t* n_alive_counter, uint32_t* n_final_counter, bool alive_from_zero, hipStream_t st, unsigned long long* host_word, uint32_t stamp) {
	SRF_REQUIRE(m, "srf_compact_rays: NULL marcher");
	SRF_REQUIRE(n_alive_counter && n_final_counter, "srf_compact_rays: NULL counter");
	if (n == 0) {
		if (alive_from_zero) return fill_u32(n_alive_counter, 1, 0u, st);
		return SRF_OK;
	}
	SRF_REQUIRE(src_payloads && src_rgba && dst_payloads && dst_rgba && final_payloads && final_rgba, "srf_compact_rays: NULL buffer");
	const uint32_t blocks = div_up(n, COMPACT_BLOCK);
	int rc = m->compact_ws.reserve(256 + (size_t)blocks * sizeof(U2));
	if (rc != SRF_OK) return rc;
	uint32_t* initial = (uint32_t*)m->compact_ws.ptr;
	U2* counts = (U2*)((char*)m->compact_ws.ptr + 256);
	hipLaunchKernelGGL(k_compact_count, dim3(blocks), dim3(COMPACT_BLOCK), 0, st, n, src_payloads, src_rgba, counts,
	                   (const uint32_t*)n_alive_counter, (const uint32_t*)n_final_counter, initial, alive_from_zero, (const RoundWords*)nullptr);
	SRF_LAUNCH_CHECK();
	hipLaunchKernelGGL(k_compact_move, dim3(blocks), dim3(COMPACT_BLOCK), 0, st, n, src_payloads, src_rgba, dst_payloads, dst_rgba, final_payloads, final_rgba,
	                   (const U2*)counts, (const uint32_t*)initial, n_alive_counter, n_final_counter, host_word, stamp, (const RoundWords*)nullptr, (RoundWords*)nullptr, 0u);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int compact_rays_paced(srf_marcher* m, uint32_t bound, uint32_t n_pixels, const RoundWords* in, RoundWords* out, const srf_ray_payload* src_payloads, const float* src_rgba,
                       srf_ray_payload* dst_payloads, float* dst_rgba, srf_ray_payload* final_payloads, float* final_rgba, uint32_t* n_final_counter,
                       hipStream_t st, unsigned long long* host_word, uint32_t stamp) {
	const uint32_t blocks = div_up(bound ? bound : 1u, COMPACT_BLOCK);      // block 0 always runs: it writes the round's words
	int rc = m->compact_ws.reserve(256 + (size_t)div_up(n_pixels, COMPACT_BLOCK) * sizeof(U2));
	if (rc != SRF_OK) return rc;
	uint32_t* initial = (uint32_t*)m->compact_ws.ptr;
	U2* counts = (U2*)((char*)m->compact_ws.ptr + 256);
	hipLaunchKernelGGL(k_compact_count, dim3(blocks), dim3(COMPACT_BLOCK), 0, st, 0u, src_payloads, src_rgba, counts,
	                   (const uint32_t*)nullptr, (const uint32_t*)n_final_counter, initial, true, in);
	SRF_LAUNCH_CHECK();
	hipLaunchKernelGGL(k_compact_move, dim3(blocks), dim3(COMPACT_BLOCK), 0, st, 0u, src_payloads, src_rgba, dst_payloads, dst_rgba, final_payloads, final_rgba,
	                   (const U2*)counts, (const uint32_t*)initial, (uint32_t*)nullptr, n_final_counter, host_word, stamp, in, out, n_pixels);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int volume_rendering_paced(srf_marcher* m, const srf_sampler* s, const srf_render_args* a, uint32_t bound, const RoundWords* round,
                           srf_ray_payload* payloads, float* rgba, const float* coords, const void* rgbsigma, hipStream_t st) {
	if (bound == 0) return SRF_OK;
	const dim3 grid(div_up(bound, 128)), block(128);
	if (a->network_output_dtype == SRF_DTYPE_F16)
		hipLaunchKernelGGL(k_volume_rendering<true>, grid, block, 0, st, s->P, *a, m->cfg.transmittance_threshold, payloads, rgba, coords, rgbsigma, round);
	else
		hipLaunchKernelGGL(k_volume_rendering<false>, grid, block, 0, st, s->P, *a, m->cfg.transmittance_threshold, payloads, rgba, coords, rgbsigma, round);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int shade_counted(uint32_t bound, const uint32_t* n_rays, const float* rgba, const srf_ray_payload* payloads, float* frame_buffer,
                  int32_t render_mode, int32_t train_in_linear_colors, hipStream_t st) {
	if (bound == 0) return SRF_OK;
	hipLaunchKernelGGL(k_shade, dim3(div_up(bound, 256)), dim3(256), 0, st, bound, rgba, payloads, frame_buffer, render_mode, train_in_linear_colors, n_rays);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

} // namespace srf

using namespace srf;

// Argument checks and per-call constants shared by the two training compositing entry points.  *empty: nothing to do.
static int loss_call_prepare(srf_marcher* m, const srf_loss_args* a, const float* rays_rgba, const uint32_t* n_rays_counter, const uint32_t* ray_coord_indices,
                             const float* dt, const float* coords, const float* compacted_coords, const uint32_t* n_compacted_coords_counter,
                             const void* network_output, const void* dloss_doutput, const float* density_grid_mean, LossConst* K_out, bool* empty) {
	*empty = false;
	SRF_REQUIRE(m && a, "srf_marcher_volume_rendering_with_loss_and_gradient: NULL argument");
	if (a->n_rays == 0) { *empty = true; return SRF_OK; }
	SRF_REQUIRE(rays_rgba && n_rays_counter && ray_coord_indices && dt && n_compacted_coords_counter && network_output && dloss_doutput,
	            "srf_marcher_volume_rendering_with_loss_and_gradient: NULL buffer");
	SRF_REQUIRE(!a->use_grid || density_grid_mean, "srf_marcher_volume_rendering_with_loss_and_gradient: use_grid needs density_grid_mean");
	SRF_REQUIRE((coords == nullptr) == (compacted_coords == nullptr), "srf_marcher_volume_rendering_with_loss_and_gradient: coords and compacted_coords go together");
	SRF_REQUIRE(a->padded_output_width >= 4, "srf_marcher_volume_rendering_with_loss_and_gradient: padded_output_width must be >= 4");
	SRF_REQUIRE(a->dt_stride >= 1, "srf_marcher_volume_rendering_with_loss_and_gradient: dt_stride must be >= 1");
	SRF_REQUIRE(a->loss_type >= SRF_LOSS_L2 && a->loss_type <= SRF_LOSS_RELATIVEL2, "Unknown loss type.");
	SRF_REQUIRE(a->rgb_activation >= 0 && a->rgb_activation <= 3 && a->density_activation >= 0 && a->density_activation <= 3, "unknown activation");
	SRF_REQUIRE((a->network_output_dtype | 1) == 1 && (a->dloss_dtype | 1) == 1, "unknown dtype");

	LossConst K;
	K.n_rays = a->n_rays;
	K.n_max_compacted = a->n_max_compacted_coords;
	K.out_width = (uint32_t)a->padded_output_width;
	K.rgb_act = a->rgb_activation; K.density_act = a->density_activation; K.loss_type = a->loss_type;
	K.loss_scale = a->loss_scale / (float)a->n_rays;
	K.min_optical_thickness = a->min_optical_thickness;
	K.use_grid = a->use_grid;
	for (int c = 0; c < 3; ++c) K.bg_in[c] = a->background_color[c];
	if (m->cfg.train_with_random_bg_color) {   // ray_marcher.cu:82-84: one draw shared by all rays
		Pcg32 r; r.state = a->rng.state; r.inc = a->rng.inc;
		K.bg_in[0] = pcg_next_float(r); K.bg_in[1] = pcg_next_float(r); K.bg_in[2] = pcg_next_float(r);
	}
	loss_const_background(K);
	K.color_space = a->color_space;
	K.train_in_linear = m->cfg.train_in_linear_color;
	K.thr = m->cfg.transmittance_threshold;
	K.dt_stride = a->dt_stride;

	*K_out = K;
	return SRF_OK;
}

// ---- device scratch that exists without any allocation ---------------------------------------
// The chain's scratch for srf_marcher_volume_rendering_with_loss_and_gradient_noalloc: part of the library's image on every
// device, found once per device with hipGetSymbolAddress (the array's name means nothing to host code).
constexpr uint32_t NOALLOC_MAX_RAYS = SRF_NOALLOC_MAX_RAYS;
constexpr size_t NOALLOC_BYTES = chain_layout(NOALLOC_MAX_RAYS, NOALLOC_MAX_PARTS, false).bytes;
static __device__ __align__(256) unsigned char g_noalloc_scratch[NOALLOC_BYTES];
constexpr int NOALLOC_MAX_DEVICES = 64;
static void* g_noalloc_ptr[NOALLOC_MAX_DEVICES];      // per device: where g_noalloc_scratch lies in its memory
static std::mutex g_noalloc_mutex;

// with the device of the call current
static int noalloc_scratch(void** out) {
	int dev = 0;
	SRF_HIP(hipGetDevice(&dev));
	if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) SRF_FAIL(SRF_ERR_INVALID, "no-allocation compositing: device index out of range");
	std::lock_guard<std::mutex> lock(g_noalloc_mutex);
	if (!g_noalloc_ptr[dev]) {
		void* p = nullptr;
		SRF_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_noalloc_scratch)));
		g_noalloc_ptr[dev] = p;
	}
	*out = g_noalloc_ptr[dev];
	return SRF_OK;
}

extern "C" {

void srf_marcher_config_default(srf_marcher_config* c) {
	if (!c) return;
	c->train_with_random_bg_color = 1;
	c->train_in_linear_color = 0;
	c->transmittance_threshold = 0.0001f;
	c->regularization_type = SRF_REG_NONE;
}

int srf_marcher_create(const srf_marcher_config* cfg, srf_marcher_t** out) {
	SRF_REQUIRE(cfg && out, "srf_marcher_create: NULL argument");
	*out = nullptr;
	SRF_REQUIRE(cfg->regularization_type == SRF_REG_NONE || cfg->regularization_type == SRF_REG_DISTORTION, "Unknown regularization type.");
	srf_marcher* m = new srf_marcher();
	m->cfg = *cfg;
	// SRF_COMPOSITE_IMPL=unfused (read once, here) selects the three-launch, one-thread-per-ray training compositing for every
	// call on this marcher; the tests use it to compare the two implementations
	const char* impl_env = getenv("SRF_COMPOSITE_IMPL");
	m->force_unfused = impl_env && strcmp(impl_env, "unfused") == 0;
	m->force_waves = impl_env && strcmp(impl_env, "waves") == 0;
	// A word of host memory that the device can write: the streaming kernel raises it when its ordered-offset chain gives up, and
	// the next call reads it without waiting for the device.  Without a device (configuration-only use) there is none.
	int n_dev = 0;
	if (hipGetDeviceCount(&n_dev) == hipSuccess && n_dev > 0) {
		void* host = nullptr;
		if (hipHostMalloc(&host, 64, hipHostMallocMapped) == hipSuccess) {
			void* dev = nullptr;
			if (hipHostGetDevicePointer(&dev, host, 0) == hipSuccess) {
				m->host_error = (volatile uint32_t*)host;
				m->host_error_dev = (uint32_t*)dev;
				*m->host_error = 0u;
			} else {
				(void)hipHostFree(host);
			}
		}
		(void)hipGetLastError();
	}
	*out = m;
	return SRF_OK;
}

void srf_marcher_destroy(srf_marcher_t* m) {
	if (!m) return;
	m->ws.release();
	m->wave_ws.release();
	m->ws2.release();
	m->reg.release();
	m->compact_ws.release();
	m->frame_ws.release();
	if (m->frame_counter_host) (void)hipHostFree(m->frame_counter_host);
	if (m->host_error) (void)hipHostFree((void*)m->host_error);
	delete m;
}

int srf_marcher_get_config(const srf_marcher_t* m, srf_marcher_config* out) {
	SRF_REQUIRE(m && out, "srf_marcher_get_config: NULL argument");
	*out = m->cfg;
	return SRF_OK;
}

int srf_marcher_set_config(srf_marcher_t* m, const srf_marcher_config* cfg) {
	SRF_REQUIRE(m && cfg, "srf_marcher_set_config: NULL argument");
	SRF_REQUIRE(cfg->regularization_type == SRF_REG_NONE || cfg->regularization_type == SRF_REG_DISTORTION, "Unknown regularization type.");
	m->cfg = *cfg;
	return SRF_OK;
}

int srf_marcher_volume_rendering_with_loss_and_gradient(srf_marcher_t* m, const srf_loss_args* a,
        const float* rays_rgba, const uint32_t* n_rays_counter, uint32_t* ray_coord_indices,
        const float* dt, const float* coords, float* compacted_coords, uint32_t* n_compacted_coords_counter,
        const void* network_output, void* dloss_doutput, float* loss_output,
        const float* density_grid_mean, float* rgb_ray_out, void* stream) {
	LossConst K;
	bool empty = false;
	int rc = loss_call_prepare(m, a, rays_rgba, n_rays_counter, ray_coord_indices, dt, coords, compacted_coords, n_compacted_coords_counter, network_output, dloss_doutput,
	                           density_grid_mean, &K, &empty);
	if (rc != SRF_OK || empty) return rc;
	hipStream_t st = (hipStream_t)stream;
	const bool hin = a->network_output_dtype == SRF_DTYPE_F16, hout = a->dloss_dtype == SRF_DTYPE_F16;
	rc = check_chain_error(m);
	if (rc != SRF_OK) return rc;
	// The distortion regulariser's side buffer is only filled by the three-launch implementation, which also serves a marcher
	// created under SRF_COMPOSITE_IMPL=unfused and one whose chain has failed in both single-launch kernels.
	// The streaming kernel by default.  The wave-per-item kernel where asked for (SRF_COMPOSITE_IMPL=waves) and after the streaming
	// kernel's chain has given up once (its items wait for workgroups that must all be running; the wave-per-item kernel's never do).
	const bool fusable = m->cfg.regularization_type != SRF_REG_DISTORTION && !m->force_unfused;
	const int level = m->degraded + (m->force_waves ? 1 : 0);
	if (fusable && level == 1) {
		const void* before = m->wave_ws.ptr;
		rc = m->wave_ws.reserve(waves_scratch_bytes(a->n_rays));
		if (rc != SRF_OK) return rc;
		if (m->wave_ws.ptr != before) SRF_HIP(hipMemsetAsync(m->wave_ws.ptr, 0, 512, st));      // a new buffer: the words that are zero between calls
		m->chain_error_dev = waves_error_word(m->wave_ws.ptr);
		return launch_waves(a, K, m->wave_ws.ptr, m->host_error_dev, m->force_waves ? m->lookback_spin_limit : (1u << 22), rays_rgba, n_rays_counter, ray_coord_indices, dt, coords,
		                    compacted_coords, n_compacted_coords_counter, network_output, dloss_doutput, loss_output, density_grid_mean, rgb_ray_out, st);
	}
	if (fusable && level == 0) {
		rc = m->ws.reserve(chain_layout(a->n_rays, STREAM_MAX_PARTS, true).bytes);
		if (rc != SRF_OK) return rc;
		m->chain_error_dev = chain_scratch_at(m->ws.ptr, a->n_rays, STREAM_MAX_PARTS, true, nullptr, 0).error;
		return launch_stream(a, K, chain_scratch_at(m->ws.ptr, a->n_rays, STREAM_MAX_PARTS, true, m->host_error_dev, m->lookback_spin_limit), rays_rgba, n_rays_counter, ray_coord_indices, dt, coords,
		                     compacted_coords, n_compacted_coords_counter, network_output, dloss_doutput, loss_output, density_grid_mean, rgb_ray_out, st);
	}

	const size_t n = a->n_rays;
	const size_t off_fwd = 0;
	const size_t off_n = align_up(off_fwd + n * sizeof(FwdRay), 256);
	const size_t off_cb = align_up(off_n + n * 4, 256);
	const size_t off_scan = align_up(off_cb + n * 4, 256);
	rc = m->ws2.reserve(off_scan + scan_scratch_bytes(a->n_rays));
	if (rc != SRF_OK) return rc;
	char* w = (char*)m->ws2.ptr;
	FwdRay* fwd = (FwdRay*)(w + off_fwd);
	uint32_t* n_fwd = (uint32_t*)(w + off_n);
	uint32_t* cbase = (uint32_t*)(w + off_cb);
	float* reg = nullptr;
	if (m->cfg.regularization_type == SRF_REG_DISTORTION) {
		rc = m->reg.reserve((size_t)a->n_max_compacted_coords * 2 * sizeof(float));
		if (rc != SRF_OK) return rc;
		reg = (float*)m->reg.ptr;
	}
	const dim3 grid(div_up(a->n_rays, 128)), block(128);
	if (hin) hipLaunchKernelGGL(k_loss_forward<true>, grid, block, 0, st, K, rays_rgba, n_rays_counter, (const uint32_t*)ray_coord_indices, dt, network_output, fwd, n_fwd, rgb_ray_out);
	else     hipLaunchKernelGGL(k_loss_forward<false>, grid, block, 0, st, K, rays_rgba, n_rays_counter, (const uint32_t*)ray_coord_indices, dt, network_output, fwd, n_fwd, rgb_ray_out);
	SRF_LAUNCH_CHECK();
	rc = scan_exclusive_u32(n_fwd, cbase, a->n_rays, n_compacted_coords_counter, n_compacted_coords_counter, w + off_scan, st);
	if (rc != SRF_OK) return rc;
#define SRF_BWD(HI, HO) hipLaunchKernelGGL((k_loss_backward<HI, HO>), grid, block, 0, st, K, n_rays_counter, ray_coord_indices, dt, coords, compacted_coords, \
	network_output, dloss_doutput, loss_output, density_grid_mean, (const FwdRay*)fwd, (const uint32_t*)n_fwd, (const uint32_t*)cbase, reg)
	if (hin && hout) SRF_BWD(true, true);
	else if (hin) SRF_BWD(true, false);
	else if (hout) SRF_BWD(false, true);
	else SRF_BWD(false, false);
#undef SRF_BWD
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int srf_marcher_volume_rendering_with_loss_and_gradient_noalloc(srf_marcher_t* m, const srf_loss_args* a,
        const float* rays_rgba, const uint32_t* n_rays_counter, uint32_t* ray_coord_indices,
        const float* dt, const float* coords, float* compacted_coords, uint32_t* n_compacted_coords_counter,
        const void* network_output, void* dloss_doutput, float* loss_output,
        const float* density_grid_mean, float* rgb_ray_out, void* stream) {
	LossConst K;
	bool empty = false;
	int rc = loss_call_prepare(m, a, rays_rgba, n_rays_counter, ray_coord_indices, dt, coords, compacted_coords, n_compacted_coords_counter, network_output, dloss_doutput,
	                           density_grid_mean, &K, &empty);
	if (rc != SRF_OK || empty) return rc;
	SRF_REQUIRE(a->n_rays <= NOALLOC_MAX_RAYS, "srf_marcher_volume_rendering_with_loss_and_gradient_noalloc: n_rays exceeds SRF_NOALLOC_MAX_RAYS (the scratch built into the library); "
	            "use srf_marcher_volume_rendering_with_loss_and_gradient");
	SRF_REQUIRE(m->cfg.regularization_type != SRF_REG_DISTORTION, "srf_marcher_volume_rendering_with_loss_and_gradient_noalloc: the distortion regulariser needs buffers that this entry point may not allocate");
	rc = check_chain_error(m);
	if (rc != SRF_OK) return rc;
	SRF_REQUIRE(!m->force_unfused && !m->force_waves && !m->degraded, "srf_marcher_volume_rendering_with_loss_and_gradient_noalloc: this marcher no longer uses the streaming kernel; the other implementations allocate");
	void* scratch = nullptr;
	rc = noalloc_scratch(&scratch);
	if (rc != SRF_OK) return rc;
	m->chain_error_dev = chain_scratch_at(scratch, a->n_rays, NOALLOC_MAX_PARTS, false, nullptr, 0).error;
	return launch_stream(a, K, chain_scratch_at(scratch, a->n_rays, NOALLOC_MAX_PARTS, false, m->host_error_dev, m->lookback_spin_limit), rays_rgba, n_rays_counter, ray_coord_indices, dt, coords,
	                     compacted_coords, n_compacted_coords_counter, network_output, dloss_doutput, loss_output, density_grid_mean, rgb_ray_out, (hipStream_t)stream);
}

int srf_marcher_sync_check(srf_marcher_t* m, void* stream) {
	SRF_REQUIRE(m, "srf_marcher_sync_check: NULL marcher");
	SRF_HIP(hipStreamSynchronize((hipStream_t)stream));
	if (m->chain_error_dev) {
		uint32_t flag = 0;
		SRF_HIP(hipMemcpy(&flag, m->chain_error_dev, 4, hipMemcpyDeviceToHost));
		if (flag) {      // reported once: the word is cleared, and the marcher's next call uses the next implementation, with an error word of its own
			const uint32_t zero = 0;
			SRF_HIP(hipMemcpy(m->chain_error_dev, &zero, 4, hipMemcpyHostToDevice));
			m->chain_error_dev = nullptr;
		}
		if (flag && m->host_error) *m->host_error = 1u;
		if (flag && !m->host_error) {
			m->degraded += 1;
			SRF_FAIL(SRF_ERR_HIP, "compositing: a workgroup gave up waiting for its predecessors' sample counts; compacted offsets of the last call are invalid");
		}
	}
	return check_chain_error(m);
}

int srf_marcher_debug_set_lookback_spin_limit(srf_marcher_t* m, uint32_t polls) {
	SRF_REQUIRE(m, "srf_marcher_debug_set_lookback_spin_limit: NULL marcher");
	m->lookback_spin_limit = polls;
	return SRF_OK;
}

int srf_marcher_volume_rendering(srf_marcher_t* m, const srf_sampler_t* s, const srf_render_args* a,
                                 srf_ray_payload* payloads, float* rgba, const float* coords, const void* rgbsigma, void* stream) {
	SRF_REQUIRE(m && s && a, "srf_marcher_volume_rendering: NULL argument");
	if (a->n_rays == 0) return SRF_OK;
	SRF_REQUIRE(payloads && rgba && coords && rgbsigma, "srf_marcher_volume_rendering: NULL buffer");
	SRF_REQUIRE(a->padded_output_width >= 4, "srf_marcher_volume_rendering: padded_output_width must be >= 4");
	SRF_REQUIRE(a->render_mode >= SRF_RENDER_AO && a->render_mode <= SRF_RENDER_COST, "srf_marcher_volume_rendering: unknown render mode");
	SRF_REQUIRE((a->network_output_dtype | 1) == 1, "srf_marcher_volume_rendering: unknown dtype");
	const dim3 grid(div_up(a->n_rays, 128)), block(128);
	if (a->network_output_dtype == SRF_DTYPE_F16)
		hipLaunchKernelGGL(k_volume_rendering<true>, grid, block, 0, (hipStream_t)stream, s->P, *a, m->cfg.transmittance_threshold, payloads, rgba, coords, rgbsigma, (const RoundWords*)nullptr);
	else
		hipLaunchKernelGGL(k_volume_rendering<false>, grid, block, 0, (hipStream_t)stream, s->P, *a, m->cfg.transmittance_threshold, payloads, rgba, coords, rgbsigma, (const RoundWords*)nullptr);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int srf_compact_rays(srf_marcher_t* m, uint32_t n, const srf_ray_payload* src_payloads, const float* src_rgba,
                     srf_ray_payload* dst_payloads, float* dst_rgba, srf_ray_payload* final_payloads, float* final_rgba,
                     uint32_t* n_alive_counter, uint32_t* n_final_counter, void* stream) {
	return srf::compact_rays(m, n, src_payloads, src_rgba, dst_payloads, dst_rgba, final_payloads, final_rgba, n_alive_counter, n_final_counter, false, (hipStream_t)stream, nullptr, 0u);
}

int srf_shade(uint32_t n_rays, const float* rgba, const srf_ray_payload* payloads, float* frame_buffer,
              int32_t render_mode, int32_t train_in_linear_colors, void* stream) {
	if (n_rays == 0) return SRF_OK;
	SRF_REQUIRE(rgba && payloads && frame_buffer, "srf_shade: NULL buffer");
	hipLaunchKernelGGL(k_shade, dim3(div_up(n_rays, 256)), dim3(256), 0, (hipStream_t)stream, n_rays, rgba, payloads, frame_buffer, render_mode, train_in_linear_colors, (const uint32_t*)nullptr);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int srf_fill_rollover(uint32_t n_elements, uint32_t stride_bytes, const uint32_t* n_input_elements, void* inout, void* stream) {
	if (n_elements == 0) return SRF_OK;
	SRF_REQUIRE(n_input_elements && inout, "srf_fill_rollover: NULL buffer");
	SRF_REQUIRE(stride_bytes % 4 == 0 && stride_bytes > 0, "srf_fill_rollover: stride must be a positive multiple of 4 bytes");
	const uint64_t words = (uint64_t)n_elements * (stride_bytes / 4);
	SRF_REQUIRE(words < 0xffffffffull, "srf_fill_rollover: buffer too large");
	hipLaunchKernelGGL(k_fill_rollover, dim3(div_up((uint32_t)words, 256)), dim3(256), 0, (hipStream_t)stream, (uint32_t)words, n_input_elements, stride_bytes / 4, (uint32_t*)inout);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int srf_fill_rollover_and_rescale(uint32_t n_elements, uint32_t stride, const uint32_t* n_input_elements, void* inout, int32_t dtype, void* stream) {
	if (n_elements == 0 || stride == 0) return SRF_OK;
	SRF_REQUIRE(n_input_elements && inout, "srf_fill_rollover_and_rescale: NULL buffer");
	SRF_REQUIRE((dtype | 1) == 1, "srf_fill_rollover_and_rescale: unknown dtype");
	SRF_REQUIRE((uint64_t)n_elements * stride < 0xffffffffull, "srf_fill_rollover_and_rescale: buffer too large");
	const uint32_t total = n_elements * stride;
	if (dtype == SRF_DTYPE_F16) hipLaunchKernelGGL(k_fill_rollover_rescale<true>, dim3(div_up(total, 256)), dim3(256), 0, (hipStream_t)stream, n_elements, stride, n_input_elements, inout);
	else hipLaunchKernelGGL(k_fill_rollover_rescale<false>, dim3(div_up(total, 256)), dim3(256), 0, (hipStream_t)stream, n_elements, stride, n_input_elements, inout);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

} // extern "C"
