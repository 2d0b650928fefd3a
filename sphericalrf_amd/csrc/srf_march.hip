// Ray generation and marching through the occupancy bitfield: the training sampler
// (count, ordered offsets, write), the rendering sampler (payload init, advance to the
// first occupied cell, fixed-size sample chunks) and the whole-frame march+composite kernel.
#include <stdlib.h>
#include "srf_internal.h"
#include "srf_bodies.h"
#include "srf_wave.h"

namespace srf {

// Counting march, one wavefront per block.  Each lane carries one ray through the phases of
// srf_bodies.h's state machine; every round the wavefront runs the phase most of its lanes are
// waiting for (stepping through known-empty space, probing the grid, or picking up the next ray
// of the block's range), so the expensive probe is issued for many lanes at once instead of
// whenever any single lane needs one.
// steps per stepping round, at most: long enough to spread the round's fixed work (phase ballots, the first reciprocal of the
// chain, the closed-form stretch) over many steps; the burst runs in groups of four and ends when no lane has a step left, so a
// long limit costs the lanes that wait for a probe little (24: 1.51 ms, 32: 1.33 ms, 48: 1.29 ms, 64: 1.35 ms for the march of
// the 2^20-ray batch, with probing lanes waiting until they outnumber the stepping ones 32 to 1)
constexpr uint32_t COUNT_STEP_BURST = 48;

// five wavefronts a SIMD: 102 registers a lane, which the counting march just fits
#define SRF_COUNT_WAVES_PER_EU 5
// counting sort of one chunk of ray indices by ray_chunk_key_body; the order inside a bin is whatever the atomics give
__global__ void __launch_bounds__(RAY_CHUNK_BINS) k_ray_order(Params P, CountArgs A, uint32_t* __restrict__ order) {
	__shared__ uint32_t bins[RAY_CHUNK_BINS];   // one thread per bin
	__shared__ uint32_t part[RAY_CHUNK_BINS];
	__shared__ uint16_t keys[RAY_CHUNK];
	const uint32_t first = blockIdx.x * RAY_CHUNK;
	const uint32_t n = A.n_rays - first < RAY_CHUNK ? A.n_rays - first : RAY_CHUNK;
	const uint32_t chunk_image = train_ray_image(first, A);
	bins[threadIdx.x] = 0;
	__syncthreads();
	for (uint32_t j = threadIdx.x; j < n; j += RAY_CHUNK_BINS) {
		const uint32_t k = ray_chunk_key_body(first + j, chunk_image, P, A);
		keys[j] = (uint16_t)k;
		atomicAdd(&bins[k], 1u);
	}
	__syncthreads();
	const uint32_t count = bins[threadIdx.x];
	part[threadIdx.x] = count;
	__syncthreads();
	for (uint32_t d = 1; d < RAY_CHUNK_BINS; d <<= 1) {
		const uint32_t v = threadIdx.x >= d ? part[threadIdx.x - d] : 0u;
		__syncthreads();
		part[threadIdx.x] += v;
		__syncthreads();
	}
	bins[threadIdx.x] = part[threadIdx.x] - count;
	__syncthreads();
	for (uint32_t j = threadIdx.x; j < n; j += RAY_CHUNK_BINS) order[first + atomicAdd(&bins[keys[j]], 1u)] = first + j;
}

template <bool SPHERE>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(SRF_COUNT_WAVES_PER_EU))) k_train_count(Params P, CountArgs A, uint32_t rays_per_wave, uint32_t probe_quorum, uint32_t begin_quorum, uint32_t probe_ratio,
                                                                                                                    const uint32_t* __restrict__ order, unsigned long long* timing) {
	const uint32_t lane = threadIdx.x;
	// The wavefronts are taken from the last rays of the batch to the first.  The kernel ends with its last wavefront, lifetimes
	// differ by a factor of three between cameras, and how the expensive ones fall in the order of dispatch moves the kernel's time by
	// a third: with the batch's 200 cameras dealt to the rays in three different rotations, 1.31 / 1.57 / 1.18 ms first to last and
	// 1.26 / 1.20 / 1.12 ms last to first.  Orders made from the cost of every chunk of 4096 rays in the batch before (most expensive
	// first; several falling ramps; the cheapest quarter last; two or four runs of neighbouring chunks side by side) were all slower than
	// the latter (presumably because whatever takes neighbouring cameras apart in time costs the lookups their locality); why the
	// falling order beats the rising one in all three is not understood beyond that its last wavefronts happened to be cheap ones.
	uint32_t next = (gridDim.x - 1u - blockIdx.x) * rays_per_wave;
#ifdef SRF_KERNEL_TIMING
	// per phase (step, probe, begin): cycles, rounds, lanes that took part
	unsigned long long t_acc_[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
	unsigned long long t_prev_ = clock64();
	const unsigned long long t_first_ = t_prev_, w_first_ = wall_clock64();
#define SRF_COUNT_STAMP(k, lanes) do { const unsigned long long now_ = clock64(); t_acc_[k] += now_ - t_prev_; t_prev_ = now_; t_acc_[3 + k] += 1; t_acc_[6 + k] += (lanes); } while (0)
#else
#define SRF_COUNT_STAMP(k, lanes) ((void)0)
#endif
	const uint32_t end = next + rays_per_wave < A.n_rays ? next + rays_per_wave : A.n_rays;
	CountLane L;
	L.phase = LANE_IDLE;
	for (;;) {
		const uint64_t m_idle = __ballot(L.phase == LANE_IDLE);
		const uint32_t n_probe = (uint32_t)__popcll(__ballot(L.phase == LANE_PROBE));
		const uint32_t n_step = (uint32_t)__popcll(__ballot(L.phase == LANE_STEP));
		const uint32_t left = end - next;
		uint32_t n_idle = (uint32_t)__popcll(m_idle);
		n_idle = n_idle < left ? n_idle : left;
		if (!(n_idle | n_probe | n_step)) break;
		// stepping is cheap and probing is not: lanes that want a probe wait while others step, until they are all of
		// the wavefront or outnumber the stepping lanes probe_ratio to one (a few long skips must not hold up the rest)
		const bool begin = n_idle >= begin_quorum || (n_idle && !n_probe && !n_step);
		const bool step = !begin && n_step && n_probe < probe_quorum && n_probe < probe_ratio * n_step;
		if (step) {
			if (L.phase == LANE_STEP) count_steps<COUNT_STEP_BURST>(L, P, A);
			SRF_COUNT_STAMP(0, n_step);
		} else if (!begin) {
			if (L.phase == LANE_PROBE) count_probe<SPHERE>(L, P, A, n_probe + n_step <= A.park_lanes);
			SRF_COUNT_STAMP(1, n_probe);
		} else {
			const uint32_t rank = (uint32_t)__popcll(m_idle & ((1ull << lane) - 1ull));
			if (L.phase == LANE_IDLE && rank < n_idle) count_begin(L, order ? order[next + rank] : next + rank, P, A);
			next += n_idle;
			SRF_COUNT_STAMP(2, n_idle);
		}
	}
#ifdef SRF_KERNEL_TIMING
	if (lane == 0) {
		for (int k = 0; k < 9; ++k) atomicAdd(&timing[(blockIdx.x & 1023u) * 16 + k], t_acc_[k]);
		atomicAdd(&timing[(blockIdx.x & 1023u) * 16 + 9], clock64() - t_first_);
		atomicAdd(&timing[(blockIdx.x & 1023u) * 16 + 10], wall_clock64() - w_first_);
		const unsigned long long life_ = wall_clock64() - w_first_;
		atomicMax(&timing[(blockIdx.x & 1023u) * 16 + 11], life_);
		// histograms: lifetime in 100 us buckets, probe rounds in buckets of 64
		const unsigned long long lb = life_ / 10000ull, pb = t_acc_[4] / 64ull;
		atomicAdd(&timing[1024 * 16 + (lb < 47 ? lb : 47)], 1ull);
		atomicAdd(&timing[1024 * 16 + 48 + (pb < 47 ? pb : 47)], 1ull);
		const unsigned long long sb = t_acc_[3] / 64ull;
		atomicAdd(&timing[1024 * 16 + 96 + (sb < 47 ? sb : 47)], 1ull);
		// of the slow wavefronts (over 1 ms): step rounds, probe rounds, lanes per step round
		if (life_ > 100000ull) { atomicAdd(&timing[1024 * 16 + 144], 1ull); atomicAdd(&timing[1024 * 16 + 145], t_acc_[3]); atomicAdd(&timing[1024 * 16 + 146], t_acc_[4]);
			atomicAdd(&timing[1024 * 16 + 147], t_acc_[6]); atomicAdd(&timing[1024 * 16 + 148], t_acc_[7]); atomicAdd(&timing[1024 * 16 + 149], t_acc_[0]); atomicAdd(&timing[1024 * 16 + 150], t_acc_[1]); }
	}
#endif
}

// The wide march of the parked rays: one ray per workgroup of two wavefronts at a time.  The second wavefront runs the
// chain of t one round (64 steps) ahead, since the step sizes do not depend on what the grid holds; in the first, every
// lane looks one of the current round's 64 positions up and lane 0 replays the loop's bookkeeping over the results.
template <bool SPHERE>
__global__ void __launch_bounds__(128) k_train_count_wide(Params P, CountArgs A) {
	__shared__ float t[2][WIDE_STEPS + 1];
	__shared__ uint64_t zero_steps[2];
	__shared__ uint32_t finished[2];      // per round parity, like t: a flag is not rewritten before both wavefronts have read it
	const uint32_t lane = threadIdx.x & 63u;
	const bool chain_wave = threadIdx.x >= 64u;
	const uint32_t filled = *A.parked_count;
	const uint32_t n = filled < A.parked_capacity ? filled : A.parked_capacity;
	for (uint32_t q = blockIdx.x; q < n; q += gridDim.x) {
		CountLane L;              // every lane has the ray (o and d are what the lookups need); lane 0 of the first wavefront advances it
		count_unpark(L, A.parked[q]);
		if (chain_wave && lane == 0) zero_steps[0] = wide_chain(P, L.t, t[0]);
		__syncthreads();
		for (uint32_t cur = 0;; cur ^= 1u) {
			if (chain_wave) {
				// the next round starts where this one ends, if the ray gets that far
				if (lane == 0) zero_steps[cur ^ 1u] = wide_chain(P, t[cur][WIDE_STEPS], t[cur ^ 1u]);
			} else {
				const uint32_t f = wide_flags(wide_lookup<SPHERE>(P, A, L.o, L.d, t[cur][lane]));
				const uint64_t m_inside = __ballot((f & 1u) != 0u), m_occ = __ballot((f & 2u) != 0u);
				if (lane == 0) {
					wide_apply(L, P, A, t[cur], m_inside, m_occ, zero_steps[cur]);
					finished[cur] = L.phase == LANE_IDLE ? 1u : 0u;
				}
			}
			__syncthreads();      // t[cur] and finished[cur] are rewritten in the round after next
			if (finished[cur]) break;
		}
	}
}

__global__ void k_zero_word(uint32_t* p) { *p = 0u; }

// Sample offsets and ray indices of a training batch in three launches.  A ray's first sample is the sum of the counts of
// all rays before it (occupancy_sampler.cu:634: the counter advances by every ray's count, kept or not); a ray is kept when
// its samples fit (train_keep_flag); a kept ray's index is the number of kept rays before it.  Tiles of 1024 rays:
//   k_train_tile_counts   count sum of every tile; copies the two counters' values at entry
//   k_train_bases         a tile's first offset = entry value + the sums of the tiles before it (every workgroup adds them up
//                         itself: 1024 words for 2^20 rays); offsets, keep flags, kept rays of the tile; new sample counter
//   k_train_ray_indices   the same over the kept flags; new ray counter
constexpr uint32_t OFFSET_THREADS = 256;
constexpr uint32_t OFFSET_TILE = 1024;

struct TrainOffsetScratch {
	uint32_t* tile_counts;   // [n_tiles]
	uint32_t* tile_kept;     // [n_tiles]
	uint32_t* entry;         // [2]: sample counter, ray counter when the call began
};

static size_t train_offset_scratch_bytes(uint32_t n_rays) { return align_up(((size_t)div_up(n_rays ? n_rays : 1u, OFFSET_TILE) * 2 + 2) * sizeof(uint32_t), 256); }

__global__ void __launch_bounds__(OFFSET_THREADS) k_train_tile_counts(uint32_t n_rays, const uint32_t* __restrict__ counts, TrainOffsetScratch S,
                                                                      const uint32_t* __restrict__ n_coords_counter, const uint32_t* __restrict__ n_rays_counter) {
	__shared__ uint32_t lds[OFFSET_THREADS / 64];
	const uint32_t first = blockIdx.x * OFFSET_TILE + threadIdx.x * 4;
	uint32_t v = 0;
	for (uint32_t k = 0; k < 4; ++k) if (first + k < n_rays) v += counts[first + k];
	const uint32_t total = block_sum_u32<OFFSET_THREADS>(v, lds);
	if (threadIdx.x == 0) S.tile_counts[blockIdx.x] = total;
	if (blockIdx.x == 0 && threadIdx.x == 0) { S.entry[0] = *n_coords_counter; S.entry[1] = *n_rays_counter; }
}

// sum of the tile sums before this workgroup's tile (wrapping, like the counter it continues)
__device__ __forceinline__ uint32_t tiles_before(const uint32_t* __restrict__ tile_sums, uint32_t* lds) {
	uint32_t v = 0;
	for (uint32_t k = threadIdx.x; k < blockIdx.x; k += OFFSET_THREADS) v += tile_sums[k];
	return block_sum_u32<OFFSET_THREADS>(v, lds);
}

__global__ void __launch_bounds__(OFFSET_THREADS) k_train_bases(uint32_t n_rays, uint32_t n_coords, const uint32_t* __restrict__ counts, TrainOffsetScratch S,
                                                                uint32_t* __restrict__ base, uint32_t* __restrict__ keep, uint32_t* __restrict__ n_coords_counter) {
	__shared__ uint32_t lds[OFFSET_THREADS / 64 + 1];
	const uint32_t before = S.entry[0] + tiles_before(S.tile_counts, lds);
	const uint32_t first = blockIdx.x * OFFSET_TILE + threadIdx.x * 4;
	uint32_t c[4];
	uint32_t sum = 0;
	for (uint32_t k = 0; k < 4; ++k) { c[k] = first + k < n_rays ? counts[first + k] : 0u; sum += c[k]; }
	uint32_t total;
	uint32_t run = before + block_exclusive_scan_u32<OFFSET_THREADS>(sum, lds, &total);
	uint32_t kept = 0;
	for (uint32_t k = 0; k < 4; ++k) {
		if (first + k < n_rays) {
			const uint32_t flag = train_keep_flag(c[k], run, n_coords);
			base[first + k] = run;
			keep[first + k] = flag;
			kept += flag;
		}
		run += c[k];
	}
	const uint32_t kept_total = block_sum_u32<OFFSET_THREADS>(kept, lds);
	if (threadIdx.x == 0) {
		S.tile_kept[blockIdx.x] = kept_total;
		if (blockIdx.x + 1 == gridDim.x) *n_coords_counter = before + total;
	}
}

__global__ void __launch_bounds__(OFFSET_THREADS) k_train_ray_indices(uint32_t n_rays, const uint32_t* __restrict__ keep, TrainOffsetScratch S,
                                                                      uint32_t* __restrict__ ridx, uint32_t* __restrict__ n_rays_counter) {
	__shared__ uint32_t lds[OFFSET_THREADS / 64 + 1];
	const uint32_t before = S.entry[1] + tiles_before(S.tile_kept, lds);
	const uint32_t first = blockIdx.x * OFFSET_TILE + threadIdx.x * 4;
	uint32_t f[4];
	uint32_t sum = 0;
	for (uint32_t k = 0; k < 4; ++k) { f[k] = first + k < n_rays ? keep[first + k] : 0u; sum += f[k]; }
	uint32_t total;
	uint32_t run = before + block_exclusive_scan_u32<OFFSET_THREADS>(sum, lds, &total);
	for (uint32_t k = 0; k < 4; ++k) {
		if (first + k < n_rays) ridx[first + k] = run;
		run += f[k];
	}
	if (threadIdx.x == 0 && blockIdx.x + 1 == gridDim.x) *n_rays_counter = before + total;
}

// Writing march, one wavefront per block.  The samples of the block's kept rays form one run of the sample arrays
// (offsets are in ray order).  The run goes through LDS in windows: each lane replays its ray's step log, which only
// yields the t of every sample, and drops t and its own number into the sample's slot; then consecutive lanes take
// consecutive slots, compute what the sample stores (warp, cell, step) and write it, so that the per-sample work
// is spread evenly whatever the rays' sample counts are, and the stores of a wavefront are contiguous.
constexpr uint32_t WRITE_WINDOW = 1024;

struct WindowEmit {
	float* win_t; uint8_t* win_ray;
	uint32_t first, size, base, lane;      // window [first, first + size) of sample indices; the ray's first sample
	__device__ bool operator()(uint32_t j, float t) const {
		const uint32_t k = base + j;
		if (k >= first + size) return false;               // the rest of the ray belongs to later windows
		if (k >= first) { win_t[k - first] = t; win_ray[k - first] = (uint8_t)lane; }
		return true;
	}
};

__global__ void __launch_bounds__(64) k_train_write(Params P, uint32_t n_rays, DatasetArgs ds, const uint8_t* __restrict__ bitfield,
                                                    const TrainRay* __restrict__ state, const uint32_t* __restrict__ counts,
                                                    const uint32_t* __restrict__ base, const uint32_t* __restrict__ keep,
                                                    const uint32_t* __restrict__ ray_index,
                                                    float* __restrict__ rays_out, float* __restrict__ rays_rgba, uint32_t* __restrict__ numsteps_out,
                                                    float* __restrict__ coords_out, float* __restrict__ sample_t, float* __restrict__ sample_dt, uint32_t* __restrict__ sample_cell, StepLog log) {
	__shared__ float win_t[WRITE_WINDOW];
	__shared__ uint8_t win_ray[WRITE_WINDOW];
	__shared__ float ray_odw[64][9];             // origin, direction, warped direction of the lanes' rays
	const uint32_t lane = threadIdx.x;
	const uint32_t i = (gridDim.x - 1u - blockIdx.x) * 64u + lane;      // last rays first, like the counting march (181 -> 171 us)
	const bool kept = i < n_rays && keep[i] != 0;
	DirectSink out;
	out.sample_t = sample_t; out.sample_dt = sample_dt; out.sample_cell = sample_cell;
	TrainRay st;
	WriteRay R;
	R.numsteps = 0; R.base = 0;
	bool replayed = false;
	if (kept) {
		st = state[i];
		R = train_write_ray(i, ds, st, counts, base, ray_index, rays_out, rays_rgba, numsteps_out);
		st3(&ray_odw[lane][0], R.o); st3(&ray_odw[lane][3], R.d); st3(&ray_odw[lane][6], R.wdir);
		replayed = log.bits != nullptr && st.logged != 0u;
		// without a usable log the ray marches again on its own
		if (!replayed) train_write_march(P, bitfield, R, train_write_cap(P, R.numsteps), coords_out, out);
	}
	// the block's run of replayed samples
	uint32_t lo = replayed ? R.base : 0xffffffffu, hi = replayed ? R.base + R.numsteps : 0u;
	for (uint32_t off = 32; off > 0; off >>= 1) {
		const uint32_t lo2 = (uint32_t)__shfl_xor((int)lo, (int)off, 64), hi2 = (uint32_t)__shfl_xor((int)hi, (int)off, 64);
		lo = lo2 < lo ? lo2 : lo;
		hi = hi2 > hi ? hi2 : hi;
	}
	for (uint32_t first = lo; first < hi; first += WRITE_WINDOW) {     // uniform: lo and hi are the same in every lane
		const uint32_t size = hi - first < WRITE_WINDOW ? hi - first : WRITE_WINDOW;
		for (uint32_t q = lane; q < size; q += 64u) win_t[q] = srf_u2f(WINDOW_EMPTY);
		__syncthreads();
		if (replayed && R.base < first + size && R.base + R.numsteps > first) {
			WindowEmit emit;
			emit.win_t = win_t; emit.win_ray = win_ray; emit.first = first; emit.size = size; emit.base = R.base; emit.lane = lane;
			train_write_replay(i, P, st, train_write_cap(P, R.numsteps), log, emit);
		}
		__syncthreads();
		for (uint32_t q = lane; q < size; q += 64u) {
			const float t = win_t[q];
			if (srf_f2u(t) == WINDOW_EMPTY) continue;      // a slot of a ray that was dropped or has marched on its own
			const float* r = ray_odw[win_ray[q]];
			train_write_sample(P, ld3(r), ld3(r + 3), ld3(r + 6), t, (size_t)first + q, coords_out, out);
		}
		__syncthreads();
	}
}

__global__ void __launch_bounds__(128) k_init_rays(Params P, PixelArgs A, srf_ray_payload* __restrict__ payloads) {
	const uint32_t x = threadIdx.x + blockDim.x * blockIdx.x;
	const uint32_t y = threadIdx.y + blockDim.y * blockIdx.y;
	if (x < (uint32_t)A.res[0] && y < (uint32_t)A.res[1]) init_ray_body(x, y, P, A, payloads);
}

// The render marches (first occupied cell, next chunk of samples, whole frame), one wavefront per block and one ray per
// lane.  Every round the wavefront runs one phase of srf_bodies.h's march machine: steps through known-empty space while
// any lane has some to take, a grid probe (with whatever the march does at an occupied cell) once all lanes wait for one.
// A lane waiting for its probe idles through the step rounds, so that the expensive probe is issued for all lanes at once.
// Letting the probing lanes go first once they outnumber the stepping ones, and stepping in bursts of a fixed length (as the
// counting march does), costs 5 to 15 % of a frame on the render workloads: here most lanes walk the same long empty
// stretches side by side.
// A ray that crawls (an empty cell and nothing to skip at every probe: it runs along occupied blocks) costs a round of dependent
// loads a step, and when it is one of the last few rays of its wavefront nothing hides them: such rays alone kept a frame of the
// bounded-object workload alive four times longer than its average wavefront.  A wavefront down to PARK_MAX_LANES rays (16: 8
// leaves a seventh of that frame's time on the table, 32 gains nothing more) therefore
// parks those that have crawled PARK_CRAWL probes in a row: the lane's state goes to a queue as it stands, and k_march_wide
// carries each parked ray on, one ray a wavefront.  There a crawling ray is taken through its next 64 steps at once: every lane
// follows the chain of t (it has to be followed step by step) and keeps the value before its own step, looks that position up, and
// the first step that is not "inside, empty, of positive size" is where the ray's own probe carries on; nothing else of the
// ray's state moves, so the march's outcome is the one of probing step by step.
// (settled on the render workloads: parking after 16 or 32 probes costs the frames without such rays 5 to 10 % in rays that
// would have stopped crawling soon; wide rounds inside the march kernel itself cost them more than that in registers)
constexpr uint32_t PARK_MAX_LANES = 16, PARK_CRAWL = 64;
struct MarchPark { void* slots; uint32_t* count; uint32_t* next_count; uint32_t capacity, max_lanes, min_crawl; };

__device__ __forceinline__ float lane_value_f32(float v, uint32_t uniform_lane) { return srf_u2f(lane_value_u32(srf_f2u(v), uniform_lane)); }
// the ray in lane `owner`; true when the next 64 steps held nothing (the ray may go wide again at once)
__device__ inline bool march_wide_round(const MarchGrid& G, MarchLane& L, uint32_t owner) {
	const Params& P = G.P;
	const uint32_t lane = threadIdx.x & 63u;
	const float cone = P.cone_angle_constant;
	const Vec3 o = mk3(lane_value_f32(L.o.x, owner), lane_value_f32(L.o.y, owner), lane_value_f32(L.o.z, owner));
	const Vec3 d = mk3(lane_value_f32(L.d.x, owner), lane_value_f32(L.d.y, owner), lane_value_f32(L.d.z, owner));
	const float t0 = lane_value_f32(L.t, owner);
	float t_mine = t0, t_end = t0;
	bool zero_mine = false, chained = false;
	const ShortForm f = disparity_short_form(P);
	if (f.usable && t0 >= f.t_lo) {
		// the whole batch in the short form, checked afterwards: every step must start inside the form's range (past it the chain
		// runs through infinity to negative values, so the last step's start alone does not tell)
		ShortChain ch = short_chain_at(t0);
		for (uint32_t k = 0; k < 64u; ++k) {
			t_mine = k == lane ? ch.t : t_mine;
			ch = short_chain_next(f, ch);
		}
		t_end = ch.t;
		chained = __ballot(!(t_mine >= f.t_lo && t_mine <= f.t_hi)) == 0ull;
	}
	if (!chained) {
		float t = t0;
		for (uint32_t k = 0; k < 64u; ++k) {
			const float dt = calc_dt(P, t, cone);
			if (k == lane) { t_mine = t; zero_mine = dt == 0.f; }
			t += dt;
		}
		t_end = t;
	}
	const Vec3 pos = along(o, d, t_mine);
	bool event = !aabb_contains(P, pos) || zero_mine;
	if (!event) {
		bool look = true;
		if (P.sphere[3] > 0.f) {
			float t_enter;
			const SphereGate g = sphere_gate(P, o, d, t_mine, &t_enter);
			event = g == SPHERE_BEYOND;
			look = g == SPHERE_INSIDE;
		}
		if (look) event = probe_at(P, G.bitfield, pos, t_mine, cone).occ;
	}
	const uint64_t m = __ballot(event);
	const float t_new = m ? lane_value_f32(t_mine, (uint32_t)__builtin_ctzll(m)) : t_end;
	if (lane == owner) { L.t = L.t_limit = t_new; L.phase = LANE_PROBE; if (m) L.crawl = 0; }
	return m == 0ull;
}

// numbers that a march takes from device memory when its kernels start, where the host only knows an upper limit of them
template <class March> __device__ __forceinline__ void march_resolve(March&) {}
__device__ __forceinline__ void march_resolve(CoordsMarch& M) { if (M.round) { M.n_rays = M.round[0]; M.n_steps = M.round[1]; } }

// the parked rays, one a wavefront: lane 0 carries the ray's state and runs its probes and steps, all lanes its wide rounds
template <class March>
__global__ void __launch_bounds__(64) k_march_wide(March M, MarchPark park) {
	march_resolve(M);
	const uint32_t lane = threadIdx.x;
	const uint32_t filled = *park.count;
	const uint32_t n = filled < park.capacity ? filled : park.capacity;
	for (uint32_t q = blockIdx.x; q < n; q += gridDim.x) {
		typename March::Lane L;
		L.m.phase = LANE_IDLE; L.m.crawl = 0;
		L.m.o = mk3(0.f, 0.f, 0.f); L.m.d = L.m.o; L.m.t = 0.f;
		if (lane == 0) L = ((const typename March::Lane*)park.slots)[q];
		for (;;) {
			const uint32_t phase = lane_value_u32(L.m.phase, 0u);
			if (phase == LANE_IDLE) break;
			MarchEnd end = MARCH_GOES_ON;
			if (phase == LANE_STEP) { if (lane == 0) end = M.steps(L); }
			else if (lane_value_u32(L.m.crawl, 0u) != 0u) march_wide_round(M.G, L.m, 0u);
			else if (lane == 0) end = M.probe(L);
			if (lane == 0 && end != MARCH_GOES_ON) { M.finish(L, end); L.m.phase = LANE_IDLE; }
		}
	}
}

#ifdef SRF_KERNEL_TIMING
// per phase (step, probe): cycles, rounds, lanes that took part; then wavefronts, their lifetime in cycles, the longest in 10 ns ticks
__device__ unsigned long long g_march_timing[16];
#endif
template <class March>
__global__ void __launch_bounds__(64) k_march_lanes(March M, MarchPark park) {
	march_resolve(M);
	const uint32_t q = blockIdx.x * 64u + threadIdx.x;
	typename March::Lane L;
	L.m.phase = LANE_IDLE;
#ifdef SRF_KERNEL_TIMING
	unsigned long long t_acc_[6] = {0, 0, 0, 0, 0, 0};
	unsigned long long t_prev_ = clock64();
	const unsigned long long t_first_ = t_prev_, w_first_ = wall_clock64();
#define SRF_MARCH_STAMP(k, lanes) do { const unsigned long long now_ = clock64(); t_acc_[k] += now_ - t_prev_; t_prev_ = now_; t_acc_[2 + k] += 1; t_acc_[4 + k] += (lanes); } while (0)
#else
#define SRF_MARCH_STAMP(k, lanes) ((void)0)
#endif
	if (q == 0 && park.next_count) *park.next_count = 0u;      // the queue counter of the march after this one
	// a lane's march ends in begin, probe or steps; its results are stored in one place, here
	MarchEnd end = q < M.lanes() ? M.begin(L, q) : MARCH_NO_RAY;
	for (;;) {
		if (end != MARCH_GOES_ON) {
			if (end != MARCH_NO_RAY) M.finish(L, end);
			L.m.phase = LANE_IDLE;
			end = MARCH_GOES_ON;
		}
		const uint32_t n_probe = (uint32_t)__popcll(__ballot(L.m.phase == LANE_PROBE));
		const uint32_t n_step = (uint32_t)__popcll(__ballot(L.m.phase == LANE_STEP));
		if (!(n_probe | n_step)) break;
		if (n_step) {
			if (L.m.phase == LANE_STEP) end = M.steps(L);
			SRF_MARCH_STAMP(0, n_step);
		} else {
			if (L.m.phase == LANE_PROBE) end = M.probe(L);
			// one of the wavefront's last few rays, crawling: it carries on in k_march_wide
			if (n_probe <= park.max_lanes && end == MARCH_GOES_ON && L.m.phase == LANE_PROBE && L.m.crawl >= park.min_crawl) {
				const uint32_t slot = atomicAdd(park.count, 1u);
				if (slot < park.capacity) { ((typename March::Lane*)park.slots)[slot] = L; L.m.phase = LANE_IDLE; }
				else L.m.crawl = 0;      // the queue is full: the ray stays
			}
			SRF_MARCH_STAMP(1, n_probe);
		}
	}
#ifdef SRF_KERNEL_TIMING
	if (threadIdx.x == 0) {
		for (int k = 0; k < 6; ++k) atomicAdd(&g_march_timing[k], t_acc_[k]);
		atomicAdd(&g_march_timing[6], 1ull);
		atomicAdd(&g_march_timing[7], clock64() - t_first_);
		atomicMax(&g_march_timing[8], wall_clock64() - w_first_);
	}
#endif
}

// the march and, behind it, the wide march of the rays it parked
template <class March>
static int launch_march(const March& M, srf_sampler* s, hipStream_t st) {
	const uint32_t n = M.lanes();
	MarchPark park;
	park.capacity = s->march_park_all ? n : n / 8u + 64u;
	park.max_lanes = s->march_park_all ? 64u : PARK_MAX_LANES;
	park.min_crawl = s->march_park_all ? 1u : PARK_CRAWL;
	int rc = s->park_ws.reserve((size_t)park.capacity * sizeof(typename March::Lane));
	if (rc != SRF_OK) return rc;
	if (!s->park_counts) {
		SRF_HIP(hipMalloc((void**)&s->park_counts, 256));
		SRF_HIP(hipMemset(s->park_counts, 0, 256));
	}
	park.slots = s->park_ws.ptr;
	park.count = s->park_counts + (s->park_turn & 1u);
	park.next_count = s->park_counts + ((s->park_turn + 1u) & 1u);
	++s->park_turn;
	hipLaunchKernelGGL(k_march_lanes<March>, dim3(div_up(n, 64u)), dim3(64), 0, st, M, park);
	hipLaunchKernelGGL(k_march_wide<March>, dim3(park.capacity < 4096u ? park.capacity : 4096u), dim3(64), 0, st, M, park);
#ifdef SRF_KERNEL_TIMING
	unsigned long long h[16], zero[16] = {0};
	if (hipStreamSynchronize(st) != hipSuccess || hipMemcpyFromSymbol(h, HIP_SYMBOL(g_march_timing), sizeof(h)) != hipSuccess) return SRF_OK;
	(void)hipMemcpyToSymbol(HIP_SYMBOL(g_march_timing), zero, sizeof(zero));
	const double nw = (double)(h[6] ? h[6] : 1);
	fprintf(stderr, "march of %u lanes: wavefront lifetime %.0f cycles mean, %.1f us longest\n", M.lanes(), (double)h[7] / nw, (double)h[8] / 100.0);
	const char* name[2] = {"step", "probe"};
	for (int k = 0; k < 2; ++k)
		fprintf(stderr, "march %-5s: %.0f cycles per wavefront, %.1f rounds, %.0f cycles per round, %.1f lanes per round\n", name[k],
		        (double)h[k] / nw, (double)h[2 + k] / nw, h[2 + k] ? (double)h[k] / (double)h[2 + k] : 0.0, h[2 + k] ? (double)h[4 + k] / (double)h[2 + k] : 0.0);
	{ uint32_t n_parked = 0; if (hipMemcpy(&n_parked, park.count, 4, hipMemcpyDeviceToHost) == hipSuccess) fprintf(stderr, "march parked %u rays (capacity %u)\n", n_parked, park.capacity); }
#endif
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

// the stretch of every ray inside a sphere; a ray that misses it gets the empty stretch (+inf, -inf).  24 B in, 8 B out a ray.
__global__ void __launch_bounds__(256) k_ray_sphere_bounds(uint32_t n_rays, const float* __restrict__ rays, Float4 sphere, float* __restrict__ t_near, float* __restrict__ t_far) {
	const uint32_t i = blockIdx.x * 256u + threadIdx.x;
	if (i >= n_rays) return;
	const float c[4] = {sphere.x, sphere.y, sphere.z, sphere.w};
	const SphereSpan sp = sphere_ray_span(c, ld3(rays + 6 * (size_t)i), ld3(rays + 6 * (size_t)i + 3));
	t_near[i] = sp.hit ? sp.t0 : srf_u2f(0x7f800000u);
	t_far[i] = sp.hit ? sp.t1 : srf_u2f(0xff800000u);
}

template <bool HALF>
__global__ void __launch_bounds__(256) k_field_eval(Params P, uint32_t n, const float* __restrict__ coords, FieldArgs F, void* __restrict__ out, uint32_t width,
                                                    const uint32_t* __restrict__ n_dev) {
	if (n_dev) n = *n_dev;
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n) field_eval_body<HALF>(i, P, coords, F, out, width);
}

// the sampler's empty-space table when it matches the bitfield, an empty one otherwise
static SkipTable sampler_skip_table(const srf_sampler* s) {
	return skip_table_for(s->P, s->skip_valid ? s->skip_dist : nullptr);
}

static MarchGrid sampler_march_grid(const srf_sampler* s) {
	MarchGrid G;
	G.P = s->P;
	G.bitfield = s->P.use_grid ? s->density_grid_bitfield : nullptr;
	G.skip = sampler_skip_table(s);
	return G;
}

static void fill_pixel_args(PixelArgs& A, const Params& P, const int32_t resolution[2], const float focal_length[2],
                            const float principal_point[2], const float camera_matrix_host[12], uint32_t spp) {
	for (int a = 0; a < 2; ++a) { A.res[a] = resolution[a]; A.focal[a] = focal_length[a]; A.pp[a] = principal_point[a]; }
	memcpy(A.cam.m, camera_matrix_host, sizeof(A.cam.m));
	ld_random_pixel_offset(P.snap_render ? 0u : spp, A.offset);
}

static int check_dataset(const srf_dataset* ds) {
	SRF_REQUIRE(ds, "NULL dataset");
	SRF_REQUIRE(ds->n_images > 0 && ds->xforms, "dataset has no camera matrices");
	SRF_REQUIRE(ds->image_resolution[0] > 0 && ds->image_resolution[1] > 0, "dataset resolution must be positive");
	SRF_REQUIRE(ds->focal_length[0] != 0.f && ds->focal_length[1] != 0.f, "dataset focal length must be non-zero");
	return SRF_OK;
}

} // namespace srf

using namespace srf;

extern "C" {

int srf_sampler_sample_coords_from_dataset(srf_sampler_t* s, uint32_t n_rays, uint32_t n_rays_shift, uint32_t n_coords,
                                           const srf_dataset* dataset, float* rays, float* rays_rgba,
                                           uint32_t* n_rays_counter, uint32_t* ray_coord_indices, float* coords,
                                           uint32_t* n_coords_counter, srf_pcg32 rng,
                                           float* sample_t, float* sample_dt, uint32_t* sample_cell, void* stream) {
	SRF_REQUIRE(s, "srf_sampler_sample_coords_from_dataset: NULL sampler");
	int rc = check_dataset(dataset);
	if (rc != SRF_OK) return rc;
	SRF_REQUIRE(rays && rays_rgba && n_rays_counter && ray_coord_indices && n_coords_counter, "srf_sampler_sample_coords_from_dataset: NULL output");
	SRF_REQUIRE(!s->P.use_grid || s->density_grid_bitfield, "srf_sampler_sample_coords_from_dataset: sampler has no bitfield");
	if (n_rays == 0) return SRF_OK;
	hipStream_t st = (hipStream_t)stream;
	const size_t n = n_rays;
	const size_t off_state = 0;
	const size_t off_counts = align_up(off_state + n * sizeof(TrainRay), 256);
	const size_t off_base = align_up(off_counts + n * 4, 256);
	const size_t off_keep = align_up(off_base + n * 4, 256);
	const size_t off_ridx = align_up(off_keep + n * 4, 256);
	const size_t off_scan = align_up(off_ridx + n * 4, 256);
	// step log: enough words for the marching-step bound of disparity stepping (n_max_steps plus start jitter and the
	// final clamp to the far plane); rays that take more steps fall back to a full second march
	uint32_t log_words = s->P.use_grid ? (s->P.n_max_steps + 64 + 31) / 32 : 0;
	if (log_words > LOG_MAX_WORDS) log_words = LOG_MAX_WORDS;
	const size_t off_log = align_up(off_scan + train_offset_scratch_bytes(n_rays), 256);
	// marching order: chunks of rays sorted by (image, pixel tile)
	constexpr bool sort_rays = true;
	const size_t off_order = align_up(off_log + (size_t)log_words * n * 8, 256);
	// rays that exhaust their probe budget are parked and finished by the wide march (0 = never)
	const uint32_t probe_budget = s->count_probe_budget;
	const uint32_t parked_capacity = probe_budget ? (n_rays / 8u > 4096u ? n_rays / 8u : 4096u) : 0u;
	const size_t off_parked = align_up(off_order + (sort_rays ? n * 4 : 0), 256);
	const size_t off_parked_count = align_up(off_parked + (size_t)parked_capacity * sizeof(ParkedRay), 256);
	rc = s->ws.reserve(off_parked_count + 256);
	if (rc != SRF_OK) return rc;
	char* w = (char*)s->ws.ptr;
	TrainRay* state = (TrainRay*)(w + off_state);
	uint32_t* counts = (uint32_t*)(w + off_counts);
	uint32_t* base = (uint32_t*)(w + off_base);
	uint32_t* keep = (uint32_t*)(w + off_keep);
	uint32_t* ridx = (uint32_t*)(w + off_ridx);
	void* scan = w + off_scan;
	StepLog log;
	log.bits = log_words ? (uint32_t*)(w + off_log) : nullptr;
	log.t0 = log_words ? (float*)(w + off_log + (size_t)log_words * n * 4) : nullptr;
	log.stride = n_rays;
	log.words = log_words;

	DatasetArgs ds;
	ds.n_images = dataset->n_images;
	for (int a = 0; a < 2; ++a) { ds.res[a] = dataset->image_resolution[a]; ds.focal[a] = dataset->focal_length[a]; ds.pp[a] = dataset->principal_point[a]; }
	ds.xforms = dataset->xforms; ds.images = dataset->images; ds.prob = dataset->sampling_probability;
	Pcg32 r; r.state = rng.state; r.inc = rng.inc;
	const uint8_t* bitfield = s->P.use_grid ? s->density_grid_bitfield : nullptr;

	CountArgs ca;
	ca.n_rays = n_rays; ca.n_rays_shift = n_rays_shift; ca.ds = ds; ca.bitfield = bitfield; ca.rng = r;
	ca.state = state; ca.counts = counts; ca.log = log;
	ca.skip = sampler_skip_table(s);
	ca.probe_budget = probe_budget;
	ca.park_lanes = s->count_park_lanes;
	ca.parked = (ParkedRay*)(w + off_parked);
	ca.parked_capacity = parked_capacity;
	ca.parked_count = (uint32_t*)(w + off_parked_count);
	if (probe_budget) hipLaunchKernelGGL(k_zero_word, dim3(1), dim3(1), 0, st, ca.parked_count);
	// rays per wavefront: enough for lanes that finish early to pick up more work, few enough for several wavefronts per SIMD
	// (settled by measurement on the 2^20-ray training batch: one ray a lane; a probe round once every lane waits for one or the stepping
	// lanes are outnumbered 32 to 1 — 4: 1.52, 8: 1.41, 16: 1.33, 24: 1.30, 32: 1.29, 48: 1.31, 64: 1.37 ms; stepping rounds are cheap since
	// whole stretches are taken in closed form, so the probes wait for nearly all of them; new rays are begun 32 at a time)
	constexpr uint32_t rays_per_wave = 64, probe_quorum = 64, begin_quorum = 32, probe_ratio = 32;
	const uint32_t* order = nullptr;
	if (sort_rays) {
		uint32_t* order_out = (uint32_t*)(w + off_order);
		hipLaunchKernelGGL(k_ray_order, dim3(div_up(n_rays, RAY_CHUNK)), dim3(RAY_CHUNK_BINS), 0, st, s->P, ca, order_out);
		SRF_LAUNCH_CHECK();
		order = order_out;
	}
	unsigned long long* timing = nullptr;
#ifdef SRF_KERNEL_TIMING
	static unsigned long long* timing_buf = nullptr;
	if (!timing_buf) { SRF_HIP(hipMalloc((void**)&timing_buf, (1024 * 16 + 192) * 8)); SRF_HIP(hipMemset(timing_buf, 0, (1024 * 16 + 192) * 8)); }
	timing = timing_buf;
#endif
	if (s->P.sphere[3] > 0.f)
		hipLaunchKernelGGL(k_train_count<true>, dim3(div_up(n_rays, rays_per_wave)), dim3(64), 0, st, s->P, ca, rays_per_wave, probe_quorum, begin_quorum, probe_ratio, order, timing);
	else
		hipLaunchKernelGGL(k_train_count<false>, dim3(div_up(n_rays, rays_per_wave)), dim3(64), 0, st, s->P, ca, rays_per_wave, probe_quorum, begin_quorum, probe_ratio, order, timing);
#ifdef SRF_KERNEL_TIMING
	{
		static unsigned long long hs[1024 * 16 + 192];
		unsigned long long h[12] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
		SRF_HIP(hipStreamSynchronize(st));
		SRF_HIP(hipMemcpy(hs, timing, sizeof(hs), hipMemcpyDeviceToHost));
		SRF_HIP(hipMemset(timing, 0, sizeof(hs)));
		for (int i = 0; i < 1024; ++i) for (int k = 0; k < 11; ++k) h[k] += hs[i * 16 + k];
		for (int i = 0; i < 1024; ++i) h[11] = hs[i * 16 + 11] > h[11] ? hs[i * 16 + 11] : h[11];
		const double nw = (double)div_up(n_rays, rays_per_wave);
		fprintf(stderr, "count march wavefront lifetime: %.0f cycles = %.1f us mean, %.1f us max\n", (double)h[9] / nw, (double)h[10] / nw / 100.0, (double)h[11] / 100.0);
		fprintf(stderr, "count march lifetime histogram (100 us buckets):");
		for (int k = 0; k < 48; ++k) fprintf(stderr, " %llu", hs[1024 * 16 + k]);
		fprintf(stderr, "\ncount march probe-round histogram (buckets of 64):");
		for (int k = 0; k < 48; ++k) fprintf(stderr, " %llu", hs[1024 * 16 + 48 + k]);
		fprintf(stderr, "\ncount march step-round histogram (buckets of 64):");
		for (int k = 0; k < 48; ++k) fprintf(stderr, " %llu", hs[1024 * 16 + 96 + k]);
		fprintf(stderr, "\n");
		{ const unsigned long long* q = hs + 1024 * 16 + 144; if (q[0]) fprintf(stderr, "count march slow wavefronts: %llu, step rounds %.0f (%.1f lanes, %.0f cycles each), probe rounds %.0f (%.1f lanes, %.0f cycles each)\n",
			q[0], (double)q[1] / q[0], (double)q[3] / (q[1] ? q[1] : 1), (double)q[5] / (q[1] ? q[1] : 1), (double)q[2] / q[0], (double)q[4] / (q[2] ? q[2] : 1), (double)q[6] / (q[2] ? q[2] : 1)); }
		const char* name[3] = {"step", "probe", "begin"};
		for (int k = 0; k < 3; ++k)
			fprintf(stderr, "count march %-5s: %.0f cycles per wavefront, %.1f rounds, %.0f cycles per round, %.1f lanes per round\n", name[k],
			        (double)h[k] / nw, (double)h[3 + k] / nw, h[3 + k] ? (double)h[k] / (double)h[3 + k] : 0.0, h[3 + k] ? (double)h[6 + k] / (double)h[3 + k] : 0.0);
		uint32_t n_parked = 0;
		if (probe_budget) SRF_HIP(hipMemcpy(&n_parked, ca.parked_count, 4, hipMemcpyDeviceToHost));
		fprintf(stderr, "count march parked rays: %u (capacity %u)\n", n_parked, parked_capacity);
	}
#endif
	SRF_LAUNCH_CHECK();
	if (probe_budget) {
		const uint32_t wide_blocks = parked_capacity < 4096u ? parked_capacity : 4096u;
		if (s->P.sphere[3] > 0.f) hipLaunchKernelGGL(k_train_count_wide<true>, dim3(wide_blocks), dim3(128), 0, st, s->P, ca);
		else hipLaunchKernelGGL(k_train_count_wide<false>, dim3(wide_blocks), dim3(128), 0, st, s->P, ca);
		SRF_LAUNCH_CHECK();
	}
	const uint32_t n_tiles = div_up(n_rays, OFFSET_TILE);
	TrainOffsetScratch os;
	os.tile_counts = (uint32_t*)scan; os.tile_kept = os.tile_counts + n_tiles; os.entry = os.tile_kept + n_tiles;
	hipLaunchKernelGGL(k_train_tile_counts, dim3(n_tiles), dim3(OFFSET_THREADS), 0, st, n_rays, (const uint32_t*)counts, os, (const uint32_t*)n_coords_counter, (const uint32_t*)n_rays_counter);
	hipLaunchKernelGGL(k_train_bases, dim3(n_tiles), dim3(OFFSET_THREADS), 0, st, n_rays, n_coords, (const uint32_t*)counts, os, base, keep, n_coords_counter);
	hipLaunchKernelGGL(k_train_ray_indices, dim3(n_tiles), dim3(OFFSET_THREADS), 0, st, n_rays, (const uint32_t*)keep, os, ridx, n_rays_counter);
	SRF_LAUNCH_CHECK();
	hipLaunchKernelGGL(k_train_write, dim3(div_up(n_rays, 64)), dim3(64), 0, st, s->P, n_rays, ds, bitfield, (const TrainRay*)state,
	                   (const uint32_t*)counts, (const uint32_t*)base, (const uint32_t*)keep, (const uint32_t*)ridx,
	                   rays, rays_rgba, ray_coord_indices, coords, sample_t, sample_dt, sample_cell, log);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int srf_sampler_set_ray_sphere_bound(srf_sampler_t* s, const float center[3], float radius) {
	SRF_REQUIRE(s, "srf_sampler_set_ray_sphere_bound: NULL sampler");
	SRF_REQUIRE(radius <= 0.f || center, "srf_sampler_set_ray_sphere_bound: NULL center");
	SRF_REQUIRE(radius == radius && radius < 3.0e38f, "srf_sampler_set_ray_sphere_bound: radius must be finite");
	for (int a = 0; a < 3; ++a) s->P.sphere[a] = radius > 0.f ? center[a] : 0.f;
	s->P.sphere[3] = radius > 0.f ? radius : 0.f;
	return SRF_OK;
}

int srf_ray_sphere_bounds(uint32_t n_rays, const float* rays, const float center[3], float radius, float* t_near, float* t_far, void* stream) {
	SRF_REQUIRE(center && radius > 0.f, "srf_ray_sphere_bounds: needs a center and a positive radius");
	if (n_rays == 0) return SRF_OK;
	SRF_REQUIRE(rays && t_near && t_far, "srf_ray_sphere_bounds: NULL buffer");
	hipLaunchKernelGGL(k_ray_sphere_bounds, dim3(div_up(n_rays, 256)), dim3(256), 0, (hipStream_t)stream, n_rays, rays,
	                   mk4(center[0], center[1], center[2], radius), t_near, t_far);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int srf_sampler_generate_rays_from_camera_matrix(srf_sampler_t* s, const int32_t resolution[2], const float focal_length[2],
                                                 const float principal_point[2], const float camera_matrix_host[12],
                                                 srf_ray_payload* payload, uint32_t spp, void* stream) {
	SRF_REQUIRE(s && resolution && focal_length && principal_point && camera_matrix_host && payload, "srf_sampler_generate_rays_from_camera_matrix: NULL argument");
	SRF_REQUIRE(resolution[0] > 0 && resolution[1] > 0, "srf_sampler_generate_rays_from_camera_matrix: resolution must be positive");
	hipStream_t st = (hipStream_t)stream;
	PixelArgs A;
	fill_pixel_args(A, s->P, resolution, focal_length, principal_point, camera_matrix_host, spp);
	const dim3 threads(16, 8, 1);
	const dim3 blocks(div_up((uint32_t)resolution[0], threads.x), div_up((uint32_t)resolution[1], threads.y), 1);
	hipLaunchKernelGGL(k_init_rays, blocks, threads, 0, st, s->P, A, payload);
	SRF_LAUNCH_CHECK();
	const uint32_t n = (uint32_t)resolution[0] * (uint32_t)resolution[1];
	AdvanceMarch M;
	M.G = sampler_march_grid(s); M.n_rays = n; M.spp = spp; M.payloads = payload;
	return launch_march(M, s, st);
}

} // extern "C"

namespace srf {
int generate_coords_paced(srf_sampler* s, uint32_t bound, const RoundWords* round, srf_ray_payload* payloads, float* coords, hipStream_t stream) {
	if (bound == 0) return SRF_OK;
	CoordsMarch M;
	M.G = sampler_march_grid(s); M.n_rays = bound; M.n_steps = FRAME_MAX_STEPS; M.payloads = payloads; M.coords = coords;
	M.round = &round->n_alive;      // {n_alive, n_steps}
	return launch_march(M, s, stream);
}
} // namespace srf

extern "C" {

int srf_sampler_generate_coords_from_rays(srf_sampler_t* s, uint32_t n_rays, uint32_t n_steps,
                                          srf_ray_payload* payloads, float* coords, void* stream) {
	SRF_REQUIRE(s, "srf_sampler_generate_coords_from_rays: NULL sampler");
	if (n_rays == 0 || n_steps == 0) return SRF_OK;
	SRF_REQUIRE(payloads && coords, "srf_sampler_generate_coords_from_rays: NULL buffer");
	CoordsMarch M;
	M.G = sampler_march_grid(s); M.n_rays = n_rays; M.n_steps = n_steps; M.payloads = payloads; M.coords = coords;
	return launch_march(M, s, (hipStream_t)stream);
}

int srf_field_eval(const srf_sampler_t* s, const srf_field* field, uint32_t n_coords, const float* coords,
                   void* rgbsigma, int32_t dtype, uint32_t padded_output_width, void* stream) {
	return srf_field_eval_counted(s, field, nullptr, n_coords, coords, rgbsigma, dtype, padded_output_width, stream);
}

int srf_field_eval_counted(const srf_sampler_t* s, const srf_field* field, const uint32_t* n_coords_dev, uint32_t n_coords, const float* coords,
                           void* rgbsigma, int32_t dtype, uint32_t padded_output_width, void* stream) {
	SRF_REQUIRE(s && field && field->table, "srf_field_eval: NULL argument");
	SRF_REQUIRE(field->table_size && !(field->table_size & (field->table_size - 1)), "srf_field_eval: table_size must be a power of two");
	SRF_REQUIRE(padded_output_width >= 4, "srf_field_eval: padded_output_width must be >= 4");
	SRF_REQUIRE(dtype == SRF_DTYPE_F16 || dtype == SRF_DTYPE_F32, "srf_field_eval: unknown dtype");
	SRF_REQUIRE(s->P.griddist_type == SRF_GRID_WARPED_EXP || s->P.griddist_type == SRF_GRID_WARPED_RECIPROCAL, "srf_field_eval: needs a warped-space grid type");
	if (n_coords == 0) return SRF_OK;
	SRF_REQUIRE(coords && rgbsigma, "srf_field_eval: NULL buffer");
	FieldArgs F; F.table = field->table; F.mask = field->table_size - 1; F.seed = field->seed;
	if (dtype == SRF_DTYPE_F16)
		hipLaunchKernelGGL(k_field_eval<true>, dim3(div_up(n_coords, 256)), dim3(256), 0, (hipStream_t)stream, s->P, n_coords, coords, F, rgbsigma, padded_output_width, n_coords_dev);
	else
		hipLaunchKernelGGL(k_field_eval<false>, dim3(div_up(n_coords, 256)), dim3(256), 0, (hipStream_t)stream, s->P, n_coords, coords, F, rgbsigma, padded_output_width, n_coords_dev);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int srf_render_frame_fused(srf_sampler_t* s, const srf_marcher_t* m, const srf_field* field,
                           const int32_t resolution[2], const float focal_length[2], const float principal_point[2],
                           const float camera_matrix_host[12], uint32_t spp, float* frame_buffer, uint32_t* n_samples, void* stream) {
	SRF_REQUIRE(s && m && field && field->table && resolution && focal_length && principal_point && camera_matrix_host && frame_buffer,
	            "srf_render_frame_fused: NULL argument");
	SRF_REQUIRE(field->table_size && !(field->table_size & (field->table_size - 1)), "srf_render_frame_fused: table_size must be a power of two");
	SRF_REQUIRE(resolution[0] > 0 && resolution[1] > 0, "srf_render_frame_fused: resolution must be positive");
	SRF_REQUIRE(s->P.griddist_type == SRF_GRID_WARPED_EXP || s->P.griddist_type == SRF_GRID_WARPED_RECIPROCAL, "srf_render_frame_fused: needs a warped-space grid type");
	PixelArgs A;
	fill_pixel_args(A, s->P, resolution, focal_length, principal_point, camera_matrix_host, spp);
	FusedMarch M;
	M.G = sampler_march_grid(s); M.A = A; M.spp = spp;
	M.F.table = field->table; M.F.mask = field->table_size - 1; M.F.seed = field->seed;
	M.thr = m->cfg.transmittance_threshold; M.to_linear = m->cfg.train_in_linear_color ? 0 : 1;
	M.frame = frame_buffer; M.n_samples = n_samples;
	return launch_march(M, s, (hipStream_t)stream);
}

} // extern "C"
