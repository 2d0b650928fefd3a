// OccupancySampler object and occupancy-grid maintenance:
// sample_positions_from_grid, update_grid (splat + decayed max), update_grid_bitfield
// (cascade-0 mean, threshold to bits, max-pool into coarser cascades).
#include <stdlib.h>
#include <hipcub/hipcub.hpp>
#include "srf_internal.h"
#include "srf_bodies.h"
#include "srf_wave.h"

namespace srf {

__global__ void k_fill_u32(uint32_t* __restrict__ p, size_t n, uint32_t v) {
	size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
	const size_t stride = (size_t)gridDim.x * blockDim.x;
	for (; i < n; i += stride) p[i] = v;
}

int fill_u32(void* p, size_t n_words, uint32_t v, hipStream_t stream) {
	if (n_words == 0) return SRF_OK;
	const uint32_t blocks = (uint32_t)(n_words / 256 + 1 > 4096 ? 4096 : n_words / 256 + 1);
	hipLaunchKernelGGL(k_fill_u32, dim3(blocks), dim3(256), 0, stream, (uint32_t*)p, n_words, v);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

// occupancy_sampler.cu:12-102 — mark_untrained_density_grid: one thread per cell; the cameras pass through LDS a batch at a time, and a
// workgroup stops as soon as every one of its cells has been seen by some camera
constexpr uint32_t MASK_CAMERAS_PER_BATCH = 128;
__global__ void __launch_bounds__(256) k_mark_untrained(Params P, uint32_t n_total, uint32_t n_images, float focal_x, float focal_y, float half_res_x, float half_res_y,
                                                        const float* __restrict__ xforms, float* __restrict__ grid_out) {
	__shared__ float cams[MASK_CAMERAS_PER_BATCH * 12];
	const uint32_t i = blockIdx.x * 256u + threadIdx.x;
	Vec3 centre = mk3(0.f, 0.f, 0.f);
	float radius = 0.f;
	bool seen = i >= n_total;      // threads past the end have nothing to look for
	if (i < n_total) mask_cell(i, P, &centre, &radius);
	for (uint32_t first = 0; first < n_images; first += MASK_CAMERAS_PER_BATCH) {
		const uint32_t n = n_images - first < MASK_CAMERAS_PER_BATCH ? n_images - first : MASK_CAMERAS_PER_BATCH;
		for (uint32_t k = threadIdx.x; k < n * 12u; k += 256u) cams[k] = xforms[(size_t)first * 12u + k];
		__syncthreads();
		for (uint32_t j = 0; j < n && !seen; ++j) seen = mask_camera_sees(&cams[j * 12u], centre, radius, focal_x, focal_y, half_res_x, half_res_y);
		if (__syncthreads_and(seen ? 1 : 0)) break;
	}
	if (i < n_total) grid_out[i] = seen ? 0.f : -1.f;
}

__global__ void __launch_bounds__(256) k_generate_grid_samples(Params P, uint32_t n_elements, Pcg32 rng, uint32_t step,
                                                                const float* __restrict__ grid_in, float thresh,
                                                                float* __restrict__ positions, uint32_t* __restrict__ indices, const uint32_t* __restrict__ above,
                                                                uint32_t tries_at_once, uint32_t first, const uint32_t* __restrict__ above_summary) {
	// the generator's skip-ahead maps, one hexadecimal digit each, worked out once per workgroup
	__shared__ uint64_t skip_m[128], skip_p[128];
	if (threadIdx.x < 128) pcg_skip16_entry(rng, threadIdx.x, &skip_m[threadIdx.x], &skip_p[threadIdx.x]);
	__syncthreads();
	// a workgroup takes several runs of 256 points: the launch is then a few thousand groups instead of one per run
	// the points from `first` on
	const uint32_t n_runs = (n_elements - first + 255u) / 256u;
	for (uint32_t run = blockIdx.x; run < n_runs; run += gridDim.x) {
		const uint32_t i = first + run * 256u + threadIdx.x;
		if (i < n_elements) grid_sample_body(i, P, n_elements, rng, step, grid_in, thresh, positions, indices, above, nullptr, tries_at_once, skip_m, skip_p, above_summary);
	}
}

// The same draw with the points dealt to the threads in the order of their first candidate cell.  Point i tries the cells
// ((i + step n) A + j B + C) mod n_cells, j = 0..9, of a random cascade: with n_cells a power of two, A odd, the points
// whose (i + step n) A mod n_cells is v, v + 1, ... try neighbouring cells at every j, so consecutive threads read the
// same few cache lines (one group per cascade) instead of 64 lines scattered over the grid.  Thread t = m n_cells + v
// takes the m-th point with that v; which thread draws a point changes nothing in what is drawn.  The results go to a
// staging array in thread order (16 bytes each, contiguous per wavefront); k_grid_samples_to_point_order then has thread i
// fetch point i's record and write the outputs in their own order, so that neither kernel scatters its stores.
constexpr uint32_t DEAL_WINDOW_MAX = 1024;      // threads of a window of k_generate_grid_samples_by_cell, at most
// SPARSE: the launch covers a multiple of the cell count that the draw's points do not fill
template <bool SPARSE>
__global__ void __launch_bounds__(256) k_generate_grid_samples_by_cell(Params P, uint32_t n_elements, Pcg32 rng, uint32_t step,
                                                                        const float* __restrict__ grid_in, float thresh,
                                                                        Float4* __restrict__ staged, const uint32_t* __restrict__ above,
                                                                        uint32_t tries_at_once, uint32_t a_inverse, uint32_t log2_cells,
                                                                        float* __restrict__ positions, uint32_t* __restrict__ indices, uint32_t first_thread,
                                                                        uint32_t n_windows, uint32_t per) {
	__shared__ uint64_t skip_m[128], skip_p[128];
	if (threadIdx.x < 128) pcg_skip16_entry(rng, threadIdx.x, &skip_m[threadIdx.x], &skip_p[threadIdx.x]);
	__syncthreads();
	// A workgroup takes several windows of `per` x 256 threads (so that the tables above are worked out a few thousand times, not
	// once per 256 points).  In a multiple of the cell count that the points do not fill only some of the threads have a point,
	// scattered evenly over it: the window's threads that have one are listed first, and the workgroup's lanes then take the listed
	// ones side by side.
	__shared__ uint16_t live[DEAL_WINDOW_MAX];
	__shared__ uint32_t n_live;
	if (threadIdx.x == 0) n_live = 0u;
	__syncthreads();
	const uint32_t mask = P.n_cells - 1u;
	auto point_of = [&](uint64_t t) -> uint64_t {
		const uint32_t v = (uint32_t)t & mask, m = (uint32_t)(t >> log2_cells);
		const uint32_t u = (v * a_inverse) & mask;                      // (i + step n) mod n_cells
		return (uint64_t)((u - step * n_elements) & mask) + ((uint64_t)m << log2_cells);
	};
	auto draw = [&](uint64_t t) {
		Vec3 pos;
		uint32_t idx;
		grid_sample_point((uint32_t)point_of(t), P, n_elements, rng, step, grid_in, thresh, &pos, &idx, above, nullptr, tries_at_once, skip_m, skip_p);
		// staged == NULL: the caller takes the points in this order (entry t of its arrays is thread t's point)
		if (staged) staged[t - first_thread] = mk4(pos.x, pos.y, pos.z, srf_u2f(idx));
		else { st3(positions + 3 * (size_t)t, pos); indices[t] = idx; }
	};
	for (uint32_t win = blockIdx.x; win < n_windows; win += gridDim.x) {
		const uint64_t t0 = (uint64_t)first_thread + (uint64_t)win * (per * 256u);      // staged holds the threads from first_thread on
		if (!SPARSE) {                       // every thread has a point
			for (uint32_t q = 0; q < per; ++q) draw(t0 + q * 256u + threadIdx.x);
			continue;
		}
		uint32_t mine = 0, count = 0;
		for (uint32_t q = 0; q < per; ++q) if (point_of(t0 + q * 256u + threadIdx.x) < n_elements) { mine |= 1u << q; ++count; }
		uint32_t slot = count ? atomicAdd(&n_live, count) : 0u;
		for (uint32_t q = 0; q < per; ++q) if (mine >> q & 1u) live[slot++] = (uint16_t)(q * 256u + threadIdx.x);
		__syncthreads();
		const uint32_t n = n_live;
		for (uint32_t k = threadIdx.x; k < n; k += 256u) draw(t0 + live[k]);
		__syncthreads();
		if (threadIdx.x == 0) n_live = 0u;
		__syncthreads();
	}
}

__global__ void __launch_bounds__(256) k_grid_samples_to_point_order(uint32_t n_cells, uint32_t n_elements, uint32_t step, uint32_t log2_cells,
                                                                      const Float4* __restrict__ staged, float* __restrict__ positions, uint32_t* __restrict__ indices,
                                                                      uint32_t first) {
	// the points from `first` (a multiple of the cell count) on; staged holds the threads from `first` on
	const uint32_t i = first + blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= n_elements) return;
	const uint32_t mask = n_cells - 1u;
	const uint32_t v = (((i + step * n_elements) & mask) * 56924617u) & mask;      // the inverse of the dealing above
	const Float4 r = staged[((uint64_t)(i >> log2_cells) << log2_cells) - first + v];
	st3(positions + 3 * (size_t)i, mk3(r.x, r.y, r.z));
	indices[i] = srf_f2u(r.w);
}

// one bit per cell for each of two thresholds: bit (i & 31) of word (i >> 5) is grid[i] > thresh; 64 cells per wavefront round.
// summary_a (cleared by the caller): bit (w & 31) of word (w >> 5) is set where word w of above_a has a bit that is not set
__global__ void __launch_bounds__(256) k_threshold_bits(const float* __restrict__ grid, uint32_t n_total, float thresh_a, float thresh_b,
                                                         uint32_t* __restrict__ above_a, uint32_t* __restrict__ above_b, uint32_t* __restrict__ summary_a) {
	constexpr uint32_t ROUNDS = 4;      // 64-cell rounds a wavefront has in flight: four independent loads a lane
	const uint32_t lane = threadIdx.x & 63u;
	const uint32_t stride = gridDim.x * blockDim.x * ROUNDS;
	for (uint32_t first = ((blockIdx.x * blockDim.x + threadIdx.x) - lane) * ROUNDS; first < n_total; first += stride) {   // uniform per wavefront
		float v[ROUNDS];
		#pragma unroll
		for (uint32_t k = 0; k < ROUNDS; ++k) { const uint32_t i = first + k * 64u + lane; v[k] = i < n_total ? grid[i] : 0.f; }
		#pragma unroll
		for (uint32_t k = 0; k < ROUNDS; ++k) {
			const uint32_t base = first + k * 64u;
			if (base >= n_total) break;
			const uint32_t i = base + lane;
			const uint64_t ma = __ballot(i < n_total && v[k] > thresh_a), mb = __ballot(i < n_total && v[k] > thresh_b);
			if (lane == 0) {
				above_a[base >> 5] = (uint32_t)ma; above_b[base >> 5] = (uint32_t)mb;
				const uint32_t w = base >> 5;      // (even: both words of the round share a summary word)
				const uint32_t some = ((uint32_t)ma != 0xffffffffu ? 1u : 0u) | ((uint32_t)(ma >> 32) != 0xffffffffu ? 2u : 0u);
				if (some) atomicOr(&summary_a[w >> 5], some << (w & 31u));
			}
			if (lane == 32 && base + 32 < n_total) { above_a[(base >> 5) + 1] = (uint32_t)(ma >> 32); above_b[(base >> 5) + 1] = (uint32_t)(mb >> 32); }
		}
	}
}

// occupancy_sampler.cu:187-212 — non-negative floats order like their bit patterns, so the
// maximum is an unsigned integer atomic.
template <bool HALF>
__global__ void __launch_bounds__(256) k_splat_grid_samples(uint32_t n_elements, const uint32_t* __restrict__ indices, uint32_t width,
                                                             const void* __restrict__ densities, int act, float min_cone_stepsize,
                                                             float* __restrict__ grid_current) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= n_elements) return;
	const float sigma = act_density(net_load<HALF>(densities, (size_t)i * width), act);
	const float thickness = sigma * min_cone_stepsize;
	// the grid was cleared to zero before this launch: a zero cannot raise any cell (most samples of a trained scene)
	if (srf_f2u(thickness) != 0u) atomicMax((unsigned int*)&grid_current[indices[i]], srf_f2u(thickness));
}

// The same splat for large batches, without device-wide atomics.  The samples fall on random cells of a grid far larger
// than the caches, and a device atomic per sample runs at some 20 G/s whatever the locality.  Sorted by slab of
// SPLAT_SLAB_CELLS consecutive cells (the maximum does not depend on the order), each slab's samples are combined in
// LDS by one workgroup, which then writes the whole slab: that also clears the cells no sample fell on.
constexpr uint32_t SPLAT_SLAB_BITS = 13;
constexpr uint32_t SPLAT_SLAB_CELLS = 1u << SPLAT_SLAB_BITS;
constexpr uint32_t SPLAT_SORT_MIN = 1u << 22;    // batches below this go through the direct splat

template <bool HALF>
__global__ void __launch_bounds__(256) k_splat_values(uint32_t n_elements, uint32_t width, const void* __restrict__ densities, int act,
                                                       float min_cone_stepsize, uint32_t* __restrict__ thickness_bits) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= n_elements) return;
	const float sigma = act_density(net_load<HALF>(densities, (size_t)i * width), act);
	thickness_bits[i] = srf_f2u(sigma * min_cone_stepsize);
}

// first position in the sorted cell list whose slab is not below `slab`
__device__ inline uint32_t splat_lower_bound(const uint32_t* __restrict__ cells, uint32_t n, uint32_t slab) {
	uint32_t lo = 0, hi = n;
	while (lo < hi) {
		const uint32_t mid = lo + (hi - lo) / 2;
		if ((cells[mid] >> SPLAT_SLAB_BITS) < slab) lo = mid + 1; else hi = mid;
	}
	return lo;
}

__global__ void __launch_bounds__(256) k_splat_slabs(uint32_t n_elements, uint32_t n_total, const uint32_t* __restrict__ cells,
                                                      const uint32_t* __restrict__ thickness_bits, uint32_t* __restrict__ grid_current_bits) {
	__shared__ uint32_t tile[SPLAT_SLAB_CELLS];
	__shared__ uint32_t range[2];
	const uint32_t slab = blockIdx.x;
	for (uint32_t j = threadIdx.x; j < SPLAT_SLAB_CELLS; j += 256u) tile[j] = 0u;
	if (threadIdx.x < 2) range[threadIdx.x] = splat_lower_bound(cells, n_elements, slab + threadIdx.x);
	__syncthreads();
	for (uint32_t i = range[0] + threadIdx.x; i < range[1]; i += 256u) atomicMax(&tile[cells[i] & (SPLAT_SLAB_CELLS - 1u)], thickness_bits[i]);
	__syncthreads();
	const uint32_t first = slab << SPLAT_SLAB_BITS;
	for (uint32_t j = threadIdx.x; j < SPLAT_SLAB_CELLS; j += 256u) if (first + j < n_total) grid_current_bits[first + j] = tile[j];
}

// The same without a sorting library: a partition by slab made for this job, in two levels of at most 256 and 64 parts so that
// every level writes runs of some hundred bytes.  Which of a slab's samples comes first does not matter (the maximum does not depend
// on the order), so nothing has to be stable.  k_part_count counts the samples of every slab (a histogram in LDS, flushed once
// per workgroup); k_part_scan turns the counts into where each slab and each bucket of 64 slabs starts; k_part_pass<1> takes chunks
// of 8192 samples, computes their (cell, thickness) pairs, reserves the chunk's share of every bucket's positions with one device
// atomic per bucket, orders the pairs by bucket in LDS and writes them out run by run; k_part_pass<2> does the same by slab with the
// chunks of one bucket at a time.  k_part_slabs then combines every slab in LDS as k_splat_slabs does, knows each slab's range from
// the scan, and, where nothing else splats after it, applies the decay to the grid in the same pass (k_ema_grid's arithmetic).
constexpr uint32_t PART_SLAB_BITS = 14;                    // 16384 cells: 64 KB of LDS per workgroup in k_part_slabs
constexpr uint32_t PART_SLAB_CELLS = 1u << PART_SLAB_BITS;
constexpr uint32_t PART_BUCKET_BITS = 6;                   // slabs per bucket
constexpr uint32_t PART_BUCKET_SLABS = 1u << PART_BUCKET_BITS;
constexpr uint32_t PART_MAX_BUCKETS = 256;
constexpr uint32_t PART_MAX_SLABS = PART_MAX_BUCKETS * PART_BUCKET_SLABS;      // 16384 slabs = 2^28 cells
constexpr uint32_t PART_THREADS = 1024;
constexpr uint32_t PART_CHUNK = 8192, PART_PASS_THREADS = 1024, PART_PER_THREAD = PART_CHUNK / PART_PASS_THREADS;

__global__ void __launch_bounds__(PART_THREADS) k_part_count(uint32_t n, const uint32_t* __restrict__ indices, uint32_t n_total, uint32_t n_slabs, uint32_t* __restrict__ counts) {
	extern __shared__ uint32_t part_h[];
	for (uint32_t b = threadIdx.x; b < n_slabs; b += PART_THREADS) part_h[b] = 0u;
	__syncthreads();
	for (size_t i = (size_t)blockIdx.x * PART_THREADS + threadIdx.x; i < n; i += (size_t)gridDim.x * PART_THREADS) {
		const uint32_t c = indices[i];
		if (c < n_total) atomicAdd(&part_h[c >> PART_SLAB_BITS], 1u);
	}
	__syncthreads();
	for (uint32_t b = threadIdx.x; b < n_slabs; b += PART_THREADS) { const uint32_t v = part_h[b]; if (v) atomicAdd(&counts[b], v); }
}

// What the scan leaves: starts[s] = samples in slabs before s (starts[n_slabs] = all), slab_cursor = a copy that pass 2 advances;
// per bucket b: bucket_cursor[b] = starts[64 b] (advanced by pass 1), chunk_first[b] = chunks of 8192 in the buckets before b.
struct PartTables { uint32_t* starts; uint32_t* slab_cursor; uint32_t* bucket_cursor; uint32_t* chunk_first; };
__global__ void __launch_bounds__(PART_THREADS) k_part_scan(uint32_t n_slabs, uint32_t n_buckets, const uint32_t* __restrict__ counts, PartTables T) {
	__shared__ uint32_t sums[PART_THREADS];
	const uint32_t per = div_up(n_slabs, PART_THREADS);
	const uint32_t lo = threadIdx.x * per, hi = lo + per < n_slabs ? lo + per : n_slabs;
	uint32_t run = 0;
	for (uint32_t b = lo; b < hi; ++b) run += counts[b];
	sums[threadIdx.x] = run;
	__syncthreads();
	if (threadIdx.x == 0) {
		uint32_t acc = 0;
		for (uint32_t k = 0; k < PART_THREADS; ++k) { const uint32_t v = sums[k]; sums[k] = acc; acc += v; }
		T.starts[n_slabs] = acc;
	}
	__syncthreads();
	run = sums[threadIdx.x];
	for (uint32_t b = lo; b < hi; ++b) { T.starts[b] = run; T.slab_cursor[b] = run; run += counts[b]; }
	__syncthreads();
	// per bucket (starts were written by other threads of this workgroup: visible after the barrier)
	uint32_t my_chunks = 0;
	if (threadIdx.x < n_buckets) {
		const uint32_t b = threadIdx.x;
		const uint32_t s0 = b << PART_BUCKET_BITS, s1 = s0 + PART_BUCKET_SLABS < n_slabs ? s0 + PART_BUCKET_SLABS : n_slabs;
		const uint32_t first = ((volatile uint32_t*)T.starts)[s0], size = ((volatile uint32_t*)T.starts)[s1] - first;
		T.bucket_cursor[b] = first;
		my_chunks = div_up(size, PART_CHUNK);
	}
	sums[threadIdx.x] = my_chunks;
	__syncthreads();
	if (threadIdx.x == 0) {
		uint32_t chunks = 0;
		for (uint32_t b = 0; b < n_buckets; ++b) { T.chunk_first[b] = chunks; chunks += sums[b]; }
		T.chunk_first[n_buckets] = chunks;
	}
}

// One level of the partition.  LEVEL 1: input = the caller's arrays, part = bucket of the cell's slab, one chunk = 8192 consecutive
// samples.  LEVEL 2: input = pass 1's pairs, part = slab within the bucket, chunks numbered bucket by bucket (chunk_first).
template <int LEVEL, bool HALF>
__global__ void __launch_bounds__(PART_PASS_THREADS) k_part_pass(uint32_t n, const uint32_t* __restrict__ indices, uint32_t width, const void* __restrict__ densities, int act,
                                                                 float min_cone_stepsize, uint32_t n_total, uint32_t n_slabs, uint32_t n_buckets, PartTables T,
                                                                 const U2* __restrict__ in_pairs, U2* __restrict__ out_pairs) {
	__shared__ U2 stage[PART_CHUNK];
	__shared__ uint32_t hist[PART_MAX_BUCKETS], lstart[PART_MAX_BUCKETS + 1], gbase[PART_MAX_BUCKETS], fill[PART_MAX_BUCKETS];
	constexpr uint32_t NONE = 0xffffffffu;
	const uint32_t n_parts = LEVEL == 1 ? n_buckets : PART_BUCKET_SLABS;
	const uint32_t n_chunks = LEVEL == 1 ? div_up(n, PART_CHUNK) : ((volatile const uint32_t*)T.chunk_first)[n_buckets];
	for (uint32_t w = blockIdx.x; w < n_chunks; w += gridDim.x) {
		size_t first, last;
		uint32_t bucket = 0;
		if (LEVEL == 1) {
			first = (size_t)w * PART_CHUNK;
			last = first + PART_CHUNK < n ? first + PART_CHUNK : n;
		} else {
			uint32_t lo = 0, hi = n_buckets;      // the bucket whose chunks include w: the last b with chunk_first[b] <= w
			while (hi - lo > 1u) { const uint32_t mid = (lo + hi) / 2u; if (T.chunk_first[mid] <= w) lo = mid; else hi = mid; }
			bucket = lo;
			const uint32_t s0 = bucket << PART_BUCKET_BITS, s1 = s0 + PART_BUCKET_SLABS < n_slabs ? s0 + PART_BUCKET_SLABS : n_slabs;
			const size_t b_first = T.starts[s0], b_last = T.starts[s1];
			first = b_first + (size_t)(w - T.chunk_first[bucket]) * PART_CHUNK;
			last = first + PART_CHUNK < b_last ? first + PART_CHUNK : b_last;
		}
		if (threadIdx.x < PART_MAX_BUCKETS) { hist[threadIdx.x] = 0u; fill[threadIdx.x] = 0u; }
		__syncthreads();
		U2 e[PART_PER_THREAD];
		uint32_t part[PART_PER_THREAD];
		#pragma unroll
		for (uint32_t k = 0; k < PART_PER_THREAD; ++k) {
			const size_t i = first + (size_t)k * PART_PASS_THREADS + threadIdx.x;
			part[k] = NONE;
			if (i < last) {
				if (LEVEL == 1) {
					e[k].x = indices[i];
					e[k].y = srf_f2u(act_density(net_load<HALF>(densities, i * width), act) * min_cone_stepsize);
					if (e[k].x < n_total) part[k] = e[k].x >> (PART_SLAB_BITS + PART_BUCKET_BITS);
				} else {
					e[k] = in_pairs[i];
					part[k] = (e[k].x >> PART_SLAB_BITS) & (PART_BUCKET_SLABS - 1u);
				}
			}
		}
		#pragma unroll
		for (uint32_t k = 0; k < PART_PER_THREAD; ++k) if (part[k] != NONE) atomicAdd(&hist[part[k]], 1u);
		__syncthreads();
		// the chunk's share of every part's positions; where the parts start in the staged order
		if (threadIdx.x < n_parts) {
			const uint32_t v = hist[threadIdx.x];
			uint32_t* cursor = LEVEL == 1 ? T.bucket_cursor + threadIdx.x : T.slab_cursor + ((bucket << PART_BUCKET_BITS) + threadIdx.x);
			gbase[threadIdx.x] = v ? atomicAdd(cursor, v) : 0u;
		}
		if (threadIdx.x < 64u) {      // exclusive scan of the 256 counts (those past n_parts are zero): four a lane, then across the wavefront
			const uint32_t d0 = threadIdx.x * 4u;
			const uint32_t h0 = hist[d0], h1 = hist[d0 + 1u], h2 = hist[d0 + 2u], h3 = hist[d0 + 3u];
			const uint32_t mine = h0 + h1 + h2 + h3;
			uint32_t incl = mine;
			#pragma unroll
			for (uint32_t step = 1; step < 64u; step <<= 1) { const uint32_t up = __shfl_up(incl, step); if (threadIdx.x >= step) incl += up; }
			const uint32_t before = incl - mine;
			lstart[d0] = before; lstart[d0 + 1u] = before + h0; lstart[d0 + 2u] = before + h0 + h1; lstart[d0 + 3u] = before + h0 + h1 + h2;
			if (threadIdx.x == 63u) lstart[PART_MAX_BUCKETS] = incl;
		}
		__syncthreads();
		#pragma unroll
		for (uint32_t k = 0; k < PART_PER_THREAD; ++k) if (part[k] != NONE) stage[lstart[part[k]] + atomicAdd(&fill[part[k]], 1u)] = e[k];
		__syncthreads();
		const uint32_t staged = lstart[PART_MAX_BUCKETS];
		for (uint32_t j = threadIdx.x; j < staged; j += PART_PASS_THREADS) {
			const U2 v = stage[j];
			const uint32_t d = LEVEL == 1 ? v.x >> (PART_SLAB_BITS + PART_BUCKET_BITS) : (v.x >> PART_SLAB_BITS) & (PART_BUCKET_SLABS - 1u);
			out_pairs[gbase[d] + (j - lstart[d])] = v;
		}
		__syncthreads();
	}
}

// EMA: also apply k_ema_grid's decayed maximum to the slab's cells of the grid.  MERGE: the cells already hold another splat.
template <bool EMA, bool MERGE>
__global__ void __launch_bounds__(PART_THREADS) k_part_slabs(uint32_t n_total, const uint32_t* __restrict__ starts, const U2* __restrict__ pairs,
                                                             uint32_t* __restrict__ grid_current_bits, float decay, float* __restrict__ grid) {
	extern __shared__ uint32_t part_h[];      // the slab's cells
	const uint32_t slab = blockIdx.x;
	for (uint32_t j = threadIdx.x; j < PART_SLAB_CELLS; j += PART_THREADS) part_h[j] = 0u;
	__syncthreads();
	const uint32_t lo = starts[slab], hi = starts[slab + 1];
	for (uint32_t i = lo + threadIdx.x; i < hi; i += PART_THREADS) {
		const U2 e = pairs[i];
		if (e.y) atomicMax(&part_h[e.x & (PART_SLAB_CELLS - 1u)], e.y);      // a zero cannot raise a cell
	}
	__syncthreads();
	const uint32_t first = slab << PART_SLAB_BITS;
	for (uint32_t j = threadIdx.x * 4u; j < PART_SLAB_CELLS; j += PART_THREADS * 4u) {
		if (first + j + 3u < n_total) {
			uint4 c = *(const uint4*)(part_h + j);
			if (MERGE) {
				const uint4 o = *(const uint4*)(grid_current_bits + first + j);
				c.x = o.x > c.x ? o.x : c.x; c.y = o.y > c.y ? o.y : c.y; c.z = o.z > c.z ? o.z : c.z; c.w = o.w > c.w ? o.w : c.w;
			}
			*(uint4*)(grid_current_bits + first + j) = c;
			if (EMA) {
				float4 g = *(const float4*)(grid + first + j);
				g.x = (g.x < 0.f) ? g.x : srf_max(g.x * decay, srf_u2f(c.x));
				g.y = (g.y < 0.f) ? g.y : srf_max(g.y * decay, srf_u2f(c.y));
				g.z = (g.z < 0.f) ? g.z : srf_max(g.z * decay, srf_u2f(c.z));
				g.w = (g.w < 0.f) ? g.w : srf_max(g.w * decay, srf_u2f(c.w));
				*(float4*)(grid + first + j) = g;
			}
		} else {
			for (uint32_t k = 0; k < 4u && first + j + k < n_total; ++k) {
				uint32_t c = part_h[j + k];
				if (MERGE) { const uint32_t o = grid_current_bits[first + j + k]; c = o > c ? o : c; }
				grid_current_bits[first + j + k] = c;
				if (EMA) { const float g = grid[first + j + k]; grid[first + j + k] = (g < 0.f) ? g : srf_max(g * decay, srf_u2f(c)); }
			}
		}
	}
}

// The splat of samples that arrive dealt by cell (k_generate_grid_samples_by_cell's order, taken as it is by the caller):
// entry t = m n_cells + v lies in cell (v + 96925573) mod n_cells of some cascade when its point's first try passed, as nearly
// all tries against the -0.01 threshold do.  A workgroup owns DEALT_CELLS consecutive cells of every cascade, reads the entries
// that the dealing puts there (one contiguous stretch per m, two where it wraps), combines them in LDS and writes its cells
// of every cascade: no sort and no device atomics.  Every entry is checked against the place it is read from; one that lies
// elsewhere (a later try, or arrays that are not in this order at all) goes to a list that k_splat_listed applies afterwards.
// MERGE: the cells already hold the splat of other samples (those not in this order), so the result is the larger of both.
constexpr uint32_t DEALT_CELLS = 2048;
constexpr uint32_t DEALT_MAX_CASCADES = 8;            // 64 KB of LDS a workgroup; grids of more cascades take the entries through the other paths
constexpr uint32_t DEALT_FIRST_CELL = 96925573u;      // the constant of the candidate-cell hash (grid_sample_tries)
template <bool HALF, bool MERGE>
__global__ void __launch_bounds__(256) k_splat_dealt(uint32_t n_cells, uint32_t log2_cells, uint32_t n_cascades, uint32_t n_blocks_m, const uint32_t* __restrict__ indices,
                                                      uint32_t width, const void* __restrict__ densities, int act, float min_cone_stepsize,
                                                      uint32_t* __restrict__ grid_current_bits, uint32_t* __restrict__ list_count, U2* __restrict__ list) {
	extern __shared__ uint32_t tiles[];                      // [cascade][DEALT_CELLS]
	const uint32_t mask = n_cells - 1u;
	const uint32_t cell0 = blockIdx.x * DEALT_CELLS;
	for (uint32_t j = threadIdx.x; j < n_cascades * DEALT_CELLS; j += 256u) tiles[j] = 0u;
	__syncthreads();
	constexpr uint32_t PER_THREAD = DEALT_CELLS / 256u;     // entries of one multiple a thread takes: all fetched before any is used
	for (uint32_t m = 0; m < n_blocks_m; ++m) {
		uint32_t idx[PER_THREAD];
		float raw[PER_THREAD];
		#pragma unroll
		for (uint32_t q = 0; q < PER_THREAD; ++q) {
			const uint32_t cell = cell0 + q * 256u + threadIdx.x;
			const size_t t = ((size_t)m << log2_cells) + ((cell - DEALT_FIRST_CELL) & mask);
			idx[q] = indices[t];
			raw[q] = net_load<HALF>(densities, t * width);
		}
		#pragma unroll
		for (uint32_t q = 0; q < PER_THREAD; ++q) {
			const uint32_t k = q * 256u + threadIdx.x;
			const uint32_t bits = srf_f2u(act_density(raw[q], act) * min_cone_stepsize);
			if (bits == 0u) continue;                        // cannot raise a cell
			const uint32_t level = idx[q] >> log2_cells;
			if ((idx[q] & mask) == cell0 + k && level < n_cascades) atomicMax(&tiles[level * DEALT_CELLS + k], bits);
			else { const uint32_t at = atomicAdd(list_count, 1u); U2 e; e.x = idx[q]; e.y = bits; list[at] = e; }
		}
	}
	__syncthreads();
	for (uint32_t level = 0; level < n_cascades; ++level) {
		uint32_t* out = grid_current_bits + (size_t)level * n_cells + cell0;
		uint32_t old[PER_THREAD];
		#pragma unroll
		for (uint32_t q = 0; q < PER_THREAD; ++q) old[q] = MERGE ? out[q * 256u + threadIdx.x] : 0u;
		#pragma unroll
		for (uint32_t q = 0; q < PER_THREAD; ++q) {
			const uint32_t v = tiles[level * DEALT_CELLS + q * 256u + threadIdx.x];
			out[q * 256u + threadIdx.x] = old[q] > v ? old[q] : v;
		}
	}
}
__global__ void __launch_bounds__(256) k_splat_listed(const uint32_t* __restrict__ list_count, const U2* __restrict__ list, uint32_t n_total, uint32_t* __restrict__ grid_current_bits) {
	const uint32_t n = *list_count;
	for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
		const U2 e = list[i];
		if (e.x < n_total) atomicMax(&grid_current_bits[e.x], e.y);
	}
}

// occupancy_sampler.cu:214-238 — decayed maximum, four cells per thread
__global__ void __launch_bounds__(256) k_ema_grid(uint32_t n_vec4, const float4* __restrict__ cur, float decay, float4* __restrict__ grid) {
	uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	const uint32_t stride = gridDim.x * blockDim.x;
	for (; i < n_vec4; i += stride) {
		const float4 c = cur[i];
		float4 g = grid[i];
		g.x = (g.x < 0.f) ? g.x : srf_max(g.x * decay, c.x);
		g.y = (g.y < 0.f) ? g.y : srf_max(g.y * decay, c.y);
		g.z = (g.z < 0.f) ? g.z : srf_max(g.z * decay, c.z);
		g.w = (g.w < 0.f) ? g.w : srf_max(g.w * decay, c.w);
		grid[i] = g;
	}
}

// Mean of max(v,0)/n over the first cascade (occupancy_sampler.cu:1065-1070) with a fixed
// summation order: tiles of 1024 cells; inside a tile each thread adds its 4 consecutive
// terms left to right, then a balanced tree of adjacent pairs in float; tiles are combined
// by the same tree in double.
__global__ void __launch_bounds__(256) k_mean_tile_partials(const float* __restrict__ grid, uint32_t n, float denom, uint32_t n_tiles,
                                                             double* __restrict__ partials) {
	__shared__ float lds[4];
	for (uint32_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
		const uint32_t e = tile * 1024u + threadIdx.x * 4u;
		float t[4];
		if (e + 3 < n) {
			const float4 v = *(const float4*)(grid + e);
			t[0] = srf_max(v.x, 0.f) / denom; t[1] = srf_max(v.y, 0.f) / denom;
			t[2] = srf_max(v.z, 0.f) / denom; t[3] = srf_max(v.w, 0.f) / denom;
		} else {
			for (uint32_t k = 0; k < 4; ++k) t[k] = (e + k < n) ? srf_max(grid[e + k], 0.f) / denom : 0.f;
		}
		float s = ((t[0] + t[1]) + t[2]) + t[3];
		#pragma unroll
		for (uint32_t d = 1; d < WAVE; d <<= 1) s = s + __shfl_xor(s, d, WAVE);
		if (lane_id() == 0) lds[threadIdx.x / WAVE] = s;
		__syncthreads();
		if (threadIdx.x == 0) partials[tile] = (double)((lds[0] + lds[1]) + (lds[2] + lds[3]));
		__syncthreads();
	}
}

// adjacent-pair tree over up to 1024 doubles per block (count per block is a power of two)
__global__ void __launch_bounds__(512) k_reduce_pairs_f64(const double* __restrict__ in, uint32_t n_in, double* __restrict__ out, float* __restrict__ out_f32) {
	__shared__ double a[1024];
	const uint32_t base = blockIdx.x * 1024u;
	const uint32_t count = (n_in - base) < 1024u ? (n_in - base) : 1024u;
	for (uint32_t k = threadIdx.x; k < 1024u; k += blockDim.x) a[k] = (k < count) ? in[base + k] : 0.0;
	__syncthreads();
	for (uint32_t s = 1; s < 1024u; s <<= 1) {
		const uint32_t k = threadIdx.x * 2u * s;
		if (k + s < 1024u) a[k] = a[k] + a[k + s];
		__syncthreads();
	}
	if (threadIdx.x == 0) {
		if (out) out[blockIdx.x] = a[0];
		if (out_f32) out_f32[blockIdx.x] = (float)a[0];
	}
}

// occupancy_sampler.cu:240-260 — bit j of byte i is grid[8i+j] > thresh.  A wave tests 64
// consecutive cells per load and its ballot IS the 8 output bytes; eight ballots are
// gathered so that lanes 0..7 store 64 contiguous bytes.
__global__ void __launch_bounds__(256) k_grid_to_bitfield(const float* __restrict__ grid, uint32_t n_total, const float* __restrict__ mean_ptr,
                                                           float min_optical_thickness, uint8_t* __restrict__ bitfield) {
	const float mean = *mean_ptr;
	const float thresh = (mean < min_optical_thickness) ? mean : min_optical_thickness;
	const uint32_t lane = lane_id();
	const uint32_t n_chunks = div_up(n_total, 512u);
	const uint32_t wave_global = (blockIdx.x * blockDim.x + threadIdx.x) / WAVE;
	const uint32_t n_waves = gridDim.x * blockDim.x / WAVE;
	for (uint32_t chunk = wave_global; chunk < n_chunks; chunk += n_waves) {
		const uint32_t base = chunk * 512u;
		float v[8];
		#pragma unroll
		for (uint32_t k = 0; k < 8; ++k) {
			const uint32_t c = base + k * 64u + lane;
			v[k] = c < n_total ? grid[c] : 0.f;
		}
		uint64_t mine = 0;
		#pragma unroll
		for (uint32_t k = 0; k < 8; ++k) {
			const uint32_t c = base + k * 64u + lane;
			const uint64_t b = __ballot(c < n_total && v[k] > thresh);
			if (lane == k) mine = b;
		}
		if (lane < 8) {
			const uint32_t first = base + lane * 64u;
			if (first + 64u <= n_total) *(uint64_t*)(bitfield + first / 8u) = mine;
			else for (uint32_t c = first; c < n_total; c += 8u) bitfield[c / 8u] = (uint8_t)(mine >> (c - first));
		}
	}
}

// occupancy_sampler.cu:262-285 — 8 bytes of the finer cascade (a 4x4x4 block of cells)
// become one byte of the next cascade, OR-ed in at the centred position.
__global__ void __launch_bounds__(256) k_bitfield_max_pool(uint32_t n_elements, uint32_t off_x, uint32_t off_y, uint32_t off_z,
                                                            const uint8_t* __restrict__ prev_level, uint8_t* __restrict__ next_level) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= n_elements) return;
	const uint64_t src = *(const uint64_t*)(prev_level + (size_t)i * 8);
	uint32_t bits = 0;
	#pragma unroll
	for (uint32_t j = 0; j < 8; ++j) bits |= ((src >> (8 * j)) & 0xffu) ? (1u << j) : 0u;
	const uint32_t x = morton3d_invert(i) + off_x, y = morton3d_invert(i >> 1) + off_y, z = morton3d_invert(i >> 2) + off_z;
	const uint32_t dst = morton3d(x, y, z);
	next_level[dst] = (uint8_t)(next_level[dst] | bits);
}

static bool is_pow2(uint32_t v) { return v && !(v & (v - 1)); }

__global__ void __launch_bounds__(256) k_skip_block_occupancy(Params P, SkipTable T, uint32_t n, const uint8_t* __restrict__ bitfield, uint8_t* __restrict__ occ) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n) skip_block_occupancy_body(i, P, T, bitfield, occ);
}
__global__ void __launch_bounds__(256) k_skip_pool(SkipTable T, uint32_t n, uint32_t level, uint8_t* occ) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n) skip_pool_body(i, T, level, occ);
}
__global__ void __launch_bounds__(256) k_skip_distance_axis(SkipTable T, uint32_t n, uint32_t axis, const uint8_t* __restrict__ in, uint8_t* __restrict__ out) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n) skip_distance_axis_body(i, T, axis, in, out);
}
__global__ void __launch_bounds__(256) k_skip_combine(Params P, SkipTable T, uint32_t n, const uint8_t* __restrict__ n_blocks, uint16_t* __restrict__ dist) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n) skip_combine_body(i, P, T, n_blocks, dist);
}

// rebuilds the empty-space table from the sampler's bitfield (stream-ordered after the bitfield update)
static int rebuild_skip_table(srf_sampler* s, hipStream_t st) {
	s->skip_valid = false;
	const Params& P = s->P;
	const uint32_t nb = skip_blocks_per_axis(P);
	if (!nb || !s->skip_dist || !s->skip_enabled) return SRF_OK;
	const SkipTable T = skip_table_for(P, s->skip_dist);
	const uint32_t n = nb * nb * nb * P.n_cascades;
	int rc = s->ws.reserve(2 * align_up(n, 256));
	if (rc != SRF_OK) return rc;
	uint8_t* a = (uint8_t*)s->ws.ptr;
	uint8_t* b = a + align_up(n, 256);
	hipLaunchKernelGGL(k_skip_block_occupancy, dim3(div_up(n, 256)), dim3(256), 0, st, P, T, n, (const uint8_t*)s->density_grid_bitfield, a);
	SRF_LAUNCH_CHECK();
	const uint32_t h3 = (nb / 2) * (nb / 2) * (nb / 2);
	for (uint32_t level = 1; level < P.n_cascades; ++level) {
		hipLaunchKernelGGL(k_skip_pool, dim3(div_up(h3, 256)), dim3(256), 0, st, T, h3, level, a);
		SRF_LAUNCH_CHECK();
	}
	hipLaunchKernelGGL(k_skip_distance_axis, dim3(div_up(n, 256)), dim3(256), 0, st, T, n, 0u, (const uint8_t*)a, b);
	SRF_LAUNCH_CHECK();
	hipLaunchKernelGGL(k_skip_distance_axis, dim3(div_up(n, 256)), dim3(256), 0, st, T, n, 1u, (const uint8_t*)b, a);
	SRF_LAUNCH_CHECK();
	hipLaunchKernelGGL(k_skip_distance_axis, dim3(div_up(n, 256)), dim3(256), 0, st, T, n, 2u, (const uint8_t*)a, b);
	SRF_LAUNCH_CHECK();
	hipLaunchKernelGGL(k_skip_combine, dim3(div_up(n, 256)), dim3(256), 0, st, P, T, n, (const uint8_t*)b, s->skip_dist);
	SRF_LAUNCH_CHECK();
	s->skip_valid = true;
	return SRF_OK;
}

} // namespace srf

using namespace srf;

extern "C" {

void srf_sampler_config_default(srf_sampler_config* c) {
	if (!c) return;
	memset(c, 0, sizeof(*c));
	c->warping_type = SRF_WARP_NGP;
	c->aabb_scale = 1.f;
	c->use_grid = 1;
	c->init_grid_with_mask = 1;
	c->grid_size[0] = c->grid_size[1] = c->grid_size[2] = 128;
	c->num_cascades = 1;
	c->ema_decay = 0.95f;
	// the reference's default string "Exp" is rejected by its own parser (occupancy_sampler.cu:895-907, 927);
	// the numeric default here is the type every shipped config names
	c->grid_distribution_type = SRF_GRID_WARPED_EXP;
	c->maximum_marching_steps = 1024;
	c->cone_angle_constant = 0.f;
	c->min_cone_stepsize = -1.f;
	c->max_cone_stepsize = -1.f;
	c->near_distance = 0.2f;
	c->far_distance = 100.f;
	c->sampling_type = SRF_SAMPLING_ORIGINAL;
	c->snap_to_pixel_centers_in_training = 1;
	c->snap_to_pixel_centers_in_rendering = 1;
	c->min_optical_thickness = 0.01f;
}

int srf_sampler_create(const srf_sampler_config* c, srf_sampler_t** out) {
	SRF_REQUIRE(c && out, "srf_sampler_create: NULL argument");
	*out = nullptr;
	SRF_REQUIRE(c->warping_type >= SRF_WARP_NGP && c->warping_type <= SRF_WARP_SINUSOIDAL, "Unknown warping type.");
	SRF_REQUIRE(c->sampling_type >= SRF_SAMPLING_ORIGINAL && c->sampling_type <= SRF_SAMPLING_LOG, "Unknown sampling type.");
	SRF_REQUIRE(c->grid_distribution_type >= SRF_GRID_WARPED_EXP && c->grid_distribution_type <= SRF_GRID_METRIC_RECIPROCAL, "Unknown grid distribution type.");
	SRF_REQUIRE(c->maximum_marching_steps > 0, "maximum_marching_steps must be positive");
	SRF_REQUIRE(c->aabb_scale >= 1.f && c->aabb_scale < 4.0e9f, "aabb_scale out of range");
	srf_sampler* s = new srf_sampler();
	Params& P = s->P;
	memset(&P, 0, sizeof(P));
	P.warping_type = c->warping_type;
	P.aabb_scale = (uint32_t)c->aabb_scale;
	const float amount = 0.5f * (float)P.aabb_scale;
	for (int a = 0; a < 3; ++a) { P.aabb_min[a] = 0.5f - amount; P.aabb_max[a] = 0.5f + amount; }
	P.use_grid = c->use_grid ? 1 : 0;
	s->init_grid_with_mask = c->init_grid_with_mask;
	P.n_cascades = 1;
	P.grid_size[0] = P.grid_size[1] = P.grid_size[2] = 1;
	P.griddist_type = c->grid_distribution_type;
	if (P.use_grid) {
		for (int a = 0; a < 3; ++a) {
			if (!is_pow2(c->grid_size[a]) || c->grid_size[a] < 2 || c->grid_size[a] > 1024) {
				delete s;
				SRF_FAIL(SRF_ERR_INVALID, "grid_size[%d]=%u: must be a power of two in [2, 1024]", a, c->grid_size[a]);
			}
			P.grid_size[a] = c->grid_size[a];
		}
		if (c->num_cascades < 1 || c->num_cascades > 16) { delete s; SRF_FAIL(SRF_ERR_INVALID, "num_cascades=%u out of range [1,16]", c->num_cascades); }
		P.n_cascades = c->num_cascades;
		const uint64_t cells = (uint64_t)P.grid_size[0] * P.grid_size[1] * P.grid_size[2];
		// the Morton code of the last cell must be cells-1, i.e. the curve is a bijection onto [0, cells)
		if ((uint64_t)morton3d(P.grid_size[0] - 1, P.grid_size[1] - 1, P.grid_size[2] - 1) + 1 != cells || cells * P.n_cascades > 0xffffffffull || cells < 8) {
			delete s;
			SRF_FAIL(SRF_ERR_INVALID, "grid %ux%ux%u x %u cascades: per-axis sizes must satisfy x >= y >= z, x <= 2z, total < 2^32",
			         P.grid_size[0], P.grid_size[1], P.grid_size[2], P.n_cascades);
		}
		P.n_cells = (uint32_t)cells;
	}
	s->n_total = P.n_cells * P.n_cascades;
	P.ema_decay = c->ema_decay;
	P.n_max_steps = c->maximum_marching_steps;
	P.cone_angle_constant = c->cone_angle_constant;
	const float SQRT3 = 1.73205080757f;
	P.min_cone_stepsize = c->min_cone_stepsize >= 0.f ? c->min_cone_stepsize : SQRT3 / (float)P.n_max_steps;
	P.max_cone_stepsize = c->max_cone_stepsize >= 0.f ? c->max_cone_stepsize
	                    : (P.use_grid ? (SQRT3 * (float)(1 << (P.n_cascades - 1)) / (float)P.grid_size[0]) : P.min_cone_stepsize);
	P.near_distance = c->near_distance;
	P.far_distance = c->far_distance;
	P.sampling_type = c->sampling_type;
	P.snap_train = c->snap_to_pixel_centers_in_training ? 1 : 0;
	P.snap_render = c->snap_to_pixel_centers_in_rendering ? 1 : 0;
	P.min_optical_thickness = c->min_optical_thickness;
	s->i_step = 0;
	s->rng.state = 0x853c49e6748fea9bULL;
	s->rng.inc = 0xda3e39cb94b95bdbULL;
	s->density_grid = s->density_grid_current = s->density_grid_mean = nullptr;
	s->density_grid_bitfield = nullptr;
	s->skip_dist = nullptr;
	s->skip_valid = false;
	{ const char* v = getenv("SRF_MARCH_SKIP"); s->skip_enabled = !(v && v[0] == '0'); }
	auto tri_state = [](const char* name) { const char* v = getenv(name); return v && v[0] == '0' ? 0 : (v && v[0] == '1' ? 1 : -1); };
	s->force_splat_sort = tri_state("SRF_SPLAT_SORT");
	{ const char* v = getenv("SRF_SPLAT_SORT"); if (v && v[0] == '2') s->force_splat_sort = 2; }      // 2: large-batch path through the library's sort
	s->force_sample_bits = tri_state("SRF_GRID_SAMPLE_BITS");
	s->force_sample_by_cell = tri_state("SRF_GRID_SAMPLE_BY_CELL");
	s->count_probe_budget = COUNT_PROBE_BUDGET;
	{ const char* v = getenv("SRF_COUNT_PROBE_BUDGET"); if (v && v[0]) s->count_probe_budget = (uint32_t)atoi(v); }
	s->count_park_lanes = COUNT_PARK_LANES;
	{ const char* v = getenv("SRF_COUNT_PARK_LANES"); if (v && v[0]) s->count_park_lanes = (uint32_t)atoi(v); }
	// SRF_MARCH_PARK_ALL=1: the render marches hand every ray that finds an empty cell without anything to skip to their
	// one-ray-per-wavefront march at once, whatever the wavefront still holds (for tests: that march then does most of a frame)
	{ const char* v = getenv("SRF_MARCH_PARK_ALL"); s->march_park_all = v && v[0] == '1'; }
	hipError_t e = hipSuccess;
	if (P.use_grid) {
		e = hipMalloc((void**)&s->density_grid_current, (size_t)s->n_total * sizeof(float));
		if (e == hipSuccess) e = hipMalloc((void**)&s->density_grid, (size_t)s->n_total * sizeof(float));
		if (e == hipSuccess) e = hipMalloc((void**)&s->density_grid_bitfield, (size_t)s->n_total / 8);
		if (e == hipSuccess) e = hipMemset(s->density_grid, 0, (size_t)s->n_total * sizeof(float));
		if (e == hipSuccess) e = hipMemset(s->density_grid_current, 0, (size_t)s->n_total * sizeof(float));
		if (e == hipSuccess) e = hipMemset(s->density_grid_bitfield, 0, (size_t)s->n_total / 8);
		const uint32_t nb = skip_blocks_per_axis(P);
		if (e == hipSuccess && nb) e = hipMalloc((void**)&s->skip_dist, (size_t)nb * nb * nb * P.n_cascades * sizeof(uint16_t));
	}
	if (e == hipSuccess) e = hipMalloc((void**)&s->density_grid_mean, 256);
	if (e == hipSuccess) e = hipMemset(s->density_grid_mean, 0, 256);
	if (e != hipSuccess) {
		srf_sampler_destroy(s);
		SRF_FAIL(SRF_ERR_HIP, "srf_sampler_create: device allocation failed: %s", hipGetErrorString(e));
	}
	*out = s;
	return SRF_OK;
}

void srf_sampler_destroy(srf_sampler_t* s) {
	if (!s) return;
	if (s->density_grid_current) (void)hipFree(s->density_grid_current);
	if (s->density_grid) (void)hipFree(s->density_grid);
	if (s->density_grid_mean) (void)hipFree(s->density_grid_mean);
	if (s->density_grid_bitfield) (void)hipFree(s->density_grid_bitfield);
	if (s->skip_dist) (void)hipFree(s->skip_dist);
	s->ws.release();
	s->park_ws.release();
	if (s->park_counts) (void)hipFree(s->park_counts);
	delete s;
}

int srf_sampler_get_info(const srf_sampler_t* s, srf_sampler_info* o) {
	SRF_REQUIRE(s && o, "srf_sampler_get_info: NULL argument");
	const Params& P = s->P;
	memset(o, 0, sizeof(*o));
	o->warping_type = P.warping_type;
	o->aabb_scale = P.aabb_scale;
	for (int a = 0; a < 3; ++a) { o->aabb_min[a] = P.aabb_min[a]; o->aabb_max[a] = P.aabb_max[a]; o->grid_size[a] = P.grid_size[a]; }
	o->use_grid = P.use_grid;
	o->init_grid_with_mask = s->init_grid_with_mask;
	o->n_grid_elements = P.n_cells;
	o->n_cascades = P.n_cascades;
	o->n_total_elements = s->n_total;
	o->i_step = s->i_step;
	o->ema_decay = P.ema_decay;
	o->n_max_steps = P.n_max_steps;
	o->cone_angle_constant = P.cone_angle_constant;
	o->min_cone_stepsize = P.min_cone_stepsize;
	o->max_cone_stepsize = P.max_cone_stepsize;
	o->near_distance = P.near_distance;
	o->far_distance = P.far_distance;
	o->sampling_type = P.sampling_type;
	o->snap_to_pixel_centers_in_training = P.snap_train;
	o->snap_to_pixel_centers_in_rendering = P.snap_render;
	o->min_optical_thickness = P.min_optical_thickness;
	o->griddist_type = P.griddist_type;
	o->density_grid_current = s->density_grid_current;
	o->density_grid = s->density_grid;
	o->density_grid_mean = s->density_grid_mean;
	o->density_grid_bitfield = s->density_grid_bitfield;
	o->rng.state = s->rng.state;
	o->rng.inc = s->rng.inc;
	return SRF_OK;
}

int srf_sampler_set_runtime(srf_sampler_t* s, int32_t snap_train, int32_t snap_render, float near_distance, float far_distance) {
	SRF_REQUIRE(s, "srf_sampler_set_runtime: NULL sampler");
	s->P.snap_train = snap_train ? 1 : 0;
	s->P.snap_render = snap_render ? 1 : 0;
	s->P.near_distance = near_distance;
	s->P.far_distance = far_distance;
	return SRF_OK;
}

int srf_sampler_init(srf_sampler_t* s, uint32_t n_images, const int32_t image_resolution[2], const float focal_length[2],
                     const float principal_point[2], const float* camera_matrices, srf_pcg32* rng_host, void* stream) {
	SRF_REQUIRE(s && rng_host, "srf_sampler_init: NULL argument");
	(void)principal_point;
	// occupancy_sampler.cu:959: the mask is only made for the NGP warp, where cameras and grid share a metric frame
	const bool mask = s->P.use_grid && s->init_grid_with_mask && s->P.warping_type == SRF_WARP_NGP;
	SRF_REQUIRE(!mask || (image_resolution && focal_length && (camera_matrices || n_images == 0)), "srf_sampler_init: the camera-visibility mask needs the cameras");
	s->i_step = 0;
	Pcg32 caller; caller.state = rng_host->state; caller.inc = rng_host->inc;
	const uint32_t seed = pcg_next_uint(caller);
	rng_host->state = caller.state; rng_host->inc = caller.inc;
	pcg_seed(s->rng, (uint64_t)seed, 1u);
	if (mask) {
		hipLaunchKernelGGL(k_mark_untrained, dim3(div_up(s->n_total, 256)), dim3(256), 0, (hipStream_t)stream, s->P, s->n_total, n_images, focal_length[0], focal_length[1],
		                   (float)image_resolution[0] * 0.5f, (float)image_resolution[1] * 0.5f, camera_matrices, s->density_grid);
		SRF_LAUNCH_CHECK();
	} else if (s->P.use_grid) {
		int rc = fill_u32(s->density_grid, s->n_total, 0u, (hipStream_t)stream);
		if (rc != SRF_OK) return rc;
	}
	return SRF_OK;
}

int srf_sampler_set_density_grid(srf_sampler_t* s, const float* density_grid, void* stream) {
	SRF_REQUIRE(s && density_grid, "srf_sampler_set_density_grid: NULL argument");
	SRF_REQUIRE(s->P.use_grid, "srf_sampler_set_density_grid: sampler has no grid");
	SRF_HIP(hipMemcpyAsync(s->density_grid, density_grid, (size_t)s->n_total * sizeof(float), hipMemcpyDeviceToDevice, (hipStream_t)stream));
	return SRF_OK;
}

int srf_sampler_load_density_grid(srf_sampler_t* s, const float* density_grid_host, uint32_t n_values, void* stream) {
	SRF_REQUIRE(s && density_grid_host, "srf_sampler_load_density_grid: NULL argument");
	SRF_REQUIRE(s->P.use_grid, "srf_sampler_load_density_grid: sampler has no grid");
	SRF_REQUIRE(n_values == s->n_total, "srf_sampler_load_density_grid: the snapshot's grid holds %u values, the configured grid has %u cells", n_values, s->n_total);
	SRF_HIP(hipMemcpyAsync(s->density_grid, density_grid_host, (size_t)s->n_total * sizeof(float), hipMemcpyHostToDevice, (hipStream_t)stream));
	SRF_HIP(hipStreamSynchronize((hipStream_t)stream));
	return srf_sampler_update_grid_bitfield(s, stream);
}

int srf_sampler_set_grid_sample_order(srf_sampler_t* s, int32_t cell_order) {
	SRF_REQUIRE(s, "srf_sampler_set_grid_sample_order: NULL sampler");
	SRF_REQUIRE(cell_order == 0 || cell_order == 1, "srf_sampler_set_grid_sample_order: order must be 0 or 1");
	s->grid_sample_cell_order = cell_order != 0;
	s->dealt_entries = 0;
	return SRF_OK;
}

int srf_sampler_sample_positions_from_grid(srf_sampler_t* s, uint32_t n_uniform, uint32_t n_nonuniform,
                                           float* grid_positions, uint32_t* grid_indices, void* stream) {
	SRF_REQUIRE(s, "srf_sampler_sample_positions_from_grid: NULL sampler");
	SRF_REQUIRE(s->P.use_grid, "srf_sampler_sample_positions_from_grid: sampler has no grid");
	SRF_REQUIRE((uint64_t)n_uniform + n_nonuniform == 0 || (grid_positions && grid_indices), "srf_sampler_sample_positions_from_grid: NULL output");
	hipStream_t st = (hipStream_t)stream;
	const uint32_t nc = s->P.n_cells;
	// With many points to draw, the two comparisons the draws make against the grid (grid > -0.01 for the uniform points,
	// grid > min_optical_thickness for the others) are tabulated first, one bit per cell: the random lookups then fall on
	// 1/32 of the memory.  (force_sample_bits: either way, for the tests.)
	bool tabulate = (uint64_t)n_uniform + n_nonuniform >= s->n_total / 8;
	if (s->force_sample_bits >= 0) tabulate = s->force_sample_bits != 0;
	tabulate = tabulate && (uint64_t)n_uniform + n_nonuniform != 0;
	// Most tries of the second draw fail (few cells are above the threshold), so its cost is the lookups: its points are
	// dealt to the threads by cell (k_generate_grid_samples_by_cell).  (force_sample_by_cell: either way, for the tests.)
	const bool can_deal = (nc & (nc - 1u)) == 0u && nc >= 256u && n_nonuniform != 0;
	bool by_cell = can_deal && n_nonuniform >= 65536u;
	if (s->force_sample_by_cell >= 0) by_cell = s->force_sample_by_cell != 0 && can_deal;
	// workspace: the two bit tables, then the staging array of the dealt draw (reserved in one go: growing frees)
	const size_t table_bytes = tabulate ? align_up((size_t)div_up(s->n_total, 32) * 4, 256) : 0;
	// Cell order (srf_sampler_set_grid_sample_order): the points of whole multiples of the cell count stay in the order of the
	// dealing, entry t = m n_cells + v of a draw holding the point whose (i + step n) A mod n_cells is v; srf_sampler_update_grid
	// then splats the uniform ones without sorting.  The other points of each draw follow in their own order.
	const bool cell_order = s->grid_sample_cell_order && (nc & (nc - 1u)) == 0u && nc >= DEALT_CELLS;
	const uint32_t n_dealt = cell_order ? n_uniform / nc * nc : 0u, n_dealt_b = cell_order ? n_nonuniform / nc * nc : 0u;
	by_cell = by_cell && n_nonuniform > n_dealt_b;
	const uint64_t dealt_threads = by_cell ? (uint64_t)div_up(n_nonuniform, nc) * nc - n_dealt_b : 0;       // those that go through the staging array
	const size_t summary_words = tabulate ? div_up(div_up(s->n_total, 32), 32) + 1 : 0;
	const size_t summary_bytes = align_up(summary_words * 4, 256);
	int rc = s->ws.reserve(2 * table_bytes + summary_bytes + dealt_threads * sizeof(Float4) + 256);
	if (rc != SRF_OK) return rc;
	const uint32_t* above_a = nullptr;
	const uint32_t* above_b = nullptr;
	const uint32_t* summary_a = nullptr;
	if (tabulate) {
		uint32_t* a = (uint32_t*)s->ws.ptr;
		uint32_t* b = (uint32_t*)((char*)s->ws.ptr + table_bytes);
		uint32_t* sum = (uint32_t*)((char*)s->ws.ptr + 2 * table_bytes);
		rc = fill_u32(sum, summary_words, 0u, st);
		if (rc != SRF_OK) return rc;
		const uint32_t blocks = div_up(s->n_total, 1024) < 16384 ? div_up(s->n_total, 1024) : 16384;
		hipLaunchKernelGGL(k_threshold_bits, dim3(blocks), dim3(256), 0, st, (const float*)s->density_grid, s->n_total, -0.01f, s->P.min_optical_thickness, a, b, sum);
		SRF_LAUNCH_CHECK();
		above_a = a; above_b = b; summary_a = sum;
	}
	const uint32_t tries = 10;    // the second draw looks all ten candidates of a point up at once: most fail in a trained grid (168 M points: 9.5 -> 6.2 ms)
	auto dealt_grid = [](uint32_t windows) { return windows < 16384u ? windows : 16384u; };
	const uint32_t deal_window = nc >= DEAL_WINDOW_MAX ? DEAL_WINDOW_MAX : 256u;      // threads of the dealing a workgroup takes at a time (the cell count, a power of two >= 256, is a multiple)
	uint32_t log2_cells = 0;
	while ((1u << log2_cells) < nc) ++log2_cells;
	uint32_t inv = 56924617u;                                  // inverse of the hash multiplier modulo 2^32, by Newton's iteration
	for (int k = 0; k < 5; ++k) inv *= 2u - 56924617u * inv;
	s->dealt_entries = n_dealt;
	if (n_dealt) {
		hipLaunchKernelGGL(k_generate_grid_samples_by_cell<false>, dim3(dealt_grid(n_dealt / deal_window)), dim3(256), 0, st, s->P, n_uniform, s->rng, s->i_step,
		                   (const float*)s->density_grid, -0.01f, (Float4*)nullptr, above_a, 1u, inv, log2_cells, grid_positions, grid_indices, 0u, n_dealt / deal_window, deal_window / 256u);
		SRF_LAUNCH_CHECK();
	}
	if (n_uniform > n_dealt) {
		const uint32_t runs = div_up(n_uniform - n_dealt, 256);
		hipLaunchKernelGGL(k_generate_grid_samples, dim3(runs < 16384u ? runs : 16384u), dim3(256), 0, st, s->P, n_uniform, s->rng, s->i_step,
		                   (const float*)s->density_grid, -0.01f, grid_positions, grid_indices, above_a, 1u, n_dealt, summary_a);   // nearly every first try passes
		SRF_LAUNCH_CHECK();
	}
	pcg_advance(s->rng, 1ull << 32);
	float* positions_b = grid_positions + 3 * (size_t)n_uniform;
	uint32_t* indices_b = grid_indices + n_uniform;
	if (n_dealt_b) {
		hipLaunchKernelGGL(k_generate_grid_samples_by_cell<false>, dim3(dealt_grid(n_dealt_b / deal_window)), dim3(256), 0, st, s->P, n_nonuniform, s->rng, s->i_step,
		                   (const float*)s->density_grid, s->P.min_optical_thickness, (Float4*)nullptr, above_b, tries, inv, log2_cells, positions_b, indices_b, 0u, n_dealt_b / deal_window, deal_window / 256u);
		SRF_LAUNCH_CHECK();
	}
	if (by_cell) {
		Float4* staged = (Float4*)((char*)s->ws.ptr + 2 * table_bytes + summary_bytes);
		// the whole multiples of the cell count, then the one the points do not fill
		const uint64_t full_threads = (uint64_t)n_nonuniform / nc * nc - n_dealt_b;
		if (full_threads) {
			hipLaunchKernelGGL(k_generate_grid_samples_by_cell<false>, dim3(dealt_grid((uint32_t)(full_threads / deal_window))), dim3(256), 0, st, s->P, n_nonuniform, s->rng, s->i_step,
			                   (const float*)s->density_grid, s->P.min_optical_thickness, staged, above_b, tries, inv, log2_cells, (float*)nullptr, (uint32_t*)nullptr, n_dealt_b,
			                   (uint32_t)(full_threads / deal_window), deal_window / 256u);
			SRF_LAUNCH_CHECK();
		}
		if (dealt_threads > full_threads) {
			hipLaunchKernelGGL(k_generate_grid_samples_by_cell<true>, dim3(dealt_grid(nc / deal_window)), dim3(256), 0, st, s->P, n_nonuniform, s->rng, s->i_step,
			                   (const float*)s->density_grid, s->P.min_optical_thickness, staged + full_threads, above_b, tries, inv, log2_cells, (float*)nullptr, (uint32_t*)nullptr,
			                   (uint32_t)(n_dealt_b + full_threads), nc / deal_window, deal_window / 256u);
			SRF_LAUNCH_CHECK();
		}
		hipLaunchKernelGGL(k_grid_samples_to_point_order, dim3(div_up(n_nonuniform - n_dealt_b, 256)), dim3(256), 0, st, nc, n_nonuniform, s->i_step, log2_cells,
		                   (const Float4*)staged, positions_b, indices_b, n_dealt_b);
		SRF_LAUNCH_CHECK();
	} else if (n_nonuniform > n_dealt_b) {
		const uint32_t runs = div_up(n_nonuniform - n_dealt_b, 256);
		hipLaunchKernelGGL(k_generate_grid_samples, dim3(runs < 16384u ? runs : 16384u), dim3(256), 0, st, s->P, n_nonuniform, s->rng, s->i_step,
		                   (const float*)s->density_grid, s->P.min_optical_thickness, positions_b, indices_b, above_b, tries, n_dealt_b, (const uint32_t*)nullptr);
		SRF_LAUNCH_CHECK();
	}
	pcg_advance(s->rng, 1ull << 32);
	return SRF_OK;
}

int srf_sampler_update_grid(srf_sampler_t* s, uint32_t n_total_positions, uint32_t padded_output_width,
                            const void* grid_densities, int32_t densities_dtype, const uint32_t* grid_indices,
                            int32_t density_activation, void* stream) {
	SRF_REQUIRE(s, "srf_sampler_update_grid: NULL sampler");
	SRF_REQUIRE(s->P.use_grid, "srf_sampler_update_grid: sampler has no grid");
	SRF_REQUIRE(n_total_positions == 0 || (grid_densities && grid_indices), "srf_sampler_update_grid: NULL input");
	SRF_REQUIRE(padded_output_width >= 1, "srf_sampler_update_grid: padded_output_width must be >= 1");
	SRF_REQUIRE(densities_dtype == SRF_DTYPE_F16 || densities_dtype == SRF_DTYPE_F32, "srf_sampler_update_grid: unknown dtype");
	SRF_REQUIRE(density_activation >= SRF_ACT_NONE && density_activation <= SRF_ACT_EXPONENTIAL, "srf_sampler_update_grid: unknown activation");
	hipStream_t st = (hipStream_t)stream;
	const bool half = densities_dtype == SRF_DTYPE_F16;
	const uint32_t nc = s->P.n_cells;
	// the leading entries that the last srf_sampler_sample_positions_from_grid left in cell order (every one of them is checked
	// where it is used: arrays in another order cost time, not correctness), and the others
	uint32_t n_dealt = s->grid_sample_cell_order && s->dealt_entries < n_total_positions ? s->dealt_entries : (s->grid_sample_cell_order ? n_total_positions : 0u);
	n_dealt = (nc & (nc - 1u)) == 0u && nc >= DEALT_CELLS && s->P.n_cascades <= DEALT_MAX_CASCADES ? n_dealt / nc * nc : 0u;
	const uint32_t n = n_total_positions - n_dealt;
	const uint32_t* rest_indices = grid_indices ? grid_indices + n_dealt : nullptr;
	const void* rest_densities = grid_densities ? (const char*)grid_densities + (size_t)n_dealt * padded_output_width * (half ? 2 : 4) : nullptr;
	bool sorted_splat = n >= SPLAT_SORT_MIN;
	if (s->force_splat_sort >= 0) sorted_splat = s->force_splat_sort != 0 && n != 0;
	// large batches: the hand-made partition by slab; grids of more slabs than its histograms hold go through the library's sort
	const uint32_t n_part_slabs = div_up(s->n_total, PART_SLAB_CELLS);
	const bool partition = sorted_splat && n_part_slabs <= PART_MAX_SLABS && s->force_splat_sort != 2;
	// who clears the cells: the dealt splat or the slabs of the sorted one, which write every cell, or else a fill
	int rc = sorted_splat || n_dealt ? SRF_OK : fill_u32(s->density_grid_current, s->n_total, 0u, st);
	if (rc != SRF_OK) return rc;
	int end_bit = (int)SPLAT_SLAB_BITS + 1;
	while (end_bit < 32 && (1ull << end_bit) < (unsigned long long)s->n_total) ++end_bit;
	size_t temp_bytes = 0;
	if (sorted_splat && !partition)
		SRF_HIP(hipcub::DeviceRadixSort::SortPairs(nullptr, temp_bytes, (const uint32_t*)nullptr, (uint32_t*)nullptr, (const uint32_t*)nullptr, (uint32_t*)nullptr,
		                                           (int)n, (int)SPLAT_SLAB_BITS, end_bit, st));
	const size_t arr = sorted_splat ? align_up((size_t)n * 4, 256) : 0;
	const size_t part_words = align_up(((size_t)3 * n_part_slabs + 1 + 2 * PART_MAX_BUCKETS + 1) * 4, 256);
	const size_t sort_bytes = !sorted_splat ? 0 : partition ? part_words + 2 * align_up((size_t)n, 32) * sizeof(U2) : align_up(3 * arr + temp_bytes, 256);
	const size_t list_bytes = n_dealt ? 256 + (size_t)n_dealt * sizeof(U2) : 0;
	rc = s->ws.reserve(sort_bytes + list_bytes);
	if (rc != SRF_OK) return rc;
	uint32_t* list_count = (uint32_t*)((char*)s->ws.ptr + sort_bytes);
	U2* list = (U2*)((char*)s->ws.ptr + sort_bytes + 256);
	bool ema_done = false;
	// the dealt entries first where the partition follows: its slabs then merge with what is there and finish the update
	auto dealt_splat = [&](bool merge) -> int {
		int rc2 = fill_u32(list_count, 1, 0u, st);
		if (rc2 != SRF_OK) return rc2;
		uint32_t log2_cells = 0;
		while ((1u << log2_cells) < nc) ++log2_cells;
		const dim3 grid(nc / DEALT_CELLS), block(256);
		const size_t lds = (size_t)s->P.n_cascades * DEALT_CELLS * sizeof(uint32_t);
#define SRF_DEALT(H, M) hipLaunchKernelGGL((k_splat_dealt<H, M>), grid, block, lds, st, nc, log2_cells, s->P.n_cascades, n_dealt / nc, grid_indices, padded_output_width, grid_densities, \
                                           density_activation, s->P.min_cone_stepsize, (uint32_t*)s->density_grid_current, list_count, list)
		if (half) { if (merge) SRF_DEALT(true, true); else SRF_DEALT(true, false); }
		else { if (merge) SRF_DEALT(false, true); else SRF_DEALT(false, false); }
#undef SRF_DEALT
		SRF_LAUNCH_CHECK();
		return SRF_OK;
	};
	auto listed_splat = [&]() -> int {
		hipLaunchKernelGGL(k_splat_listed, dim3(1024), dim3(256), 0, st, (const uint32_t*)list_count, (const U2*)list, s->n_total, (uint32_t*)s->density_grid_current);
		SRF_LAUNCH_CHECK();
		return SRF_OK;
	};
	if (partition) {
		if (n_dealt) {
			rc = dealt_splat(false);
			if (rc == SRF_OK) rc = listed_splat();
			if (rc != SRF_OK) return rc;
		}
		const uint32_t n_buckets = div_up(n_part_slabs, PART_BUCKET_SLABS);
		uint32_t* counts = (uint32_t*)s->ws.ptr;
		PartTables T;
		T.starts = counts + n_part_slabs;
		T.slab_cursor = T.starts + n_part_slabs + 1;
		T.bucket_cursor = T.slab_cursor + n_part_slabs;
		T.chunk_first = T.bucket_cursor + PART_MAX_BUCKETS;
		const uint32_t* starts = T.starts;
		U2* pairs_a = (U2*)((char*)s->ws.ptr + part_words);
		U2* pairs = pairs_a + align_up((size_t)n, 32);
		rc = fill_u32(counts, n_part_slabs, 0u, st);
		if (rc != SRF_OK) return rc;
		int dev = 0, n_cu = 0;
		SRF_HIP(hipGetDevice(&dev));
		SRF_HIP(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
		uint32_t groups = (uint32_t)n_cu * 2u;               // two workgroups of 1024 threads fill a CU
		if (groups > div_up(n, PART_THREADS * 16u)) groups = div_up(n, PART_THREADS * 16u);
		hipLaunchKernelGGL(k_part_count, dim3(groups), dim3(PART_THREADS), (size_t)n_part_slabs * sizeof(uint32_t), st, n, rest_indices, s->n_total, n_part_slabs, counts);
		SRF_LAUNCH_CHECK();
		hipLaunchKernelGGL(k_part_scan, dim3(1), dim3(PART_THREADS), 0, st, n_part_slabs, n_buckets, (const uint32_t*)counts, T);
		SRF_LAUNCH_CHECK();
		const uint32_t n_chunks = div_up(n, PART_CHUNK);
		const uint32_t pass_groups = n_chunks + n_buckets < (uint32_t)n_cu * 8u ? n_chunks + n_buckets : (uint32_t)n_cu * 8u;      // pass 2 has at most n_chunks + n_buckets chunks
#define SRF_PART_PASS(L, H) hipLaunchKernelGGL((k_part_pass<L, H>), dim3(pass_groups), dim3(PART_PASS_THREADS), 0, st, n, rest_indices, padded_output_width, rest_densities, \
                                               density_activation, s->P.min_cone_stepsize, s->n_total, n_part_slabs, n_buckets, T, (const U2*)pairs_a, L == 1 ? pairs_a : pairs)
		if (half) SRF_PART_PASS(1, true); else SRF_PART_PASS(1, false);
		SRF_LAUNCH_CHECK();
		SRF_PART_PASS(2, false);
		SRF_LAUNCH_CHECK();
#undef SRF_PART_PASS
		const size_t slab_lds = (size_t)PART_SLAB_CELLS * sizeof(uint32_t);
		if (n_dealt)
			hipLaunchKernelGGL((k_part_slabs<true, true>), dim3(n_part_slabs), dim3(PART_THREADS), slab_lds, st, s->n_total, (const uint32_t*)starts, (const U2*)pairs,
			                   (uint32_t*)s->density_grid_current, s->P.ema_decay, s->density_grid);
		else
			hipLaunchKernelGGL((k_part_slabs<true, false>), dim3(n_part_slabs), dim3(PART_THREADS), slab_lds, st, s->n_total, (const uint32_t*)starts, (const U2*)pairs,
			                   (uint32_t*)s->density_grid_current, s->P.ema_decay, s->density_grid);
		SRF_LAUNCH_CHECK();
		ema_done = true;
	} else {
		if (sorted_splat) {
			uint32_t* thick = (uint32_t*)s->ws.ptr;
			uint32_t* cells_sorted = (uint32_t*)((char*)s->ws.ptr + arr);
			uint32_t* thick_sorted = (uint32_t*)((char*)s->ws.ptr + 2 * arr);
			void* temp = (char*)s->ws.ptr + 3 * arr;
			if (half)
				hipLaunchKernelGGL(k_splat_values<true>, dim3(div_up(n, 256)), dim3(256), 0, st, n, padded_output_width, rest_densities, density_activation, s->P.min_cone_stepsize, thick);
			else
				hipLaunchKernelGGL(k_splat_values<false>, dim3(div_up(n, 256)), dim3(256), 0, st, n, padded_output_width, rest_densities, density_activation, s->P.min_cone_stepsize, thick);
			SRF_LAUNCH_CHECK();
			SRF_HIP(hipcub::DeviceRadixSort::SortPairs(temp, temp_bytes, rest_indices, cells_sorted, (const uint32_t*)thick, thick_sorted, (int)n, (int)SPLAT_SLAB_BITS, end_bit, st));
			hipLaunchKernelGGL(k_splat_slabs, dim3(div_up(s->n_total, SPLAT_SLAB_CELLS)), dim3(256), 0, st, n, s->n_total, (const uint32_t*)cells_sorted,
			                   (const uint32_t*)thick_sorted, (uint32_t*)s->density_grid_current);
			SRF_LAUNCH_CHECK();
		}
		if (n_dealt) {
			rc = dealt_splat(sorted_splat);
			if (rc != SRF_OK) return rc;
		}
		if (!sorted_splat && n) {
			if (half)
				hipLaunchKernelGGL(k_splat_grid_samples<true>, dim3(div_up(n, 256)), dim3(256), 0, st, n, rest_indices,
				                   padded_output_width, rest_densities, density_activation, s->P.min_cone_stepsize, s->density_grid_current);
			else
				hipLaunchKernelGGL(k_splat_grid_samples<false>, dim3(div_up(n, 256)), dim3(256), 0, st, n, rest_indices,
				                   padded_output_width, rest_densities, density_activation, s->P.min_cone_stepsize, s->density_grid_current);
			SRF_LAUNCH_CHECK();
		}
		if (n_dealt) {
			rc = listed_splat();
			if (rc != SRF_OK) return rc;
		}
	}
	if (!ema_done) {
		const uint32_t n_vec4 = s->n_total / 4;
		const uint32_t blocks = div_up(n_vec4, 256) < 8192 ? div_up(n_vec4, 256) : 8192;
		hipLaunchKernelGGL(k_ema_grid, dim3(blocks), dim3(256), 0, st, n_vec4, (const float4*)s->density_grid_current, s->P.ema_decay, (float4*)s->density_grid);
		SRF_LAUNCH_CHECK();
	}
	++s->i_step;
	return SRF_OK;
}

int srf_sampler_update_grid_bitfield(srf_sampler_t* s, void* stream) {
	SRF_REQUIRE(s, "srf_sampler_update_grid_bitfield: NULL sampler");
	SRF_REQUIRE(s->P.use_grid, "srf_sampler_update_grid_bitfield: sampler has no grid");
	hipStream_t st = (hipStream_t)stream;
	const Params& P = s->P;
	const uint32_t n_tiles = div_up(P.n_cells, 1024);
	const uint32_t n_level2 = div_up(n_tiles, 1024);
	int rc = s->ws.reserve(((size_t)n_tiles + n_level2 + 2) * sizeof(double));
	if (rc != SRF_OK) return rc;
	double* part_a = (double*)s->ws.ptr;
	double* part_b = part_a + n_tiles;
	{
		const uint32_t blocks = n_tiles < 4096 ? n_tiles : 4096;
		hipLaunchKernelGGL(k_mean_tile_partials, dim3(blocks), dim3(256), 0, st, (const float*)s->density_grid, P.n_cells, (float)P.n_cells, n_tiles, part_a);
		SRF_LAUNCH_CHECK();
		double* src = part_a; double* dst = part_b;
		uint32_t n = n_tiles;
		for (;;) {
			const uint32_t nb = div_up(n, 1024);
			hipLaunchKernelGGL(k_reduce_pairs_f64, dim3(nb), dim3(512), 0, st, (const double*)src, n, nb > 1 ? dst : (double*)nullptr,
			                   nb > 1 ? (float*)nullptr : s->density_grid_mean);
			SRF_LAUNCH_CHECK();
			if (nb == 1) break;
			n = nb;
			double* t = src; src = dst; dst = t;
		}
	}
	{
		const uint32_t n_chunks = div_up(s->n_total, 512);
		const uint32_t waves_per_block = 4;
		const uint32_t blocks = div_up(n_chunks, waves_per_block) < 16384 ? div_up(n_chunks, waves_per_block) : 16384;
		hipLaunchKernelGGL(k_grid_to_bitfield, dim3(blocks), dim3(256), 0, st, (const float*)s->density_grid, s->n_total,
		                   (const float*)s->density_grid_mean, P.min_optical_thickness, s->density_grid_bitfield);
		SRF_LAUNCH_CHECK();
	}
	if (P.griddist_type == SRF_GRID_WARPED_EXP || P.griddist_type == SRF_GRID_METRIC_EXP) {
		const uint32_t n = P.n_cells / 64;
		for (uint32_t level = 1; level < P.n_cascades && n > 0; ++level) {
			hipLaunchKernelGGL(k_bitfield_max_pool, dim3(div_up(n, 256)), dim3(256), 0, st, n, P.grid_size[0] / 8, P.grid_size[1] / 8, P.grid_size[2] / 8,
			                   (const uint8_t*)(s->density_grid_bitfield + (size_t)P.n_cells * (level - 1) / 8),
			                   s->density_grid_bitfield + (size_t)P.n_cells * level / 8);
			SRF_LAUNCH_CHECK();
		}
	}
	return rebuild_skip_table(s, st);
}

} // extern "C"
