// RayMarcher: training compositing (forward, loss, ordered compaction, backward), one wavefront per item.
#include "srf_internal.h"
#include "srf_bodies.h"
#include "srf_composite_wave.h"
#include "srf_chain.h"

namespace srf {

// Device scratch of the wave-per-item kernel.  The words that have to be zero when a call begins lie first, where they stay
// whatever the number of rays; copies of the call's arguments follow them (written by the preparing kernel for the main
// kernel's out-of-line path, which reads them from memory instead of having them passed in registers).
struct WaveLayout { size_t off_status, off_seg, off_prefix, off_desc, bytes; };
SRF_HD constexpr WaveLayout wave_layout(uint32_t n_rays) {
	const size_t cap = wv::max_items(n_rays);
	WaveLayout L = {};
	L.off_status = 1024;
	L.off_seg = (L.off_status + cap * 8 + 255) / 256 * 256;
	L.off_prefix = (L.off_seg + (cap + 63) / 64 * 8 * SEG_STRIDE + 255) / 256 * 256;
	L.off_desc = (L.off_prefix + (cap + 63) / 64 * 8 + 255) / 256 * 256;
	L.bytes = (L.off_desc + cap * sizeof(wv::ItemDesc) + 255) / 256 * 256;
	return L;
}
ChainScratch wave_scratch_at(void* base, uint32_t n_rays, uint32_t* host_error, uint32_t spin_limit) {
	const WaveLayout L = wave_layout(n_rays);
	ChainScratch S = {};
	uint32_t* words = (uint32_t*)base;
	S.ticket = words; S.disorder = words + 1; S.exits = words + 2;
	S.initial = words + 8; S.error = words + 9; S.n_items = words + 10; S.stride = words + 11;
	static_assert(128 + sizeof(fused::Args) <= 512 && 512 + sizeof(ChainScratch) <= 1024, "the argument copies fit the header");
	S.args_copy = (char*)base + 128;
	S.scratch_copy = (char*)base + 512;
	S.item_status = (unsigned long long*)((char*)base + L.off_status);
	S.seg_status = (unsigned long long*)((char*)base + L.off_seg);
	S.seg_prefix = (unsigned long long*)((char*)base + L.off_prefix);
	S.item_desc = (char*)base + L.off_desc;
	S.host_error = host_error;
	S.spin_limit = spin_limit;
	return S;
}

// ---- one wavefront per item ---------------------------------------------------------------------
// The phases are in srf_composite_wave.h.  k_wave_prepare finds the stride of the sample windows and every item's
// first ray, checks that the rays are laid out in increasing order and clears the status words of the ordered-offset
// chain.  k_composite_waves: workgroups of four wavefronts draw rounds of four consecutive items from a counter, so an
// item only ever waits for items that a resident workgroup holds or has finished, however many workgroups the device
// runs at once; a round's wavefronts work side by side without meeting until the next draw.
constexpr uint32_t WAVES_THREADS = wv::ITEMS_PER_TICKET * WAVE;
constexpr uint32_t PREPARE_THREADS = 256;

__global__ void __launch_bounds__(PREPARE_THREADS) k_wave_prepare(fused::Args A, const uint32_t* __restrict__ n_rays_counter, ChainScratch S, const uint32_t* __restrict__ counter) {
	const uint32_t i = blockIdx.x * PREPARE_THREADS + threadIdx.x;
	const uint32_t cap = wv::max_items(A.K.n_rays);
	const uint32_t counter_now = *n_rays_counter;
	const uint32_t n_active = counter_now < A.K.n_rays ? counter_now : A.K.n_rays;
	if (i < cap) {
		S.item_status[i] = 0ull;
		if (i % WAVE == 0) { S.seg_status[(size_t)(i / WAVE) * SEG_STRIDE] = 0ull; S.seg_prefix[i / WAVE] = 0ull; }
	}
	const wv::Windows W = wv::windows_of(n_active, A.ray_coord_indices, cap);
	if (i == 0) {
		*S.initial = *counter; *S.error = 0u; *S.n_items = W.n_items; *S.stride = W.stride;
		*(fused::Args*)S.args_copy = A;
		*(ChainScratch*)S.scratch_copy = S;
	}
	bool in_order = true;
	if (i < n_active) in_order = wv::prepare_ray(i, n_active, A.ray_coord_indices, W, cap, (wv::ItemDesc*)S.item_desc);
	if (__ballot(!in_order) != 0ull && lane_id() == 0) atomicOr(S.disorder, 1u);
}

// the rays a wavefront takes through its LDS window together: rays [rb, rb + nb), nb <= 64
struct WaveBatch {
	uint32_t rb, nb;           // the same in every lane, like s0, range and n_chunks
	uint64_t s0;               // first sample
	uint32_t range, n_chunks;  // samples from s0 to the end of the last ray; windows that takes
	uint32_t n, rbase;         // the lane's ray: its samples, and where the first lies in the range
	Float4 tgt;                // its target colour
};

// what one lane's accesses to the wavefront's LDS window leave must be there for the other lanes' later ones: the
// wavefront's LDS operations are carried out in the order they are issued, so all this has to keep is the compiler's order
__device__ __forceinline__ void wave_sync() {
	__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
	__builtin_amdgcn_wave_barrier();
}

__device__ __forceinline__ WaveBatch wave_load_batch(uint32_t lane, uint32_t rb, uint32_t nb, const fused::Args& A) {
	WaveBatch B;
	B.rb = rb; B.nb = nb;
	uint32_t n = 0, base = 0;
	B.tgt = mk4(0.f, 0.f, 0.f, 0.f);
	if (lane < nb) {
		const U2 rec = *(const U2*)(A.ray_coord_indices + 2 * (size_t)(rb + lane));
		B.tgt = *(const Float4*)(A.rays_rgba + 4 * (size_t)(rb + lane));
		n = rec.x; base = rec.y;
	}
	const uint32_t last = nb ? nb - 1 : 0u;
	const uint32_t s0 = nb ? lane_value_u32(base, 0) : 0u;
	const uint32_t end = nb ? lane_value_u32(base, last) + lane_value_u32(n, last) : 0u;
	B.s0 = s0;
	B.range = end - s0;
	B.n_chunks = div_up(B.range, wv::WIN);
	B.n = n;
	B.rbase = lane < nb ? base - s0 : B.range;
	return B;
}

__device__ __forceinline__ void wave_chain(uint32_t lane, const WaveBatch& B, uint32_t chunk_lo, float thr, wv::Lds& w, wv::RayState& rs) {
	uint32_t k0, k1;
	wv::chain_span(B.n, B.rbase, chunk_lo, &k0, &k1);
	const uint32_t steps = wave_max_fast(k1 - k0);
	for (uint32_t j = 0; j < steps; j += wv::CHAIN_UNROLL) {
		if (__ballot(k0 + j < k1 && rs.dead == 0u) == 0ull) break;     // nobody has a live step left
		wv::chain_stretch(lane, j, k0, k1, B.rbase, chunk_lo, thr, w, rs);
	}
}

// rows and chain of every chunk of the batch; the last chunk's records (and `st`) are left in place.
// ONE_CHUNK: the batch's samples fit the window (known when the code is compiled: no loop)
template <bool HI, bool PL, bool ONE_CHUNK>
__device__ __forceinline__ void wave_forward(uint32_t lane, const WaveBatch& B, const fused::Args& A, wv::Lds& w, fused::SlotState<wv::G, HI>& st, wv::RayState& rs) {
	wv::ray_reset(rs);
	const uint32_t n_chunks = ONE_CHUNK || B.n_chunks == 0 ? 1u : B.n_chunks;
	for (uint32_t c = 0; c < n_chunks; ++c) {
		const uint32_t chunk_lo = c * wv::WIN;
		wave_sync();
		wv::rows_load<HI>(lane, A, B.s0, B.range, chunk_lo, st);
		wv::rows_alpha<HI, PL>(lane, A, w, B.range, chunk_lo, st);
		wave_sync();
		wave_chain(lane, B, chunk_lo, A.K.thr, w, rs);
	}
}

// After wave_forward: colours, loss and offsets of the batch's rays, then the gradients.  cbase_of_batch() is called once
// the number of samples every ray keeps is known and gives the compacted offset of the batch's first ray (CHAIN_FAILED: none).
template <bool HI, bool HO, bool PL, bool ONE_CHUNK, class Offset>
__device__ __forceinline__ void wave_backward(uint32_t lane, const WaveBatch& B, const fused::Args& A, wv::Lds& w, fused::SlotState<wv::G, HI>& st, wv::RayState& rs,
                                              Offset cbase_of_batch) {
	const bool mine = lane < B.nb;
	const uint32_t n_fwd = mine ? rs.cnt : 0u;
	const uint32_t incl = wave_inclusive_scan_fast(n_fwd);
	const uint32_t total = lane_value_u32(incl, WAVE - 1);
	float loss = 0.f;
	const uint32_t first = cbase_of_batch(total, [&]() { if (mine) loss = wv::finish_lane(lane, B.rb + lane, B.n, A, w, rs, B.tgt); });
	const uint32_t cbase = first == CHAIN_FAILED ? CHAIN_FAILED : first + incl - n_fwd;
	if (mine) wv::commit_lane(lane, B.rb + lane, n_fwd, B.rbase, cbase, loss, A, w); else wv::commit_none(lane, w);
	wave_sync();
	if (ONE_CHUNK || B.n_chunks <= 1) {
		wv::rows_grads<HI, HO, PL>(lane, A, w, B.s0, B.range, 0u, st);
	} else {
		wv::ray_reset(rs);
		for (uint32_t c = 0; c < B.n_chunks; ++c) {
			const uint32_t chunk_lo = c * wv::WIN;
			wave_sync();
			wv::rows_load<HI>(lane, A, B.s0, B.range, chunk_lo, st);
			wv::rows_alpha<HI, PL>(lane, A, w, B.range, chunk_lo, st);
			wave_sync();
			wave_chain(lane, B, chunk_lo, A.K.thr, w, rs);
			wave_sync();
			wv::rows_grads<HI, HO, PL>(lane, A, w, B.s0, B.range, chunk_lo, st);
		}
	}
	wave_sync();
}

// The item's total goes to the items after it, and the totals of the items before it make its offset; meanwhile() runs
// between the two, while the predecessors' words are on their way.
template <class Meanwhile>
__device__ __forceinline__ uint32_t item_offset(const ChainScratch& S, uint32_t item, uint32_t total, Meanwhile meanwhile) {
	chain_publish(S, item, total);
	const ChainPeek peek = chain_peek(S, item);
	meanwhile();
	return chain_resolve(S, item, total, peek);
}

// The workgroup's LDS: one window per wavefront, and the round numbers the workgroup has drawn (a ring: this round's,
// the next one's, and the one being drawn).
__shared__ wv::Lds g_window[wv::ITEMS_PER_TICKET];
__shared__ uint32_t g_round_slot[4];
constexpr uint32_t NO_ITEM = 0xffffffffu;

// What an item's out-of-line code gets; the call's arguments it reads from the copies in device memory (see wave_layout).
struct ItemCall {
	uint32_t item, n_items;
	uint32_t n_active;
	float mean_density;
	const void* args_copy;
	const void* scratch_copy;
	uint32_t* compacted_counter;
	uint32_t wave;              // which of the workgroup's windows
};

// (through the constant address space: the table is not written while this kernel runs, and a load from there at an address
// that is the same in every lane goes through the scalar unit, whose results nothing else has to wait for)
__device__ __forceinline__ wv::ItemDesc item_desc(const ChainScratch& S, uint32_t item) {
	typedef const __attribute__((address_space(4))) uint32_t* ConstWords;
	ConstWords p = (ConstWords)(uintptr_t)((const wv::ItemDesc*)S.item_desc + item);
	wv::ItemDesc d;
	d.r0 = p[0]; d.s0 = p[1]; d.r_end = p[2]; d.s_end = p[3];
	return d;
}
__device__ __forceinline__ bool item_fits(const wv::ItemDesc& d) { return d.r_end - d.r0 <= WAVE && d.s_end - d.s0 <= wv::WIN; }

__device__ __forceinline__ void item_done(uint32_t item, uint32_t n_items, uint32_t* compacted_counter, uint32_t prefix, uint32_t total) {
	if (item == n_items - 1 && lane_id() == 0) *compacted_counter = prefix == CHAIN_FAILED ? CHAIN_FAILED : prefix + total;
}

// The lane's ray of an item that fits the window: its record (samples, first sample) and its target colour, as they are
// loaded.  The item has rays; a lane past them gets a copy of the last one (ray_rec_mask makes it a ray without samples).
struct RayRec { U2 rec; Float4 tgt; };
__device__ __forceinline__ RayRec ray_rec_load(uint32_t lane, const wv::ItemDesc& d, const fused::Args& A) {
	const uint32_t n_r = d.r_end - d.r0;
	const uint32_t i = d.r0 + (lane < n_r ? lane : n_r - 1);
	RayRec r;
	r.rec = *(const U2*)((const char*)A.ray_coord_indices + (size_t)d.r0 * 8 + (uint32_t)((i - d.r0) * 8u));
	r.tgt = *(const Float4*)((const char*)A.rays_rgba + (size_t)d.r0 * 16 + (uint32_t)((i - d.r0) * 16u));
	return r;
}

// Every other item: a batch in several chunks, more rays than lanes (every batch is counted first, then every batch runs
// again with its offset known), and, when the call's rays are not laid out in order, rays anywhere in the sample buffer
// (one lane per ray, straight from memory: ray_marcher.cu:57-201 as it stands).  Out of line, with the call's arguments
// read from their copies in memory, so that the common path's registers are allocated without regard to this one.
template <bool HI, bool HO, bool PL>
__device__ __noinline__ void wave_item_general(ItemCall c, bool in_order) {
	const fused::Args A0 = *(const fused::Args*)c.args_copy;
	const ChainScratch S = *(const ChainScratch*)c.scratch_copy;
	fused::Args A = A0;
	A.n_active = c.n_active; A.mean_density = c.mean_density;
	wv::Lds& w = g_window[c.wave];
	const uint32_t lane = lane_id();
	const uint32_t item = c.item;
	uint32_t r0, n_r;
	if (in_order) {
		const wv::ItemDesc d = item_desc(S, item);
		r0 = SRF_UNIFORM_U32(d.r0); n_r = SRF_UNIFORM_U32(d.r_end) - r0;
	} else {
		r0 = item * wv::GROUP;
		n_r = c.n_active - r0 < wv::GROUP ? c.n_active - r0 : wv::GROUP;
	}
	uint32_t prefix = 0, item_total = 0;
	if (in_order) {
		fused::SlotState<wv::G, HI> st;
		wv::RayState rs;
		const uint32_t n_batches = n_r ? div_up(n_r, WAVE) : 1u;
		uint32_t run = 0;
		// with one batch: its forward pass, the chain of offsets, its gradients.  With several: a first pass that only counts
		for (uint32_t pass = n_batches > 1 ? 0u : 1u; pass < 2u; ++pass) {
			for (uint32_t b = 0; b < n_batches; ++b) {
				const WaveBatch B = wave_load_batch(lane, r0 + b * WAVE, n_r - b * WAVE < WAVE ? n_r - b * WAVE : WAVE, A);
				wave_forward<HI, PL, false>(lane, B, A, w, st, rs);
				if (pass == 0u) { item_total += wave_sum_fast(lane < B.nb ? rs.cnt : 0u); continue; }
				uint32_t batch_total = 0;
				wave_backward<HI, HO, PL, false>(lane, B, A, w, st, rs, [&](uint32_t t, auto&& meanwhile) -> uint32_t {
					batch_total = t;
					if (n_batches > 1) { meanwhile(); return run; }
					item_total = t;
					prefix = item_offset(S, item, t, meanwhile);
					return prefix;
				});
				if (run != CHAIN_FAILED) run += batch_total;
			}
			if (pass == 0u) { prefix = item_offset(S, item, item_total, []() {}); run = prefix; }
		}
	} else {
		const uint32_t i = r0 + lane;
		const bool mine = lane < n_r;
		FwdRay fw;
		uint32_t nf = 0;
		if (mine) loss_forward_body<HI>(i, A.K, A.rays_rgba, A.n_active, A.ray_coord_indices, A.dt_arr, A.net, &fw, &nf, A.rgb_ray_out);
		const uint32_t incl = wave_inclusive_scan_fast(nf);
		item_total = lane_value_u32(incl, WAVE - 1);
		prefix = item_offset(S, item, item_total, []() {});
		const uint32_t cbase = prefix == CHAIN_FAILED ? CHAIN_FAILED : prefix + incl - nf;
		if (mine) loss_backward_body<HI, HO>(i, A.K, A.n_active, A.ray_coord_indices, A.dt_arr, A.coords, A.compacted_coords, A.net, A.dloss, A.loss_output,
		                                     A.mean_density, fw, nf, cbase, nullptr);
	}
	item_done(c.item, c.n_items, c.compacted_counter, prefix, item_total);
}

// two workgroups per CU: eight wavefronts, two per SIMD, with up to 256 registers each
#define SRF_WAVES_OCCUPANCY __attribute__((amdgpu_waves_per_eu(2, 2)))
constexpr uint32_t WAVES_WORKGROUPS_PER_CU = 2;

// The common item (at most 64 rays laid out in order, samples that fit the window in one piece) runs in the kernel's own
// loop, with the next item's description, ray records and samples asked for while this one is worked on:
//
//   alpha          {alpha, colour} of every sample to the window (the samples were loaded during the previous item)
//   chain          one lane per ray; the item's total goes out to the items after it
//   look ahead     the next item's ray records and samples are asked for; the totals of the items before this one too
//   finish, grads  loss and its gradient per ray; the samples' gradients, staged in the window
//   offsets        the earlier items' totals have come in by now: compacted offsets, the rays' records and losses
//   stores         the next item's samples are waited for first (so that nothing ever waits for these stores), then the
//                  kept samples' gradients go out
//
// A workgroup draws the number of a round two rounds ahead, so every wavefront knows its next item when a round begins.
template <bool HI, bool HO, bool PL>
__global__ void __launch_bounds__(WAVES_THREADS) SRF_WAVES_OCCUPANCY k_composite_waves(fused::Args A, const uint32_t* __restrict__ n_rays_counter, const float* __restrict__ mean_density_ptr,
                                                                                       ChainScratch S, uint32_t* __restrict__ compacted_counter) {
	const uint32_t tid = threadIdx.x, lane = lane_id();
	const uint32_t wave = SRF_UNIFORM_U32(tid / WAVE);
	// (what the kernel reads once goes to scalar registers here: a value that sits in a vector register since a load before
	// the loop is waited for again, with everything else under way, wherever the loop uses it)
	const uint32_t counter_now = SRF_UNIFORM_U32(*n_rays_counter);
	A.mean_density = mean_density_ptr ? srf_u2f(SRF_UNIFORM_U32(srf_f2u(*mean_density_ptr))) : 0.f;
	A.n_active = counter_now < A.K.n_rays ? counter_now : A.K.n_rays;
	ItemCall c;
	c.mean_density = A.mean_density; c.n_active = A.n_active;
	c.args_copy = S.args_copy; c.scratch_copy = S.scratch_copy; c.compacted_counter = compacted_counter; c.wave = wave;
	const bool in_order = SRF_UNIFORM_U32(*S.disorder) == 0u;
	const uint32_t n_items = in_order ? SRF_UNIFORM_U32(*S.n_items) : div_up(A.n_active, wv::GROUP);
	c.n_items = n_items;
	const uint32_t n_rounds = div_up(n_items, wv::ITEMS_PER_TICKET);
	const uint32_t initial = SRF_UNIFORM_U32(*S.initial);          // the compacted counter's value before the call
	wv::Lds& w = g_window[wave];
	wv::RayLds2& rl = w.staged();
#ifdef SRF_KERNEL_TIMING
	unsigned long long wt[12] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
	unsigned long long wt_prev_ = clock64();
#define SRF_WT(k) do { const unsigned long long now_ = clock64(); wt[k] += now_ - wt_prev_; wt_prev_ = now_; } while (0)
#else
#define SRF_WT(k) ((void)0)
#endif
	if (tid == 0) { g_round_slot[0] = atomicAdd(S.ticket, 1u); g_round_slot[1] = atomicAdd(S.ticket, 1u); }
	// Carried from one round to the next: the item asked for during the previous one (its description, ray records and
	// samples, all of them arrived), if any.
	wv::RowData<HI> in;
	RayRec rec;
	wv::ItemDesc d;
	uint32_t item_here = NO_ITEM;
	rec.rec = {}; rec.tgt = mk4(0.f, 0.f, 0.f, 0.f);
	d.r0 = d.s0 = d.r_end = d.s_end = 0;
	#pragma unroll
	for (uint32_t j = 0; j < wv::ROWS; ++j) { in.raw[j] = {}; in.dt[j] = 0.f; }
	// Loads of an item's ray records and samples are issued whether or not there is such an item (without one they read the
	// first ray's record over and over), so that the code has no branch that a register's value would have to be carried round.
	auto records_of = [&](bool there, const wv::ItemDesc& dd) -> RayRec {
		wv::ItemDesc safe;
		safe.r0 = there ? dd.r0 : 0u; safe.r_end = there ? dd.r_end : 1u; safe.s0 = 0; safe.s_end = 0;
		return ray_rec_load(lane, safe, A);
	};
	auto samples_of = [&](bool there, const wv::ItemDesc& dd, uint32_t j0, uint32_t n, wv::RowData<HI>& out) {
		fused::Args B = A;
		if (!there) { B.net = A.ray_coord_indices; B.dt_arr = (const float*)A.ray_coord_indices; }
		wv::fit_rows_load_some<HI>(lane, j0, n, B, there ? dd.s0 : 0u, there ? dd.s_end - dd.s0 : 1u, out);
	};
	for (uint32_t round = 0;; ++round) {
		__syncthreads();
		SRF_WT(9);
		const uint32_t t = SRF_UNIFORM_U32(g_round_slot[round & 3u]), t1 = SRF_UNIFORM_U32(g_round_slot[(round + 1u) & 3u]);
		if (t >= n_rounds) break;
		uint32_t drawn;                                          // (only thread 0's is ever looked at; no value that the load's result would have to be merged with)
		if (tid == 0) drawn = atomicAdd(S.ticket, 1u);           // the round after the next; looked at after the chain
		const uint32_t item = t * wv::ITEMS_PER_TICKET + wave;
		uint32_t item1 = t1 < n_rounds ? t1 * wv::ITEMS_PER_TICKET + wave : NO_ITEM;
		if (item1 != NO_ITEM && (item1 >= n_items || !in_order)) item1 = NO_ITEM;
		// this item: asked for during the previous one, or fetched now
		bool fits = false;
		if (item < n_items && in_order) {
			if (__builtin_expect(item_here != item, 0)) {
				d = item_desc(S, item);
				if (item_fits(d)) {
					rec = records_of(d.r_end != d.r0, d);
					samples_of(d.s_end != d.s0, d, 0, wv::ROWS, in);
					// (waited for here, so that where this path joins the common one no load is under way)
					asm volatile("" : "+v"(rec.rec.x), "+v"(rec.tgt.x));
					#pragma unroll
					for (uint32_t j = 0; j < wv::ROWS; ++j) asm volatile("" : "+v"(in.raw[j].x), "+v"(in.dt[j]));
				}
			}
			fits = item_fits(d);
		}
		if (__builtin_expect(!fits, 0)) {
			if (tid == 0) g_round_slot[(round + 2u) & 3u] = drawn;
			c.item = item;
			if (item < n_items) wave_item_general<HI, HO, PL>(c, in_order);
			// nothing is carried across that call
			item_here = NO_ITEM;
			rec.rec = {}; rec.tgt = mk4(0.f, 0.f, 0.f, 0.f);
			d.r0 = d.s0 = d.r_end = d.s_end = 0;
			#pragma unroll
			for (uint32_t j = 0; j < wv::ROWS; ++j) { in.raw[j] = {}; in.dt[j] = 0.f; }
			continue;
		}
		const uint32_t range = d.s_end - d.s0, n_r = d.r_end - d.r0;
		wv::ItemDesc d1;
		d1.r0 = d1.s0 = d1.r_end = d1.s_end = 0;
		if (item1 != NO_ITEM) d1 = item_desc(S, item1);          // (needed after the chain)
		float alpha[wv::ROWS];
		SRF_WT(0);
		// alpha, chain
		wave_sync();
		wv::fit_rows_alpha<HI, PL>(lane, A, w.S, w.owner, range, in, alpha);
		wave_sync();
		SRF_WT(1);
		const bool mine = lane < n_r;
		const uint32_t ray_n = mine ? rec.rec.x : 0u;
		const uint32_t rbase = mine ? rec.rec.y - d.s0 : range;
		wv::RayState rs;
		wv::ray_reset(rs);
		{
			// two stretches a turn: each one's records are read while the one before it is worked on
			const uint32_t steps = wave_max_fast(ray_n);
			wv::ChainReads ca, cb;
			wv::chain_read(0u, 0u, ray_n, rbase, 0u, w, ca);
			for (uint32_t j = 0; j < steps; j += 2 * wv::CHAIN_UNROLL) {
				if (__ballot(j < ray_n && rs.dead == 0u) == 0ull) break;     // nobody has a live step left
				wv::chain_read(j + wv::CHAIN_UNROLL, 0u, ray_n, rbase, 0u, w, cb);
				wv::chain_apply(lane, A.K.thr, w, rs, ca);
				wv::chain_read(j + 2 * wv::CHAIN_UNROLL, 0u, ray_n, rbase, 0u, w, ca);
				wv::chain_apply(lane, A.K.thr, w, rs, cb);
			}
		}
		SRF_WT(2);
		if (tid == 0) g_round_slot[(round + 2u) & 3u] = drawn;
		// the item's total goes out; the earlier items' totals and the next item are asked for
		const uint32_t n_fwd = mine ? rs.cnt : 0u;
		const uint32_t incl = wave_inclusive_scan_fast(n_fwd);
		const uint32_t item_total = lane_value_u32(incl, WAVE - 1);
		chain_publish(S, item, item_total);
		const ChainPeek peek = chain_peek(S, item, initial);
		const bool fits1 = item1 != NO_ITEM && item_fits(d1);
		wv::RowData<HI> ahead;
		const RayRec rec_ahead = records_of(fits1 && d1.r_end != d1.r0, d1);
		SRF_WT(3);
		// finish, gradients; the next item's samples are asked for four rows at a time, into the registers that this item's rows leave
		float loss = 0.f;
		if (mine) loss = wv::fit_finish_lane(lane, d.r0 + lane, ray_n, A, rl, rs, rec.tgt);
		wave_sync();
		SRF_WT(4);
		#pragma unroll
		for (uint32_t jb = 0; jb < wv::ROWS; jb += wv::ROW_BATCH) {
			wv::fit_rows_grads_some<HI, PL>(lane, jb, A, w.S, w.owner, rl, range, in, alpha);
			samples_of(fits1 && d1.s_end != d1.s0, d1, jb, wv::ROW_BATCH, ahead);
		}
		SRF_WT(5);
		// offsets
		const uint32_t prefix = chain_resolve(S, item, item_total, peek);
		SRF_WT(6);
		const uint32_t cbase = prefix == CHAIN_FAILED ? CHAIN_FAILED : prefix + incl - n_fwd;
		if (mine) wv::fit_commit_lane(lane, d.r0 + lane, n_fwd, rbase, cbase, prefix, loss, A, rl); else wv::fit_commit_none(lane, rl);
		item_done(item, n_items, compacted_counter, prefix, item_total);
		wave_sync();
		// What was asked for of the next item becomes the carried item here, before this item's stores go out: the
		// copies wait for the loads, and nothing will ever wait for the stores.
		const uint32_t s0_here = d.s0;
		rec.rec = rec_ahead.rec; rec.tgt = rec_ahead.tgt;
		#pragma unroll
		for (uint32_t j = 0; j < wv::ROWS; ++j) { in.raw[j] = ahead.raw[j]; in.dt[j] = ahead.dt[j]; }
		d = d1;
		item_here = fits1 ? item1 : NO_ITEM;
		asm volatile("" : "+v"(rec.rec.x), "+v"(rec.tgt.x));
		#pragma unroll
		for (uint32_t j = 0; j < wv::ROWS; ++j) asm volatile("" : "+v"(in.raw[j].x), "+v"(in.dt[j]));
		SRF_WT(7);
		wv::fit_rows_store<HO>(lane, A, w.S, w.owner, rl, s0_here, range, prefix);
		wave_sync();
		SRF_WT(8);
	}
#ifdef SRF_KERNEL_TIMING
	if (lane == 0) for (int k = 0; k < 11; ++k) atomicAdd((unsigned long long*)((char*)S.args_copy + 256) + k, wt[k]);
#endif
	// the last workgroup to leave puts the words back that the next call expects to be zero
	if (tid == 0) {
		__threadfence();
		if (atomicInc(S.exits, gridDim.x - 1u) == gridDim.x - 1u) { *S.ticket = 0u; *S.disorder = 0u; }
	}
#undef SRF_WT
}

// Workgroups of the wave-per-item kernel to launch: as many as the device runs at once (more would only queue up behind them;
// the kernel is correct with any number).
static int waves_grid(uint32_t* out) {
	static uint32_t per_device[64];
	int dev = 0;
	SRF_HIP(hipGetDevice(&dev));
	if (dev < 0 || dev >= 64) SRF_FAIL(SRF_ERR_INVALID, "compositing: device index out of range");
	if (!per_device[dev]) {
		hipDeviceProp_t prop;
		SRF_HIP(hipGetDeviceProperties(&prop, dev));
		per_device[dev] = (uint32_t)prop.multiProcessorCount * WAVES_WORKGROUPS_PER_CU;
	}
	*out = per_device[dev];
	return SRF_OK;
}

int launch_waves(const srf_loss_args* a, const LossConst& K, void* scratch, uint32_t* host_error, uint32_t spin_limit, const float* rays_rgba, const uint32_t* n_rays_counter,
                        uint32_t* ray_coord_indices, const float* dt, const float* coords, float* compacted_coords, uint32_t* n_compacted_coords_counter,
                        const void* network_output, void* dloss_doutput, float* loss_output, const float* density_grid_mean, float* rgb_ray_out, hipStream_t st) {
	const ChainScratch S = wave_scratch_at(scratch, a->n_rays, host_error, spin_limit);
	fused::Args A;
	A.K = K;
	A.n_active = 0;
	A.rays_rgba = rays_rgba; A.ray_coord_indices = ray_coord_indices; A.dt_arr = dt; A.coords = coords; A.compacted_coords = compacted_coords;
	A.net = network_output; A.dloss = dloss_doutput; A.loss_output = loss_output; A.rgb_ray_out = rgb_ray_out; A.mean_density = 0.f;
	const bool hin = a->network_output_dtype == SRF_DTYPE_F16, hout = a->dloss_dtype == SRF_DTYPE_F16;
	const bool plain = a->rgb_activation == SRF_ACT_NONE && a->density_activation == SRF_ACT_NONE;
	uint32_t resident = 0;
	int rc = waves_grid(&resident);
	if (rc != SRF_OK) return rc;
	const uint32_t most_rounds = div_up(wv::max_items(a->n_rays), wv::ITEMS_PER_TICKET);
	const dim3 grid(most_rounds < resident ? most_rounds : resident), block(WAVES_THREADS);
	hipLaunchKernelGGL(k_wave_prepare, dim3(div_up(a->n_rays + 2 * PREPARE_THREADS, PREPARE_THREADS)), dim3(PREPARE_THREADS), 0, st, A, n_rays_counter, S, (const uint32_t*)n_compacted_coords_counter);
	SRF_LAUNCH_CHECK();
#define SRF_WAVES(HI, HO, PL) hipLaunchKernelGGL((k_composite_waves<HI, HO, PL>), grid, block, 0, st, A, n_rays_counter, density_grid_mean, S, n_compacted_coords_counter)
#define SRF_WAVES_IO(PL) do { if (hin && hout) SRF_WAVES(true, true, PL); else if (hin) SRF_WAVES(true, false, PL); else if (hout) SRF_WAVES(false, true, PL); else SRF_WAVES(false, false, PL); } while (0)
#ifdef SRF_ONLY_BENCH_VARIANT      // (development builds: one variant compiles in a fraction of the time)
	if (!(plain && hin && !hout)) SRF_FAIL(SRF_ERR_UNSUPPORTED, "development build: fp16 in, fp32 out, no activations only");
	SRF_WAVES(true, false, true);
#else
	if (plain) SRF_WAVES_IO(true); else SRF_WAVES_IO(false);
#endif
#undef SRF_WAVES_IO
#undef SRF_WAVES
	SRF_LAUNCH_CHECK();
#ifdef SRF_KERNEL_TIMING
	{
		unsigned long long h[12];
		SRF_HIP(hipStreamSynchronize(st));
		SRF_HIP(hipMemcpy(h, (char*)S.args_copy + 256, sizeof(h), hipMemcpyDeviceToHost));
		SRF_HIP(hipMemset((char*)S.args_copy + 256, 0, sizeof(h)));
		static const char* names[11] = {"fetch", "alpha", "chain", "publish+ahead", "finish", "grads", "resolve", "commit+wait", "stores", "barrier", "-"};
		fprintf(stderr, "wave timing, cycles summed over wavefronts:");
		for (int k = 0; k < 11; ++k) fprintf(stderr, " %s %llu", names[k], h[k]);
		fprintf(stderr, "\n");
	}
#endif
	return SRF_OK;
}

size_t waves_scratch_bytes(uint32_t n_rays) { return wave_layout(n_rays).bytes; }
uint32_t* waves_error_word(void* scratch) { return wave_scratch_at(scratch, 0, nullptr, 0).error; }

} // namespace srf
