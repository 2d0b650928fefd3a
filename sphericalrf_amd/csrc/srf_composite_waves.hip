// RayMarcher: training compositing (forward, loss, ordered compaction, backward), one wavefront per item.
#include "srf_internal.h"
#include "srf_bodies.h"
#include "srf_composite_wave.h"
#include "srf_chain.h"

namespace srf {

// Device scratch of the wave-per-item kernel.  The words that have to be zero when a call begins lie first, where they stay
// whatever the number of rays; copies of the call's arguments follow them (written by the preparing kernel for the main
// kernel's out-of-line path, which reads them from memory instead of having them passed in registers).
struct WaveLayout { size_t off_status, off_seg, off_prefix, off_first, bytes; };
SRF_HD constexpr WaveLayout wave_layout(uint32_t n_rays) {
	const size_t cap = wv::max_items(n_rays);
	WaveLayout L = {};
	L.off_status = 1024;
	L.off_seg = (L.off_status + cap * 8 + 255) / 256 * 256;
	L.off_prefix = (L.off_seg + (cap + 63) / 64 * 8 * SEG_STRIDE + 255) / 256 * 256;
	L.off_first = (L.off_prefix + (cap + 63) / 64 * 8 + 255) / 256 * 256;
	L.bytes = (L.off_first + (cap + 1) * 4 + 255) / 256 * 256;
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
	S.item_first = (uint32_t*)((char*)base + L.off_first);
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
	if (i < n_active) in_order = wv::prepare_ray(i, n_active, A.ray_coord_indices, W, cap, S.item_first);
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

// The workgroup's LDS: one window per wavefront, and the numbers of the round of items in progress and of the next one.
__shared__ wv::Lds g_window[wv::ITEMS_PER_TICKET];
__shared__ uint32_t g_round_slot[2];

// What an item's code gets; the call's arguments it reads from the copies in device memory (see wave_layout).
struct ItemCall {
	uint32_t item, n_items;
	uint32_t n_active;
	float mean_density;
	const void* args_copy;
	const void* scratch_copy;
	uint32_t* compacted_counter;
	uint32_t wave;              // which of the workgroup's windows
	uint32_t round;             // of the workgroup; its first thread draws the next round's number while it works on this one's item
	uint32_t* ticket;
};

// The first thread of the workgroup asks for the next round's number at the start of its item and looks at the answer
// midway (between the item's loads and its stores, when nothing else of its memory traffic is waited for).
__device__ __forceinline__ uint32_t next_round_ask(const ItemCall& c) { return threadIdx.x == 0 ? atomicAdd(c.ticket, 1u) : 0u; }
__device__ __forceinline__ void next_round_note(const ItemCall& c, uint32_t next) { if (threadIdx.x == 0) g_round_slot[(c.round + 1u) & 1u] = next; }

__device__ __forceinline__ void item_rays(const ItemCall& c, const ChainScratch& S, bool in_order, uint32_t* r0, uint32_t* n_r) {
	if (in_order) {
		*r0 = SRF_UNIFORM_U32(S.item_first[c.item]);
		*n_r = SRF_UNIFORM_U32(S.item_first[c.item + 1]) - *r0;
	} else {
		*r0 = c.item * wv::GROUP;
		*n_r = c.n_active - *r0 < wv::GROUP ? c.n_active - *r0 : wv::GROUP;
	}
}

__device__ __forceinline__ void item_done(const ItemCall& c, uint32_t prefix, uint32_t total) {
	if (c.item == c.n_items - 1 && lane_id() == 0) *c.compacted_counter = prefix == CHAIN_FAILED ? CHAIN_FAILED : prefix + total;
}

// The common item: at most 64 rays, laid out in order, whose samples fit the window in one piece.  Returns false, with
// nothing done but the next round's number noted, for any other item.
template <bool HI, bool HO, bool PL>
__device__ __forceinline__ bool wave_item_fit(const ItemCall& c, const fused::Args& A, const ChainScratch& S) {
	const uint32_t lane = lane_id();
	const uint32_t next = next_round_ask(c);
	uint32_t r0, n_r;
	item_rays(c, S, true, &r0, &n_r);
	bool fits = n_r <= WAVE;
	WaveBatch B;
	if (fits) {
		B = wave_load_batch(lane, r0, n_r, A);
		fits = B.n_chunks <= 1;
	}
	if (!fits) { next_round_note(c, next); return false; }
	wv::Lds& w = g_window[c.wave];
	fused::SlotState<wv::G, HI> st;
	wv::RayState rs;
	uint32_t prefix = 0, item_total = 0;
	wave_forward<HI, PL, true>(lane, B, A, w, st, rs);
	next_round_note(c, next);
	wave_backward<HI, HO, PL, true>(lane, B, A, w, st, rs, [&](uint32_t t, auto&& meanwhile) -> uint32_t {
		item_total = t;
		prefix = item_offset(S, c.item, t, meanwhile);
		return prefix;
	});
	item_done(c, prefix, item_total);
	return true;
}

// Every other item: a batch in several chunks, more rays than lanes (every batch is counted first, then every batch runs
// again with its offset known), and, when the call's rays are not laid out in order, rays anywhere in the sample buffer
// (one lane per ray, straight from memory: ray_marcher.cu:57-201 as it stands).  draws: the workgroup's next round
// number is still to be drawn (it is not when wave_item_fit has turned the item down).  Out of line, with the call's
// arguments read from their copies in memory, so that the common path's registers are allocated without regard to this one.
template <bool HI, bool HO, bool PL>
__device__ __noinline__ void wave_item_general(ItemCall c, bool in_order, bool draws) {
	const fused::Args A0 = *(const fused::Args*)c.args_copy;
	const ChainScratch S = *(const ChainScratch*)c.scratch_copy;
	fused::Args A = A0;
	A.n_active = c.n_active; A.mean_density = c.mean_density;
	if (draws) next_round_note(c, next_round_ask(c));
	wv::Lds& w = g_window[c.wave];
	const uint32_t lane = lane_id();
	const uint32_t item = c.item;
	uint32_t r0, n_r;
	item_rays(c, S, in_order, &r0, &n_r);
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
	item_done(c, prefix, item_total);
}

// two workgroups per CU: eight wavefronts, two per SIMD, with up to 256 registers each
#define SRF_WAVES_OCCUPANCY __attribute__((amdgpu_waves_per_eu(2, 2)))
constexpr uint32_t WAVES_WORKGROUPS_PER_CU = 2;

template <bool HI, bool HO, bool PL>
__global__ void __launch_bounds__(WAVES_THREADS) SRF_WAVES_OCCUPANCY k_composite_waves(fused::Args A, const uint32_t* __restrict__ n_rays_counter, const float* __restrict__ mean_density_ptr,
                                                                                       ChainScratch S, uint32_t* __restrict__ compacted_counter) {
	const uint32_t tid = threadIdx.x;
	const uint32_t counter_now = *n_rays_counter;
	ItemCall c;
	c.mean_density = mean_density_ptr ? *mean_density_ptr : 0.f;
	c.n_active = counter_now < A.K.n_rays ? counter_now : A.K.n_rays;
	A.mean_density = c.mean_density; A.n_active = c.n_active;
	c.args_copy = S.args_copy; c.scratch_copy = S.scratch_copy; c.compacted_counter = compacted_counter; c.ticket = S.ticket;
	c.wave = tid / WAVE;
	const bool in_order = *S.disorder == 0u;
	c.n_items = in_order ? *S.n_items : div_up(c.n_active, wv::GROUP);
	const uint32_t n_rounds = div_up(c.n_items, wv::ITEMS_PER_TICKET);
	if (tid == 0) g_round_slot[0] = atomicAdd(S.ticket, 1u);
	for (c.round = 0;; ++c.round) {
		__syncthreads();
		const uint32_t t = SRF_UNIFORM_U32(g_round_slot[c.round & 1u]);
		if (t >= n_rounds) break;
		c.item = t * wv::ITEMS_PER_TICKET + c.wave;
		if (c.item >= c.n_items) { next_round_note(c, next_round_ask(c)); continue; }
		bool done = false;
		if (in_order) done = wave_item_fit<HI, HO, PL>(c, A, S);
		if (!done) wave_item_general<HI, HO, PL>(c, in_order, !in_order);
	}
	// the last workgroup to leave puts the words back that the next call expects to be zero
	if (tid == 0) {
		__threadfence();
		if (atomicInc(S.exits, gridDim.x - 1u) == gridDim.x - 1u) { *S.ticket = 0u; *S.disorder = 0u; }
	}
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
	return SRF_OK;
}

size_t waves_scratch_bytes(uint32_t n_rays) { return wave_layout(n_rays).bytes; }
uint32_t* waves_error_word(void* scratch) { return wave_scratch_at(scratch, 0, nullptr, 0).error; }

} // namespace srf
