// Host build of the kernels' per-item bodies (sphericalrf_amd/csrc/srf_bodies.h): every
// "thread" is run in a plain loop by a host compiler, with the prefix sums that the
// device computes between launches done serially.  Test infrastructure only: lets the
// CPU test-suite compare the kernel logic with the oracle bit for bit without a GPU.
#include <stdint.h>
static uint64_t g_probe_count = 0;
#define SRF_COUNT_PROBE() (++g_probe_count)
static uint64_t g_radius_hist[8][4] = {};   // [cascade][radius 0, 1-block, 2-3, more] of the empty probes
#define SRF_COUNT_RADIUS(n, level) (++g_radius_hist[(level) & 7][(n) == 0 ? 0 : ((n) >> (level)) <= 1 ? 1 : ((n) >> (level)) <= 3 ? 2 : 3])
#include <cstring>
#include <vector>
#include <array>
#include <cstdlib>
#include <algorithm>
#include "../../sphericalrf_amd/csrc/srf_bodies.h"
#include "../../sphericalrf_amd/csrc/srf_composite_fused.h"
#include "../../sphericalrf_amd/csrc/srf_composite_wave.h"
#include "../../oracle/srf_oracle.h"

using namespace srf;

static_assert(sizeof(srf_ray_payload) == 40, "payload layout");
static_assert(sizeof(orc_params) + sizeof(uint32_t) + 4 * sizeof(float) == sizeof(Params), "Params mirrors orc_params plus n_cells and the optional sphere");

// the optional sphere bound of the marches (the reference and the oracle have none): set by hs_set_sphere for the calls that follow
static float g_sphere[4] = {0.f, 0.f, 0.f, 0.f};

static Params to_params(const orc_params* p) {
	Params P;
	std::memcpy(&P, p, sizeof(orc_params));
	P.n_cells = p->grid_size[0] * p->grid_size[1] * p->grid_size[2];
	for (int k = 0; k < 4; ++k) P.sphere[k] = g_sphere[k];
	return P;
}

static LossConst make_loss_const(const orc_loss_args* a) {
	LossConst K;
	K.n_rays = a->n_rays; K.n_max_compacted = a->n_max_compacted_coords; K.out_width = (uint32_t)a->padded_output_width;
	K.rgb_act = a->rgb_activation; K.density_act = a->density_activation; K.loss_type = a->loss_type;
	K.loss_scale = a->loss_scale / (float)a->n_rays;
	K.min_optical_thickness = a->min_optical_thickness; K.use_grid = a->use_grid;
	for (int c = 0; c < 3; ++c) K.bg_in[c] = a->background_color[c];
	if (a->train_with_random_bg_color) {
		Pcg32 r; r.state = a->rng.state; r.inc = a->rng.inc;
		K.bg_in[0] = pcg_next_float(r); K.bg_in[1] = pcg_next_float(r); K.bg_in[2] = pcg_next_float(r);
	}
	loss_const_background(K);
	K.color_space = a->color_space; K.train_in_linear = a->train_in_linear_color; K.thr = a->transmittance_threshold; K.dt_stride = a->dt_stride;
	return K;
}


// The single-launch compositing, group by group and phase by phase, in the control flow of the device kernels: the
// groups the streaming kernel does not take (rays not laid out back to back, more samples than one window) get their
// forward pass first and leave their per-ray counts; the streaming loop then runs every group in order (count, chain
// with the count known, finish, ordered offsets, phase C), handing the listed groups only their offsets; the listed
// groups' second forward pass and their gradients come last.
// items a group may be cut into (what the device's scratch has room for), and the most that a group of the last call made
static uint32_t g_fused_max_parts = fused::MAX_PARTS, g_fused_most_parts = 0;

template <bool HI, bool HO>
static void run_fused(const orc_loss_args* a, const float* rays_rgba, uint32_t n_rays_counter, uint32_t* ray_coord_indices, const float* dt,
                      const float* coords, float* compacted_coords, uint32_t* n_compacted_counter, const void* net, void* dloss, float* loss_output,
                      float* rgb_ray_out, uint32_t* n_scattered_groups, uint32_t* n_multi_window_groups) {
	using namespace fused;
	using GS = StreamGeometry;   // the streaming kernel's sample threads and window
	using GW = WideGeometry;     // the kernel for the listed groups
	Args A;
	A.K = make_loss_const(a);
	A.n_active = n_rays_counter < a->n_rays ? n_rays_counter : a->n_rays;
	A.rays_rgba = rays_rgba; A.ray_coord_indices = ray_coord_indices; A.dt_arr = dt; A.coords = coords; A.compacted_coords = compacted_coords;
	A.net = net; A.dloss = dloss; A.loss_output = loss_output; A.rgb_ray_out = rgb_ray_out; A.mean_density = a->mean_density;
	const bool plain = A.K.rgb_act == SRF_ACT_NONE && A.K.density_act == SRF_ACT_NONE;
	const uint32_t n_groups = (A.n_active + RAYS - 1) / RAYS;
	std::vector<SlotState<GS, HI>> st_s(GS::THREADS);
	std::vector<SlotState<GW, HI>> st_w(GW::THREADS);
	std::vector<RayCarry> c(RAYS);
	std::vector<uint32_t> side((size_t)n_groups * RAYS, 0);
	std::vector<uint32_t> slow;
	Window<GS>* ws = new Window<GS>[2];
	Window<GW>* ww = new Window<GW>();
	RayLds* rlp = new RayLds();
	RayLds& rl = *rlp;
	Plan plans[NPLAN];
	auto make_plan = [&](uint32_t g, Plan& pl, std::vector<Float4>* tgt) {
		const uint32_t ray0 = g * RAYS;
		pl.misc[M_SUM] = 0; pl.misc[M_CONTIG] = 1;
		Float4 dummy;
		for (uint32_t t = 0; t < RAYS; ++t) load_ray(t, ray0, A, pl, tgt ? &(*tgt)[t] : &dummy);
		for (uint32_t t = 0; t < RAYS; ++t) plan_lane(t, ray0, A, pl);
		for (uint32_t t = 0; t < RAYS; ++t) plan_finish_lane(t, ray0, A, pl);
	};
	// k_chain_prepare and k_chain_items: the items in ray order, and which of them belong to listed groups
	std::vector<U2> items;
	for (uint32_t g = 0; g < n_groups; ++g) {
		make_plan(g, plans[0], nullptr);
		const uint64_t cuts = plan_cuts<GS>(plans[0], g_fused_max_parts);
		const uint32_t word = group_items_word(cuts);
		U2 it[MAX_PARTS];
		const uint32_t n = items_of_group(g, word, cuts, it);
		g_fused_most_parts = n > g_fused_most_parts ? n : g_fused_most_parts;
		if (item_listed(it[0])) {
			slow.push_back(g);
			if (plans[0].misc[M_CONTIG] == 0) ++*n_scattered_groups; else ++*n_multi_window_groups;
		}
		for (uint32_t k = 0; k < n; ++k) items.push_back(it[k]);
	}
	// k_slow_groups, forward and backward
	auto slow_groups = [&](bool backward) {
		Args B = A;
		if (!backward) B.rgb_ray_out = nullptr;
		Plan& pl = plans[0];
		for (uint32_t g : slow) {
			const uint32_t ray0 = g * RAYS;
			std::vector<Float4> tgt(RAYS);
			make_plan(g, pl, &tgt);
			if (pl.misc[M_CONTIG] != 0) {
				// part by part (the device deals a group's parts to several workgroups)
				Plan group = pl;
				uint64_t cuts = plan_cuts_any_length<GW>(group);
				while (cuts) {
					const uint32_t lo = (uint32_t)__builtin_ctzll(cuts);
					cuts &= cuts - 1ull;
					const uint32_t hi = cuts ? (uint32_t)__builtin_ctzll(cuts) : RAYS;
					for (uint32_t t = 0; t < RAYS; ++t) plan_part_lane(t, group, lo, hi, g, pl);
					const uint32_t n_win = (pl.misc[M_TOTAL] + GW::WIN - 1) / GW::WIN;
					auto live = [&](uint32_t t) { return ray0 + t < B.n_active && t >= lo && t < hi; };
					for (uint32_t t = 0; t < RAYS; ++t) reset_carry(t, pl, c[t]);
					for (uint32_t win = 0; win < n_win; ++win) {
						for (uint32_t t = 0; t < GW::THREADS; ++t) phase_a<GW, HI>(t, win, B, *ww, pl, st_w[t]);
						for (uint32_t t = 0; t < RAYS; ++t) chain<GW>(t, win, B, *ww, rl, pl, c[t]);
					}
					for (uint32_t t = 0; t < RAYS; ++t) finish_ray(t, ray0, B, rl, c[t], tgt[t], lo, hi);
					if (!backward) {
						for (uint32_t t = 0; t < RAYS; ++t) if (live(t)) side[ray0 + t] = rl.rnf[t];
					} else {
						for (uint32_t t = 0; t < RAYS; ++t) commit_ray(t, ray0, live(t) ? side[ray0 + t] : 0u, B, rl, pl, lo, hi);
						for (uint32_t t = 0; t < RAYS; ++t) reset_carry(t, pl, c[t]);
						for (uint32_t win = 0; win < n_win; ++win) {
							for (uint32_t t = 0; t < GW::THREADS; ++t) phase_a<GW, HI>(t, win, B, *ww, pl, st_w[t]);
							for (uint32_t t = 0; t < RAYS; ++t) chain<GW>(t, win, B, *ww, rl, pl, c[t]);
							for (uint32_t t = 0; t < GW::THREADS; ++t) phase_c<GW, HI, HO>(t, win, B, *ww, rl, pl, st_w[t]);
						}
					}
				}
			} else {
				for (uint32_t t = 0; t < RAYS; ++t) {
					uint32_t n = 0;
					FwdRay fw;
					loss_forward_body<HI>(ray0 + t, B.K, B.rays_rgba, B.n_active, B.ray_coord_indices, B.dt_arr, B.net, &fw, &n, B.rgb_ray_out);
					if (ray0 + t >= B.n_active) continue;
					if (!backward) side[ray0 + t] = n;
					else loss_backward_body<HI, HO>(ray0 + t, B.K, B.n_active, B.ray_coord_indices, B.dt_arr, B.coords, B.compacted_coords, B.net, B.dloss, B.loss_output,
					                                B.mean_density, fw, n, side[ray0 + t], nullptr);
				}
			}
		}
	};
	slow_groups(false);
	// k_composite_stream (items in order and one at a time; the device spreads them over persistent workgroups and
	// keeps three of a workgroup's items under way in two windows)
	uint32_t prefix = *n_compacted_counter;
	Plan group_plan;
	for (size_t i = 0; i < items.size(); ++i) {
		const U2 item = items[i];
		const uint32_t g = item.x, ray0 = g * RAYS, lo = item_lo(item), hi = item_hi(item);
		std::vector<Float4> tgt(RAYS);
		make_plan(g, group_plan, &tgt);
		Plan& pl = plans[i % NPLAN];
		Window<GS>& w = ws[i % 2];
		for (uint32_t t = 0; t < RAYS; ++t) plan_part_lane(t, group_plan, lo, hi, g, pl);
		const bool fast = !item_listed(item);
		std::vector<uint32_t> n(RAYS, 0);
		if (fast) {
			for (uint32_t t = 0; t < GS::THREADS; ++t) phase_a_load_single<GS, HI>(t, A, pl, st_s[t]);
			for (uint32_t t = 0; t < GS::THREADS; ++t) { if (plain) phase_a_compute<GS, HI, true>(t, 0, A, w, pl, st_s[t]); else phase_a_compute<GS, HI, false>(t, 0, A, w, pl, st_s[t]); }
			uint32_t rn_max = 0, n_max = 0;
			for (uint32_t t = 0; t < RAYS; ++t) rn_max = pl.rn[t] > rn_max ? pl.rn[t] : rn_max;
			for (uint32_t t = 0; t < RAYS; ++t) n[t] = count_lane<GS>(t, rn_max, A, w, pl);
			for (uint32_t t = 0; t < RAYS; ++t) n_max = n[t] > n_max ? n[t] : n_max;
			for (uint32_t t = 0; t < RAYS; ++t) chain_counted<GS, false>(t, n[t], n_max, w, rl, pl, c[t]);
			for (uint32_t t = 0; t < RAYS; ++t) mark_owners<GS>(t, rn_max, w, pl);
			for (uint32_t t = 0; t < RAYS; ++t) finish_ray(t, ray0, A, rl, c[t], tgt[t], lo, hi);
		} else {
			for (uint32_t t = 0; t < RAYS; ++t) n[t] = ray0 + t < A.n_active ? side[ray0 + t] : 0u;
		}
		uint32_t run = prefix;
		for (uint32_t t = 0; t < RAYS; ++t) {
			if (fast) commit_ray(t, ray0, run, A, rl, pl, lo, hi);
			else if (ray0 + t < A.n_active) side[ray0 + t] = run;
			run += n[t];
		}
		prefix = run;
		if (fast) {
			for (uint32_t t = 0; t < GS::THREADS; ++t) { if (plain) phase_c<GS, HI, HO, true, false>(t, 0, A, w, rl, pl, st_s[t]); else phase_c<GS, HI, HO, false, false>(t, 0, A, w, rl, pl, st_s[t]); }
			if (A.compacted_coords) for (uint32_t q0 = 0; q0 < pl.misc[M_TOTAL]; q0 += COORDS_DEPTH * RAYS) for (uint32_t t = 0; t < RAYS; ++t) coords_copy_rows<GS>(t, q0, A, w, rl, pl);
		}
	}
	*n_compacted_counter = prefix;
	slow_groups(true);
	delete[] ws; delete ww; delete rlp;
}

// The wave-per-item compositing, item by item and phase by phase, in the control flow of the device kernel: the
// preparing pass (stride of the sample windows, first ray of every item, whether the rays are laid out in order),
// then every item in order.  An item's rays go through the LDS window 64 at a time (a batch): a batch whose samples
// fit the window in one piece, or chunk by chunk with a second sweep for the gradients; an item of several batches
// counts all of them first.  Every item of a call whose rays are not in order is composited one lane per ray from memory.
// counts: batches that fit the window / chunked batches / per-ray items / items of several batches.
template <bool HI, bool HO>
static void run_wave(const orc_loss_args* a, const float* rays_rgba, uint32_t n_rays_counter, uint32_t* ray_coord_indices, const float* dt,
                     const float* coords, float* compacted_coords, uint32_t* n_compacted_counter, const void* net, void* dloss, float* loss_output,
                     float* rgb_ray_out, uint32_t counts[4], uint32_t force_stride) {
	using namespace wv;
	Args A;
	A.K = make_loss_const(a);
	A.n_active = n_rays_counter < a->n_rays ? n_rays_counter : a->n_rays;
	A.rays_rgba = rays_rgba; A.ray_coord_indices = ray_coord_indices; A.dt_arr = dt; A.coords = coords; A.compacted_coords = compacted_coords;
	A.net = net; A.dloss = dloss; A.loss_output = loss_output; A.rgb_ray_out = rgb_ray_out; A.mean_density = a->mean_density;
	const bool plain = A.K.rgb_act == SRF_ACT_NONE && A.K.density_act == SRF_ACT_NONE;
	const uint32_t cap = max_items(a->n_rays);
	// preparing pass
	Windows W = windows_of(A.n_active, ray_coord_indices, cap);
	if (force_stride) { W.stride = force_stride; W.n_items = A.n_active ? (uint32_t)((ray_coord_indices[2 * (size_t)(A.n_active - 1) + 1] - W.base0) / W.stride) + 1 : 0; }
	std::vector<ItemDesc> desc((size_t)cap);
	std::memset(desc.data(), 0xdb, desc.size() * sizeof(ItemDesc));
	bool irregular = false;
	for (uint32_t i = 0; i < A.n_active; ++i) if (!prepare_ray(i, A.n_active, ray_coord_indices, W, cap, desc.data())) irregular = true;
	if (!irregular && W.n_items > cap) irregular = true;      // (a forced stride may ask for more items than the table holds)
	const uint32_t n_items = irregular ? (A.n_active + GROUP - 1) / GROUP : W.n_items;
	Lds* wp = new Lds();
	Lds& w = *wp;
	std::vector<SlotState<G, HI>> st(LANES);
	uint32_t prefix = *n_compacted_counter;

	// one batch: rays [rb, rb + nb) of the call, nb <= 64
	struct Batch { uint32_t rb, nb; uint64_t s0; uint32_t range, n_chunks; uint32_t n[LANES], rbase[LANES]; Float4 tgt[LANES]; RayState rs[LANES]; };
	Batch B;
	auto load_batch = [&](uint32_t rb, uint32_t nb) {
		B.rb = rb; B.nb = nb;
		uint64_t base[LANES];
		for (uint32_t l = 0; l < LANES; ++l) {
			B.n[l] = 0; base[l] = 0; B.tgt[l] = mk4(0.f, 0.f, 0.f, 0.f);
			if (l < nb) { B.n[l] = ray_coord_indices[2 * (size_t)(rb + l)]; base[l] = ray_coord_indices[2 * (size_t)(rb + l) + 1]; B.tgt[l] = *(const Float4*)(rays_rgba + 4 * (size_t)(rb + l)); }
		}
		B.s0 = nb ? base[0] : 0;
		B.range = nb ? (uint32_t)(base[nb - 1] + B.n[nb - 1] - B.s0) : 0;
		for (uint32_t l = 0; l < LANES; ++l) B.rbase[l] = l < nb ? (uint32_t)(base[l] - B.s0) : B.range;
		B.n_chunks = (B.range + WIN - 1) / WIN;
	};
	auto rows = [&](uint32_t chunk_lo) {
		for (uint32_t l = 0; l < LANES; ++l) rows_load<HI>(l, A, B.s0, B.range, chunk_lo, st[l]);
		for (uint32_t l = 0; l < LANES; ++l) { if (plain) rows_alpha<HI, true>(l, A, w, B.range, chunk_lo, st[l]); else rows_alpha<HI, false>(l, A, w, B.range, chunk_lo, st[l]); }
	};
	auto chain_all = [&](uint32_t chunk_lo) {
		uint32_t steps = 0;
		for (uint32_t l = 0; l < LANES; ++l) { uint32_t k0, k1; chain_span(B.n[l], B.rbase[l], chunk_lo, &k0, &k1); steps = k1 - k0 > steps ? k1 - k0 : steps; }
		// stretch by stretch across the lanes, as the wavefront runs it (with its early exit)
		for (uint32_t j = 0; j < steps; j += CHAIN_UNROLL) {
			bool any_live = false;
			for (uint32_t l = 0; l < LANES; ++l) { uint32_t k0, k1; chain_span(B.n[l], B.rbase[l], chunk_lo, &k0, &k1); if (k0 + j < k1 && B.rs[l].dead == 0) any_live = true; }
			if (!any_live) break;
			for (uint32_t l = 0; l < LANES; ++l) { uint32_t k0, k1; chain_span(B.n[l], B.rbase[l], chunk_lo, &k0, &k1); chain_stretch(l, j, k0, k1, B.rbase[l], chunk_lo, A.K.thr, w, B.rs[l]); }
		}
	};
	auto grads = [&](uint32_t chunk_lo) {
		for (uint32_t l = 0; l < LANES; ++l) {
			if (plain) rows_grads<HI, HO, true>(l, A, w, B.s0, B.range, chunk_lo, st[l]); else rows_grads<HI, HO, false>(l, A, w, B.s0, B.range, chunk_lo, st[l]);
		}
	};
	auto forward = [&]() {       // every chunk's rows and chain; the last chunk's records stay in the window
		for (uint32_t l = 0; l < LANES; ++l) ray_reset(B.rs[l]);
		for (uint32_t c = 0; c < (B.n_chunks ? B.n_chunks : 1u); ++c) { rows(c * WIN); chain_all(c * WIN); }
	};
	auto batch_total = [&]() { uint32_t t = 0; for (uint32_t l = 0; l < B.nb; ++l) t += B.rs[l].cnt; return t; };
	auto finish_commit_grads = [&](uint32_t cbase0) {     // after forward(), with the batch's first compacted offset known
		float loss[LANES];
		for (uint32_t l = 0; l < B.nb; ++l) loss[l] = finish_lane(l, B.rb + l, B.n[l], A, w, B.rs[l], B.tgt[l]);
		uint32_t run = cbase0;
		for (uint32_t l = 0; l < LANES; ++l) {
			if (l < B.nb) { commit_lane(l, B.rb + l, B.rs[l].cnt, B.rbase[l], run, loss[l], A, w); run += B.rs[l].cnt; } else commit_none(l, w);
		}
		if (B.n_chunks <= 1) { ++counts[0]; grads(0); }
		else {
			++counts[1];
			for (uint32_t l = 0; l < LANES; ++l) ray_reset(B.rs[l]);
			for (uint32_t c = 0; c < B.n_chunks; ++c) { rows(c * WIN); chain_all(c * WIN); grads(c * WIN); }
		}
	};

	for (uint32_t item = 0; item < n_items; ++item) {
		uint32_t r0, n_r;
		if (irregular) { r0 = item * GROUP; n_r = A.n_active - r0 < GROUP ? A.n_active - r0 : GROUP; }
		else { r0 = desc[item].r0; n_r = desc[item].r_end - r0; }
		if (!irregular) {
			const uint32_t n_batches = (n_r + LANES - 1) / LANES;
			if (n_batches <= 1 && desc[item].s_end - desc[item].s0 <= WIN) {
				// the common item: in one piece, with the gradients staged in the window before the item's offset is looked at
				++counts[0];
				load_batch(r0, n_r);
				if (B.s0 != desc[item].s0 && n_r) std::abort();
				if (B.range != desc[item].s_end - desc[item].s0) std::abort();
				std::vector<RowData<HI>> in(LANES);
				std::vector<std::array<float, ROWS>> alpha(LANES);
				RayLds2& rl = w.staged();
				if (B.range) for (uint32_t l = 0; l < LANES; ++l) fit_rows_load<HI>(l, A, B.s0, B.range, in[l]);
				for (uint32_t l = 0; l < LANES; ++l) { if (plain) fit_rows_alpha<HI, true>(l, A, w.S, w.owner, B.range, in[l], alpha[l].data()); else fit_rows_alpha<HI, false>(l, A, w.S, w.owner, B.range, in[l], alpha[l].data()); }
				for (uint32_t l = 0; l < LANES; ++l) ray_reset(B.rs[l]);
				chain_all(0);
				float loss[LANES];
				for (uint32_t l = 0; l < B.nb; ++l) loss[l] = fit_finish_lane(l, B.rb + l, B.n[l], A, rl, B.rs[l], B.tgt[l]);
				for (uint32_t l = 0; l < LANES; ++l) { if (plain) fit_rows_grads<HI, true>(l, A, w.S, w.owner, rl, B.range, in[l], alpha[l].data()); else fit_rows_grads<HI, false>(l, A, w.S, w.owner, rl, B.range, in[l], alpha[l].data()); }
				uint32_t run = prefix;        // (the device publishes the total before the gradients and chains it to the earlier items' after them)
				for (uint32_t l = 0; l < LANES; ++l) {
					if (l < B.nb) { fit_commit_lane(l, B.rb + l, B.rs[l].cnt, B.rbase[l], run, prefix, loss[l], A, rl); run += B.rs[l].cnt; } else fit_commit_none(l, rl);
				}
				for (uint32_t l = 0; l < LANES; ++l) fit_rows_store<HO>(l, A, w.S, w.owner, rl, B.s0, B.range, prefix);
				prefix = run;
			} else if (n_batches <= 1) {
				load_batch(r0, n_r);
				forward();
				const uint32_t total = batch_total();
				finish_commit_grads(prefix);        // (the device publishes the total and chains it to the earlier items' here)
				prefix += total;
			} else {
				++counts[3];
				uint32_t total = 0;
				for (uint32_t b = 0; b < n_batches; ++b) { load_batch(r0 + b * LANES, n_r - b * LANES < LANES ? n_r - b * LANES : LANES); forward(); total += batch_total(); }
				uint32_t run = prefix;
				for (uint32_t b = 0; b < n_batches; ++b) {
					load_batch(r0 + b * LANES, n_r - b * LANES < LANES ? n_r - b * LANES : LANES);
					forward();
					const uint32_t t = batch_total();
					finish_commit_grads(run);
					run += t;
				}
				prefix += total;
			}
		} else {
			++counts[2];
			std::vector<FwdRay> fw(n_r);
			std::vector<uint32_t> nf(n_r, 0);
			for (uint32_t k = 0; k < n_r; ++k) loss_forward_body<HI>(r0 + k, A.K, A.rays_rgba, A.n_active, A.ray_coord_indices, A.dt_arr, A.net, &fw[k], &nf[k], A.rgb_ray_out);
			uint32_t run = prefix;
			for (uint32_t k = 0; k < n_r; ++k) {
				loss_backward_body<HI, HO>(r0 + k, A.K, A.n_active, A.ray_coord_indices, A.dt_arr, A.coords, A.compacted_coords, A.net, A.dloss, A.loss_output,
				                           A.mean_density, fw[k], nf[k], run, nullptr);
				run += nf[k];
			}
			prefix = run;
		}
	}
	*n_compacted_counter = prefix;
	delete wp;
}

extern "C" {

float hs_elem(int which, float a, float b) {
	switch (which) {
	case 0: return srf_expf(a); case 1: return srf_logf(a); case 2: return srf_sinf(a); case 3: return srf_cosf(a);
	case 4: return srf_asinf(a); case 5: return srf_atan2f(a, b); case 6: return srf_powf(a, b); case 7: return srf_sqrt(a); case 8: return a / b;
	case 9: return half_bits_to_float(float_to_half_bits(a));
	case 10: return srf_rcp(a);
	}
	return 0.f;
}
uint16_t hs_float_to_half(float f) { return float_to_half_bits(f); }
float hs_half_to_float(uint16_t h) { return half_bits_to_float(h); }
uint32_t hs_morton3d(uint32_t x, uint32_t y, uint32_t z) { return morton3d(x, y, z); }
uint32_t hs_morton3d_invert(uint32_t x) { return morton3d_invert(x); }
float hs_ld_random_val(uint32_t index, uint32_t seed, uint32_t dim) { return ld_random_val01(index, seed, dim); }
void hs_ld_random_pixel_offset(uint32_t spp, float out[2]) { ld_random_pixel_offset(spp, out); }
uint32_t hs_pcg_sequence(uint64_t state, uint64_t inc, uint64_t advance, uint32_t n, uint32_t* out_u, float* out_f) {
	Pcg32 r; r.state = state; r.inc = inc;
	pcg_advance(r, advance);
	for (uint32_t k = 0; k < n; ++k) { Pcg32 c = r; out_u[k] = pcg_next_uint(r); out_f[k] = pcg_next_float(c); }
	return 0;
}

void hs_point(const orc_params* p, const float pos[3], float t, float warped[3], float* dt, uint32_t* level, uint32_t* idx, float unwarped[3]) {
	const Params P = to_params(p);
	const Vec3 x = ld3(pos);
	const Vec3 w = warp_position(P, x);
	st3(warped, w);
	const Probe pr = probe_at(P, nullptr, x, t, P.cone_angle_constant);
	*dt = pr.dt;
	*level = pr.level;
	*idx = pr.idx;
	st3(unwarped, unwarp_position(P, w));
}

// cascade and cell of a warped position: the generic functions and the shortcut used for the WarpedSpace_Exp grid
void hs_cell_both(const Params* Pp, const float* w, uint32_t* generic, uint32_t* fast) {
	const Params& P = *Pp;
	const Vec3 x = mk3(w[0], w[1], w[2]);
	generic[0] = level_from_pos(P, x, x);
	generic[1] = cascaded_grid_idx_at(P, x, x, generic[0]);
	fast[0] = level_warped_exp(P, x);
	fast[1] = grid_idx_warped_exp(P, x, fast[0]);
}

void hs_ray_intersect(const orc_params* p, const float o[3], const float d[3], float out[2]) {
	const Params P = to_params(p);
	aabb_ray_intersect(P, ld3(o), ld3(d), &out[0], &out[1]);
}

void hs_generate_grid_samples(const orc_params* p, uint32_t n, orc_pcg32 rng, uint32_t step, const float* grid, float thresh, float* pos, uint32_t* idx) {
	const Params P = to_params(p);
	Pcg32 r; r.state = rng.state; r.inc = rng.inc;
	for (uint32_t i = 0; i < n; ++i) grid_sample_body(i, P, n, r, step, grid, thresh, pos, idx, nullptr, nullptr, 1u + i % 4u);   // every batch size of the lookups
}

// radii read by empty probes since the last reset: out[cascade * 4 + class]
void hs_radius_hist(uint64_t* out, int reset) { for (int l = 0; l < 8; ++l) for (int k = 0; k < 4; ++k) { out[l * 4 + k] = g_radius_hist[l][k]; if (reset) g_radius_hist[l][k] = 0; } }

// probes of the grid made by the counting march since the last reset
uint64_t hs_probe_count(int reset) { const uint64_t v = g_probe_count; if (reset) g_probe_count = 0; return v; }

// the empty-space table as the library builds it, one body call per item; returns blocks per axis (0: no table for this grid).
// dist must hold nb^3 * n_cascades entries (at most 64^3 * n_cascades).
uint32_t hs_build_skip_table(const orc_params* p, const uint8_t* bitfield, uint16_t* dist) {
	const Params P = to_params(p);
	const SkipTable T = skip_table_for(P, dist);
	if (!T.nb) return 0;
	const uint32_t nb = T.nb, n = nb * nb * nb * P.n_cascades, h3 = (nb / 2) * (nb / 2) * (nb / 2);
	std::vector<uint8_t> a(n), b(n);
	for (uint32_t i = 0; i < n; ++i) skip_block_occupancy_body(i, P, T, bitfield, a.data());
	for (uint32_t level = 1; level < P.n_cascades; ++level)
		for (uint32_t i = 0; i < h3; ++i) skip_pool_body(i, T, level, a.data());
	for (uint32_t i = 0; i < n; ++i) skip_distance_axis_body(i, T, 0, a.data(), b.data());
	for (uint32_t i = 0; i < n; ++i) skip_distance_axis_body(i, T, 1, b.data(), a.data());
	for (uint32_t i = 0; i < n; ++i) skip_distance_axis_body(i, T, 2, a.data(), b.data());
	for (uint32_t i = 0; i < n; ++i) skip_combine_body(i, P, T, b.data(), dist);
	return nb;
}

// block radius (in warped units) that the table gives for a warped position, with the cascade and block it was read from
float hs_skip_radius_at(const orc_params* p, const uint16_t* dist, const float* w, uint32_t* level_out) {
	const Params P = to_params(p);
	const SkipTable T = skip_table_for(P, dist);
	const Vec3 x = mk3(w[0], w[1], w[2]);
	const uint32_t level = level_warped_exp(P, x);
	uint32_t cx, cy, cz;
	cell_warped_exp(P, x, level, &cx, &cy, &cz);
	*level_out = level;
	return (float)T.dist[skip_index(T.nb, level, cx >> T.sx, cy >> T.sy, cz >> T.sz)] * T.side0;
}

// one wavefront of the counting kernel, lanes run one after the other: the same phase choice per round as the device kernel
static void count_wave_sim(const Params& P, const CountArgs& A, uint32_t first, uint32_t end, const uint32_t* order) {
	CountLane L[64];
	for (auto& l : L) l.phase = LANE_IDLE;
	uint32_t next = first;
	for (;;) {
		uint32_t n_idle = 0, n_probe = 0, n_step = 0;
		for (auto& l : L) { n_idle += l.phase == LANE_IDLE; n_probe += l.phase == LANE_PROBE; n_step += l.phase == LANE_STEP; }
		const uint32_t left = end - next;
		n_idle = n_idle < left ? n_idle : left;
		if (!(n_idle | n_probe | n_step)) break;
		const bool begin = n_idle >= 32 || (n_idle && !n_probe && !n_step);
		const bool step = !begin && n_step && n_probe < 64 && n_probe < 8 * n_step;
		if (step) {
			for (auto& l : L) if (l.phase == LANE_STEP) count_steps<24>(l, P, A);
		} else if (!begin) {
			for (auto& l : L) if (l.phase == LANE_PROBE) count_probe(l, P, A);
		} else {
			uint32_t rank = 0;
			for (auto& l : L) if (l.phase == LANE_IDLE) { if (rank < n_idle) count_begin(l, order[next + rank], P, A); ++rank; }
			next += n_idle;
		}
	}
}

void hs_generate_training_samples(const orc_params* p, uint32_t n_rays, uint32_t n_rays_shift, uint32_t n_coords, const orc_dataset* d,
                                  const uint8_t* bitfield, orc_pcg32 rng, uint32_t* ray_counter, uint32_t* numsteps_counter,
                                  float* rays_out, float* rays_rgba, uint32_t* numsteps_out, float* coords_out, float* t_out, float* dt_out, uint32_t* cell,
                                  uint32_t log_words_override, const uint16_t* skip_dist, uint32_t rays_per_wave, uint32_t probe_budget) {
	const Params P = to_params(p);
	DatasetArgs ds;
	ds.n_images = d->n_images;
	for (int a = 0; a < 2; ++a) { ds.res[a] = d->resolution[a]; ds.focal[a] = d->focal_length[a]; ds.pp[a] = d->principal_point[a]; }
	ds.xforms = d->xforms; ds.images = d->images; ds.prob = d->sampling_probability;
	Pcg32 r; r.state = rng.state; r.inc = rng.inc;
	std::vector<TrainRay> state(n_rays);
	std::vector<uint32_t> counts(n_rays), base(n_rays), keep(n_rays), ridx(n_rays);
	// step log sized as the library sizes it; log_words_override (when not 0xffffffff) forces a smaller log to exercise the fallback
	uint32_t log_words = P.use_grid ? (P.n_max_steps + 64 + 31) / 32 : 0;
	if (log_words_override != 0xffffffffu) log_words = log_words_override;
	if (log_words > LOG_MAX_WORDS) log_words = LOG_MAX_WORDS;
	std::vector<uint32_t> logbits((size_t)log_words * n_rays + 1);
	std::vector<float> logt((size_t)log_words * n_rays + 1);
	StepLog log; log.bits = log_words ? logbits.data() : nullptr; log.t0 = logt.data(); log.stride = n_rays; log.words = log_words;
	CountArgs ca;
	ca.n_rays = n_rays; ca.n_rays_shift = n_rays_shift; ca.ds = ds; ca.bitfield = bitfield; ca.rng = r;
	ca.state = state.data(); ca.counts = counts.data(); ca.log = log; ca.skip = skip_table_for(P, skip_dist);
	// rays that use up probe_budget lookups are parked and finished by the wide march, as in the library (0: never);
	// a queue smaller than the number of rays exercises the refusal as well
	std::vector<ParkedRay> parked(probe_budget ? n_rays / 2 + 1 : 0);
	uint32_t parked_count = 0;
	ca.probe_budget = probe_budget; ca.park_lanes = 64; ca.parked = parked.data(); ca.parked_capacity = (uint32_t)parked.size(); ca.parked_count = &parked_count;
	// rays_per_wave 0: every ray start to end on its own; otherwise wavefronts of 64 lanes sharing rays_per_wave rays as on the device
	if (rays_per_wave == 0) for (uint32_t i = 0; i < n_rays; ++i) train_count_body(i, P, ca);
	else {
		// marching order of the library: each chunk of ray indices sorted by image and pixel tile
		std::vector<uint32_t> order(n_rays), key(n_rays);
		for (uint32_t first = 0; first < n_rays; first += RAY_CHUNK) {
			const uint32_t last = std::min(first + RAY_CHUNK, n_rays), chunk_image = train_ray_image(first, ca);
			for (uint32_t i = first; i < last; ++i) { order[i] = i; key[i] = ray_chunk_key_body(i, chunk_image, P, ca); }
			std::stable_sort(order.begin() + first, order.begin() + last, [&](uint32_t a, uint32_t b) { return key[a] < key[b]; });
		}
		for (uint32_t f = 0; f < n_rays; f += rays_per_wave) count_wave_sim(P, ca, f, std::min(f + rays_per_wave, n_rays), order.data());
	}
	for (uint32_t q = 0; q < std::min(parked_count, ca.parked_capacity); ++q) wide_march_serial(parked[q], P, ca);
	uint32_t run = *numsteps_counter;
	for (uint32_t i = 0; i < n_rays; ++i) { base[i] = run; run += counts[i]; }
	*numsteps_counter = run;
	run = *ray_counter;
	for (uint32_t i = 0; i < n_rays; ++i) { keep[i] = train_keep_flag(counts[i], base[i], n_coords); ridx[i] = run; run += keep[i]; }
	*ray_counter = run;
	for (uint32_t i = 0; i < n_rays; ++i)
		train_write_body(i, P, ds, bitfield, state.data(), counts.data(), base.data(), keep.data(), ridx.data(), rays_out, rays_rgba, numsteps_out, coords_out, DirectSink{t_out, dt_out, cell}, log);
}

static PixelArgs pixel_args(const Params& P, const int32_t res[2], const float focal[2], const float pp[2], const float cam[12], uint32_t spp) {
	PixelArgs A;
	for (int a = 0; a < 2; ++a) { A.res[a] = res[a]; A.focal[a] = focal[a]; A.pp[a] = pp[a]; }
	std::memcpy(A.cam.m, cam, sizeof(A.cam.m));
	ld_random_pixel_offset(P.snap_render ? 0u : spp, A.offset);
	return A;
}

// wide_apply against the loop it stands for: random batches of 64 steps (inside / occupied / zero-step masks, ray state
// near the sample cap, short logs) go through wide_apply and through one count_probe-like step at a time; returns the
// number of cases in which any field of the ray, the log or the finished ray's record differs
uint32_t hs_wide_apply_mismatches(uint32_t seed, uint32_t n_cases) {
	Pcg32 rng; pcg_seed(rng, seed, 7);
	auto rnd = [&](uint32_t n) { return pcg_next_uint(rng) % n; };
	uint32_t bad = 0;
	for (uint32_t c = 0; c < n_cases; ++c) {
		Params P{};
		P.n_max_steps = 8 + rnd(120);
		const uint32_t log_words = rnd(4) == 0 ? 2 : 8;
		std::vector<uint32_t> bits_a(log_words, 0xdeadbeefu), bits_b(log_words, 0xdeadbeefu);
		std::vector<float> t0_a(log_words, -1.f), t0_b(log_words, -1.f);
		TrainRay st_a{}, st_b{};
		uint32_t cnt_a = 0xffffffffu, cnt_b = 0xffffffffu;
		CountArgs A{}, B{};
		A.state = &st_a; A.counts = &cnt_a; A.log = StepLog{bits_a.data(), t0_a.data(), 1u, log_words};
		B.state = &st_b; B.counts = &cnt_b; B.log = StepLog{bits_b.data(), t0_b.data(), 1u, log_words};
		CountLane L{};
		L.phase = LANE_PROBE; L.i = 0; L.img = rnd(9);
		L.o = mk3(0.1f, 0.2f, 0.3f); L.d = mk3(0.f, 0.6f, 0.8f);
		L.step = rnd(150); L.cur_w = L.step >> 5;
		if (rnd(2)) L.cur_w = L.cur_w ? L.cur_w - 1 : 0;       // the word being filled may be an earlier one
		L.word = L.cur_w == (L.step >> 5) ? (rnd(2) ? (pcg_next_uint(rng) & ((1u << (L.step & 31u)) - 1u)) : 0u) : (pcg_next_uint(rng) | 1u);
		L.j = rnd(3) ? rnd(P.n_max_steps + 1) : (uint32_t)__builtin_popcount(L.word);
		L.t_word = 0.25f; L.startt = 0.125f; L.logged = rnd(8) != 0; L.mask[0] = rnd(2) ? 1u << (L.cur_w ? L.cur_w - 1 : 0) : 0u;
		float t[WIDE_STEPS + 1];
		uint64_t m_zero = 0;
		t[0] = 1.f + (float)rnd(100);
		const uint32_t zero_at = rnd(4) == 0 ? rnd(64) : 64;
		for (uint32_t k = 0; k < WIDE_STEPS; ++k) { const bool z = k == zero_at; m_zero |= (uint64_t)z << k; t[k + 1] = z ? t[k] : t[k] + 0.5f; }
		L.t = L.t_limit = t[0];
		const uint32_t out_at = rnd(3) == 0 ? rnd(65) : 64;
		uint64_t m_inside = out_at >= 64 ? ~0ull : ((1ull << out_at) - 1ull);
		if (out_at < 63 && rnd(2)) m_inside |= ~0ull << (out_at + 1);          // positions past the exit may read as inside again
		const uint32_t dens = rnd(4);
		uint64_t m_occ = 0;
		for (uint32_t k = 0; k < 64; ++k) m_occ |= (uint64_t)(dens == 0 ? 0u : dens == 3 ? 1u : rnd(dens + 1) != 0) << k;
		m_occ &= m_inside;      // a position outside the box is never looked up
		CountLane La = L, Lb = L;
		wide_apply(La, P, A, t, m_inside, m_occ, m_zero);
		for (uint32_t k = 0; k < WIDE_STEPS && Lb.phase != LANE_IDLE; ++k) {
			if (!(((m_inside >> k) & 1ull) && Lb.j < P.n_max_steps)) { count_finish(Lb, B); break; }
			if ((m_occ >> k) & 1ull) {
				++Lb.j;
				const uint32_t w = Lb.step >> 5;
				if (w != Lb.cur_w) { step_log_flush(B.log, Lb.i, Lb.cur_w, Lb.word, Lb.t_word, Lb.logged, Lb.mask); Lb.word = 0; Lb.cur_w = w; }
				if (!Lb.word) Lb.t_word = t[k];
				Lb.word |= 1u << (Lb.step & 31u);
			}
			++Lb.step;
			Lb.t = Lb.t_limit = t[k + 1];
			if ((m_zero >> k) & 1ull) count_finish(Lb, B);
		}
		bool same = La.phase == Lb.phase && La.j == Lb.j && La.logged == Lb.logged && La.mask[0] == Lb.mask[0] && La.mask[1] == Lb.mask[1] && La.mask[2] == Lb.mask[2]
		            && bits_a == bits_b && t0_a == t0_b && cnt_a == cnt_b && std::memcmp(&st_a, &st_b, sizeof(TrainRay)) == 0;
		if (La.phase != LANE_IDLE) same = same && La.step == Lb.step && La.t == Lb.t && La.word == Lb.word && La.cur_w == Lb.cur_w && (La.word == 0 || La.t_word == Lb.t_word);
		bad += !same;
	}
	return bad;
}

// table-driven skip-ahead of the generator against the plain one: number of (stream, state, delta) triples that differ
uint32_t hs_pcg_skip_mismatches(uint32_t seed, uint32_t n_cases) {
	Pcg32 g; pcg_seed(g, seed, 3);
	uint32_t bad = 0;
	for (uint32_t c = 0; c < n_cases; ++c) {
		Pcg32 a;
		pcg_seed(a, ((uint64_t)pcg_next_uint(g) << 32) | pcg_next_uint(g), pcg_next_uint(g));
		Pcg32 b = a;
		PcgSkip T;
		pcg_skip_table(a, T);
		uint32_t delta = pcg_next_uint(g);
		if (c % 7 == 0) delta = 0; else if (c % 7 == 1) delta = 0xffffffffu; else if (c % 7 == 2) delta >>= (c % 31);
		Pcg32 h = a;
		uint64_t m16[128], p16[128];
		for (uint32_t e = 0; e < 128; ++e) pcg_skip16_entry(a, e, &m16[e], &p16[e]);
		pcg_advance(a, (uint64_t)delta);
		pcg_advance_u32(b, delta, T);
		pcg_advance_skip16(h, delta, m16, p16);
		bad += a.state != b.state || a.inc != b.inc || a.state != h.state || a.inc != h.inc;
	}
	return bad;
}

void hs_set_sphere(const float sphere[4]) { for (int k = 0; k < 4; ++k) g_sphere[k] = sphere ? sphere[k] : 0.f; }

// stretch of n rays (origin, direction) inside a sphere; hit[i] = 0 for a miss
void hs_sphere_spans(uint32_t n, const float* rays, const float sphere[4], float* t0, float* t1, uint8_t* hit) {
	for (uint32_t i = 0; i < n; ++i) {
		const SphereSpan sp = sphere_ray_span(sphere, ld3(rays + 6 * (size_t)i), ld3(rays + 6 * (size_t)i + 3));
		t0[i] = sp.t0; t1[i] = sp.t1; hit[i] = sp.hit ? 1 : 0;
	}
}

// the reciprocal that the disparity chain carries: for how many of the 2^23 mantissas of g does one fused Newton step
// from g miss the correctly rounded 1/RN(1/g)?
uint32_t hs_carried_reciprocal_failures() {
	uint32_t fails = 0;
	for (uint32_t m = 0; m < (1u << 23); ++m) {
		const float g = srf_u2f(0x3f800000u | m);
		const float q = 1.0f / g;
		const float want = 1.0f / q;
		const float got = srf_fma(srf_fma(-q, g, 1.0f), g, g);
		fails += got != want;
	}
	return fails;
}

// short_chain_jump against the loop of additions it stands for, on random operands of every kind the marches can hand it
// (any binade, c from a few to millions of units of the binade's spacing, S anywhere between the lowest admissible value and r):
// out[0] = cases where the closed form applied, out[1] = cases it declined, return = cases where count or end value differ
uint32_t hs_chain_jump_mismatches(uint32_t seed, uint32_t n_cases, uint32_t* out) {
	uint64_t state = 0x9e3779b97f4a7c15ull * (seed + 1);
	auto next = [&]() { state = state * 6364136223846793005ull + 1442695040888963407ull; return (uint32_t)(state >> 33); };
	uint32_t bad = 0;
	out[0] = out[1] = 0;
	for (uint32_t it = 0; it < n_cases; ++it) {
		const uint32_t e = 40u + next() % 170u;                                  // binade
		const float bin = srf_u2f(e << 23);
		const uint32_t m = 0x00800000u | (next() & 0x007fffffu);
		float r = srf_u2f((e << 23) | (m & 0x007fffffu));
		// |c|: 1.5 .. 2^21 spacings, with a random mantissa; one case in eight exactly halfway between two multiples
		const uint32_t units = 2u + next() % (1u << (1 + next() % 21));
		float c = -(float)units * srf_u2f((e - 23u) << 23);
		if ((next() & 7u) == 0u) c -= 0.5f * srf_u2f((e - 23u) << 23);
		else c *= 1.0f + (float)(next() & 0xffffu) * (1.0f / 16777216.0f);
		const float S_lo = (bin - c) * 1.0000002f;
		if (!(r > S_lo) || (!(c + r < bin * 1.4142134f) && (next() & 1u))) continue;
		float S = S_lo + (r - S_lo) * ((float)(next() & 0xffffu) / 65536.0f);
		if (!(S >= S_lo)) S = S_lo;
		if (!(r > S)) continue;
		float r_loop = r;
		uint32_t k_loop = 0;
		do { r_loop = c + r_loop; ++k_loop; } while (r_loop > S && k_loop < (1u << 24));
		float r_jump = r;
		const uint32_t k = short_chain_jump(c, bin, S, r_jump);
		if (k == 0) { ++out[1]; if (srf_f2u(r_jump) != srf_f2u(r)) ++bad; continue; }
		++out[0];
		if (k != k_loop || srf_f2u(r_jump) != srf_f2u(r_loop)) ++bad;
	}
	return bad;
}

// n steps from t0 by calc_dt and by the short form (which stops where its range ends); returns the short form's step count
uint32_t hs_disparity_chains(const orc_params* p, float t0, uint32_t n, float* t_calc, float* t_short) {
	const Params P = to_params(p);
	const ShortForm f = disparity_short_form(P);
	float t = t0;
	for (uint32_t k = 0; k < n; ++k) { t_calc[k] = t; t += calc_dt(P, t, P.cone_angle_constant); }
	uint32_t taken = 0;
	if (f.usable && t0 >= f.t_lo) {
		ShortChain ch = short_chain_at(t0);
		while (taken < n && ch.t <= f.t_hi) { t_short[taken++] = ch.t; ch = short_chain_next(f, ch); }
		if (taken < n) t_short[taken++] = ch.t;      // the value the last covered step leads to
	}
	return taken;
}

// the stretch of ray parameter over which the sinusoidal warp is bounded to move less than rho, and the branch-cut window of the ray
float hs_skip_stretch(const float o[3], const float d[3], float t, float rho, float cut[2]) {
	const SkipRay R = skip_ray_setup(ld3(o), ld3(d));
	cut[0] = R.cut_lo; cut[1] = R.cut_hi;
	return skip_stretch(R, ld3(d), t, rho);
}

// empty-space table used by the render bodies below (NULL: probe every step)
static const uint16_t* g_render_skip = nullptr;
void hs_set_render_skip_table(const uint16_t* dist) { g_render_skip = dist; }

void hs_generate_rays(const orc_params* p, const int32_t res[2], const float focal[2], const float pp[2], const float cam[12], uint32_t spp,
                      const uint8_t* bitfield, srf_ray_payload* payloads) {
	const Params P = to_params(p);
	const PixelArgs A = pixel_args(P, res, focal, pp, cam, spp);
	for (int32_t y = 0; y < res[1]; ++y) for (int32_t x = 0; x < res[0]; ++x) init_ray_body((uint32_t)x, (uint32_t)y, P, A, payloads);
	const uint32_t n = (uint32_t)res[0] * (uint32_t)res[1];
	for (uint32_t i = 0; i < n; ++i) advance_pos_body(i, P, spp, payloads, P.use_grid ? bitfield : nullptr, skip_table_for(P, g_render_skip));
}

void hs_generate_coords(const orc_params* p, uint32_t n_rays, uint32_t n_steps, const uint8_t* bitfield, srf_ray_payload* payloads, float* coords) {
	const Params P = to_params(p);
	for (uint32_t i = 0; i < n_rays; ++i) generate_coords_body(i, P, n_steps, P.use_grid ? bitfield : nullptr, payloads, coords, skip_table_for(P, g_render_skip));
}

void hs_render_fused(const orc_params* p, const orc_field* f, const uint8_t* bitfield, const int32_t res[2], const float focal[2], const float pp[2],
                     const float cam[12], uint32_t spp, float thr, int to_linear, float* frame, uint32_t* n_samples) {
	const Params P = to_params(p);
	const PixelArgs A = pixel_args(P, res, focal, pp, cam, spp);
	FieldArgs F; F.table = f->table; F.mask = f->table_size - 1; F.seed = f->seed;
	const uint32_t n = (uint32_t)res[0] * (uint32_t)res[1];
	for (uint32_t i = 0; i < n; ++i) render_fused_body(i, P, A, spp, P.use_grid ? bitfield : nullptr, F, thr, to_linear, frame, n_samples, skip_table_for(P, g_render_skip));
}

void hs_loss(const orc_loss_args* a, const float* rays_rgba, uint32_t n_rays_counter, uint32_t* ray_coord_indices, const float* dt,
             const float* coords, float* compacted_coords, uint32_t* n_compacted_counter, const void* net, void* dloss, float* loss_output,
             float* reg_buffer, float* rgb_ray_out) {
	const LossConst K = make_loss_const(a);
	const uint32_t n = a->n_rays;
	std::vector<FwdRay> fwd(n);
	std::vector<uint32_t> nf(n), cb(n);
	const bool hin = a->network_output_dtype == ORC_DTYPE_F16, hout = a->dloss_dtype == ORC_DTYPE_F16;
	for (uint32_t i = 0; i < n; ++i) {
		if (hin) loss_forward_body<true>(i, K, rays_rgba, n_rays_counter, ray_coord_indices, dt, net, &fwd[i], &nf[i], rgb_ray_out);
		else loss_forward_body<false>(i, K, rays_rgba, n_rays_counter, ray_coord_indices, dt, net, &fwd[i], &nf[i], rgb_ray_out);
	}
	uint32_t run = *n_compacted_counter;
	for (uint32_t i = 0; i < n; ++i) { cb[i] = run; run += nf[i]; }
	*n_compacted_counter = run;
	float* reg = a->regularization_type == ORC_REG_DISTORTION ? reg_buffer : nullptr;
	for (uint32_t i = 0; i < n; ++i) {
		if (hin && hout) loss_backward_body<true, true>(i, K, n_rays_counter, ray_coord_indices, dt, coords, compacted_coords, net, dloss, loss_output, a->mean_density, fwd[i], nf[i], cb[i], reg);
		else if (hin) loss_backward_body<true, false>(i, K, n_rays_counter, ray_coord_indices, dt, coords, compacted_coords, net, dloss, loss_output, a->mean_density, fwd[i], nf[i], cb[i], reg);
		else if (hout) loss_backward_body<false, true>(i, K, n_rays_counter, ray_coord_indices, dt, coords, compacted_coords, net, dloss, loss_output, a->mean_density, fwd[i], nf[i], cb[i], reg);
		else loss_backward_body<false, false>(i, K, n_rays_counter, ray_coord_indices, dt, coords, compacted_coords, net, dloss, loss_output, a->mean_density, fwd[i], nf[i], cb[i], reg);
	}
}

void hs_fused_set_max_parts(uint32_t n) { g_fused_max_parts = n; }
uint32_t hs_fused_most_parts() { return g_fused_most_parts; }

void hs_loss_fused(const orc_loss_args* a, const float* rays_rgba, uint32_t n_rays_counter, uint32_t* ray_coord_indices, const float* dt,
                   const float* coords, float* compacted_coords, uint32_t* n_compacted_counter, const void* net, void* dloss, float* loss_output,
                   float* rgb_ray_out, uint32_t* n_scattered_groups, uint32_t* n_multi_window_groups) {
	const bool hin = a->network_output_dtype == ORC_DTYPE_F16, hout = a->dloss_dtype == ORC_DTYPE_F16;
	*n_scattered_groups = 0; *n_multi_window_groups = 0;
	g_fused_most_parts = 0;
#define RUN(HI, HO) run_fused<HI, HO>(a, rays_rgba, n_rays_counter, ray_coord_indices, dt, coords, compacted_coords, n_compacted_counter, net, dloss, loss_output, rgb_ray_out, n_scattered_groups, n_multi_window_groups)
	if (hin && hout) RUN(true, true); else if (hin) RUN(true, false); else if (hout) RUN(false, true); else RUN(false, false);
#undef RUN
}

void hs_loss_wave(const orc_loss_args* a, const float* rays_rgba, uint32_t n_rays_counter, uint32_t* ray_coord_indices, const float* dt,
                  const float* coords, float* compacted_coords, uint32_t* n_compacted_counter, const void* net, void* dloss, float* loss_output,
                  float* rgb_ray_out, uint32_t counts[4], uint32_t force_stride) {
	const bool hin = a->network_output_dtype == ORC_DTYPE_F16, hout = a->dloss_dtype == ORC_DTYPE_F16;
	counts[0] = counts[1] = counts[2] = counts[3] = 0;
#define RUN(HI, HO) run_wave<HI, HO>(a, rays_rgba, n_rays_counter, ray_coord_indices, dt, coords, compacted_coords, n_compacted_counter, net, dloss, loss_output, rgb_ray_out, counts, force_stride)
	if (hin && hout) RUN(true, true); else if (hin) RUN(true, false); else if (hout) RUN(false, true); else RUN(false, false);
#undef RUN
}

uint32_t hs_window_stride(uint32_t n_active, uint64_t span, uint64_t end, uint32_t item_cap) { return wv::window_stride(n_active, span, end, item_cap); }


void hs_volume_rendering(const orc_params* p, const orc_render_args* a, srf_ray_payload* payloads, float* rgba, const float* coords, const void* net) {
	const Params P = to_params(p);
	srf_render_args A;
	A.n_rays = a->n_rays; A.n_steps = a->n_steps; A.i_steps_offset = a->n_steps_offset; A.padded_output_width = a->padded_output_width;
	A.density_activation = a->density_activation; A.rgb_activation = a->rgb_activation; A.render_mode = a->render_mode;
	std::memcpy(A.camera_matrix, a->camera, sizeof(A.camera_matrix));
	A.depth_scale = a->depth_scale; A.network_output_dtype = a->network_output_dtype;
	for (uint32_t i = 0; i < a->n_rays; ++i) {
		if (a->network_output_dtype == ORC_DTYPE_F16) volume_rendering_body<true>(i, P, A, a->transmittance_threshold, payloads, rgba, coords, net);
		else volume_rendering_body<false>(i, P, A, a->transmittance_threshold, payloads, rgba, coords, net);
	}
}

void hs_shade(uint32_t n, const float* rgba, const srf_ray_payload* payloads, float* frame, int render_mode, int train_in_linear) {
	for (uint32_t i = 0; i < n; ++i) shade_body(i, rgba, payloads, frame, render_mode, train_in_linear);
}

} // extern "C"
