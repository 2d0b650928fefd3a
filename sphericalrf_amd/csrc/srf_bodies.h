// Per-item bodies of the thread-per-ray / thread-per-cell kernels, written as
// `__host__ __device__` functions of the item index so that the identical code can
// be run under a host compiler (bounds-checked, single-threaded) as well as being
// launched on the device.  Reference citations are per function.
#pragma once
#include "srf_device.h"
#include "srf_skip.h"

// hook for host builds that count how many steps of a march probe the grid
#ifndef SRF_COUNT_PROBE
#define SRF_COUNT_PROBE() ((void)0)
#endif

namespace srf {

struct alignas(16) Float4 { float x, y, z, w; };
struct alignas(8) U2 { uint32_t x, y; };
struct alignas(16) U4 { uint32_t x, y, z, w; };
SRF_HD Float4 mk4(float x, float y, float z, float w) { Float4 v; v.x = x; v.y = y; v.z = z; v.w = w; return v; }

struct DatasetArgs {
	uint32_t n_images;
	int32_t  res[2];
	float    focal[2];
	float    pp[2];
	const float*    xforms;
	const uint16_t* images;
	const uint16_t* prob;
};

// what the counting march of a training ray leaves for the writing march
struct TrainRay {
	float    o[3];
	float    d[3];
	float    startt;
	float    xy[2];
	uint32_t img;
	uint32_t logged;        // 1: every sample of the ray is in the step log
	uint32_t word_mask[3];  // which words of the step log hold samples
};
constexpr uint32_t LOG_MAX_WORDS = 96;

// The counting march leaves, for every aligned run of 32 steps that produced a sample, one word
// with a bit per step (1 = sample) and the value of t at the run's first sample, so that the
// writing march only replays the t chain from there to the run's last sample and evaluates the
// warp at the set bits.  Word w of ray i lives at [w * stride + i]: the rays of a wave touch
// consecutive addresses.  Runs without samples are not stored; the ray's word_mask says which are.
struct StepLog { uint32_t* bits; float* t0; uint32_t stride; uint32_t words; };

SRF_HD void step_log_flush(const StepLog& log, uint32_t i, uint32_t w, uint32_t word, float t_word, bool& logged, uint32_t* mask) {
	if (!word || !logged) return;
	if (w >= log.words) { logged = false; return; }
	log.bits[(size_t)w * log.stride + i] = word;
	log.t0[(size_t)w * log.stride + i] = t_word;
	const uint32_t bit = 1u << (w & 31u);
	mask[0] |= w < 32u ? bit : 0u;
	mask[1] |= (w >= 32u && w < 64u) ? bit : 0u;
	mask[2] |= w >= 64u ? bit : 0u;
}

SRF_HD uint64_t pixel_index(const float xy[2], const int32_t res[2], uint32_t img) {   // common_device.h:191-201
	const int32_t px = clamp_i(srf_f2i(xy[0] * (float)res[0]), 0, res[0] - 1);
	const int32_t py = clamp_i(srf_f2i(xy[1] * (float)res[1]), 0, res[1] - 1);
	return (uint64_t)px + (uint64_t)py * (uint64_t)res[0] + (uint64_t)img * (uint64_t)res[0] * (uint64_t)res[1];
}

// ---- display post-process (internal/utils/render_buffer.cu) ----------------------------------
// render_buffer.cu:46-85 — the running mean over the frames accumulated so far; an sRGB buffer takes the frame encoded
SRF_HD Float4 accumulate_body(Float4 color, Float4 tmp, float sample_count, int32_t color_space) {
	if (color_space == SRF_COLOR_VISPOSNEG) {
		const float val = color.x - color.y;
		float tmp_val = tmp.x - tmp.y;
		tmp_val = (tmp_val * sample_count + val) / (sample_count + 1);
		tmp.x = srf_max(tmp_val, 0.0f);
		tmp.y = srf_max(-tmp_val, 0.0f);
	} else {
		if (color_space == SRF_COLOR_SRGB) { color.x = linear_to_srgb(color.x); color.y = linear_to_srgb(color.y); color.z = linear_to_srgb(color.z); }
		tmp.x = (tmp.x * sample_count + color.x) / (sample_count + 1);
		tmp.y = (tmp.y * sample_count + color.y) / (sample_count + 1);
		tmp.z = (tmp.z * sample_count + color.z) / (sample_count + 1);
	}
	tmp.w = (tmp.w * sample_count + color.w) / (sample_count + 1);
	return tmp;
}

struct TonemapArgs { float scale; float background[4]; int32_t color_space, output_color_space, curve; };

// render_buffer.cu:87-140 — the tone curves: rational polynomials with the exposure bias and white point folded into their coefficients
SRF_HD void tonemap_curve(float x[3], int32_t curve) {
	if (curve == SRF_TONEMAP_IDENTITY) return;
	for (int c = 0; c < 3; ++c) x[c] = srf_max(x[c], 0.f);
	float k0, k1, k2, k3, k4, k5;
	if (curve == SRF_TONEMAP_ACES) {
		k0 = 0.6f * 0.6f * 2.51f; k1 = 0.6f * 0.03f; k2 = 0.0f; k3 = 0.6f * 0.6f * 2.43f; k4 = 0.6f * 0.59f; k5 = 0.14f;
	} else if (curve == SRF_TONEMAP_HABLE) {
		const float A = 0.15f, B = 0.50f, C = 0.10f, D = 0.20f, E = 0.02f, F = 0.30f, W = 11.2f;
		k0 = A * F - A * E; k1 = C * B * F - B * E; k2 = 0.0f; k3 = A * F; k4 = B * F; k5 = D * F * F;
		const float nom = k0 * (W * W) + k1 * W + k2, denom = k3 * (W * W) + k4 * W + k5;
		const float white_scale = denom / nom;
		k0 = 4.0f * k0 * white_scale; k1 = 2.0f * k1 * white_scale; k2 = k2 * white_scale; k3 = 4.0f * k3; k4 = 2.0f * k4;
	} else {   // Reinhard, on the luminance
		const float Y = (0.2126f * x[0] + 0.7152f * x[1]) + 0.0722f * x[2];
		const float k = 1.f / (Y + 1.0f);
		for (int c = 0; c < 3; ++c) x[c] = x[c] * k;
		return;
	}
	for (int c = 0; c < 3; ++c) {
		const float sq = x[c] * x[c];
		const float nom = (sq * k0 + k1 * x[c]) + k2, denom = (k3 * sq + k4 * x[c]) + k5;
		x[c] = nom / denom;
	}
}

// render_buffer.cu:142-178 — one pixel from the accumulation buffer to the display buffer
SRF_HD Float4 tonemap_body(Float4 color, const TonemapArgs& A) {
	float rgb[3] = {color.x * A.scale, color.y * A.scale, color.z * A.scale};
	float bg[3] = {A.background[0], A.background[1], A.background[2]};
	if (A.color_space != SRF_COLOR_SRGB) for (int c = 0; c < 3; ++c) bg[c] = srgb_to_linear(bg[c]);     // the background colour is given in sRGB
	const float weight = (1 - color.w) * A.background[3];
	for (int c = 0; c < 3; ++c) rgb[c] += bg[c] * weight;
	const float alpha = color.w + weight;
	if (A.color_space == SRF_COLOR_SRGB) for (int c = 0; c < 3; ++c) rgb[c] = srgb_to_linear(rgb[c]);
	tonemap_curve(rgb, A.curve);
	if (A.output_color_space == SRF_COLOR_SRGB) for (int c = 0; c < 3; ++c) rgb[c] = linear_to_srgb(rgb[c]);
	return mk4(rgb[0], rgb[1], rgb[2], alpha);
}

// occupancy_sampler.cu:28-80 — where cell i of the cascaded grid lies in metric space and how far its corners reach, as the
// camera-visibility mask sees them.  The reference's switch over the grid distribution falls through from MetricSpace_Exp into
// MetricSpace_Reciprocal (:52-57), so a MetricSpace_Exp grid is scaled and shifted twice; that is kept.  (The reference's grid is
// cubic: the radius uses the first axis' size.)
SRF_HD void mask_cell(uint32_t i, const Params& P, Vec3* centre, float* radius) {
	const uint32_t level = i / P.n_cells, cell = i % P.n_cells;
	Vec3 p = mk3(((float)morton3d_invert(cell >> 0) + 0.5f) / (float)P.grid_size[0] - 0.5f,
	             ((float)morton3d_invert(cell >> 1) + 0.5f) / (float)P.grid_size[1] - 0.5f,
	             ((float)morton3d_invert(cell >> 2) + 0.5f) / (float)P.grid_size[2] - 0.5f);
	const float shrink = srf_exp2i(-(int)(P.n_cascades - level - 1)), parts = (float)(P.n_cascades - level);
	float r = 0.5f * 1.73205080757f * (float)P.aabb_scale / (float)P.grid_size[0];
	const bool metric = P.griddist_type == SRF_GRID_METRIC_EXP || P.griddist_type == SRF_GRID_METRIC_RECIPROCAL;
	if (P.griddist_type == SRF_GRID_WARPED_EXP) p = mk3(p.x * shrink + 0.5f, p.y * shrink + 0.5f, p.z * shrink + 0.5f);
	else if (P.griddist_type == SRF_GRID_WARPED_RECIPROCAL) p = mk3(p.x / parts + 0.5f, p.y / parts + 0.5f, p.z / parts + 0.5f);
	if (P.griddist_type == SRF_GRID_METRIC_EXP) { const float k = (float)P.aabb_scale * shrink; p = mk3(p.x * k + 0.5f, p.y * k + 0.5f, p.z * k + 0.5f); }
	if (metric) { const float k = (float)P.aabb_scale / parts; p = mk3(p.x * k + 0.5f, p.y * k + 0.5f, p.z * k + 0.5f); }
	else p = unwarp_position(P, p);
	if (P.griddist_type == SRF_GRID_WARPED_EXP || P.griddist_type == SRF_GRID_METRIC_EXP) r *= shrink; else r /= parts;
	*centre = p; *radius = r;
}

// occupancy_sampler.cu:82-99 — does the camera with the column-major 3x4 matrix m see a ball of that radius round the point
SRF_HD bool mask_camera_sees(const float* m, Vec3 p, float radius, float focal_x, float focal_y, float half_res_x, float half_res_y) {
	const Vec3 l = mk3(p.x - m[9], p.y - m[10], p.z - m[11]);
	const float cx = (l.x * m[0] + l.y * m[1]) + l.z * m[2];
	const float cy = (l.x * m[3] + l.y * m[4]) + l.z * m[5];
	const float cz = (l.x * m[6] + l.y * m[7]) + l.z * m[8];
	return cz > 0.f && srf_abs(cx) - radius < cz / focal_x * half_res_x && srf_abs(cy) - radius < cz / focal_y * half_res_y;
}

// ------------------------------------------------------------------------------------
// occupancy_sampler.cu:104-185 — one candidate point: pick a cascade, probe up to ten
// hashed cells for one above the threshold, jitter a point inside it.
// ------------------------------------------------------------------------------------
// occupancy_sampler.cu:121-130 — the up to ten tries of one point; POW2: the cell count is a power of two
// The ten candidate cells do not depend on what the grid holds, so BATCH of them (1, 2, 5 or 10) are looked up side by side;
// the first that passes, in the reference's order, is taken, the tenth if none does.  One dependent lookup after the other
// makes a wavefront wait for its unluckiest lane, a memory round trip per try.
template <bool POW2, uint32_t BATCH>
SRF_HD void grid_sample_tries_batched(uint32_t i, const Params& P, uint32_t n_elements, uint32_t step, uint32_t level, const float* grid_in, float thresh,
                                      const uint32_t* above, uint32_t* cell_out, uint32_t* idx_out, const uint32_t* above_summary = nullptr) {
	static_assert(10 % BATCH == 0, "whole batches");
	uint32_t cell = 0, idx = 0;
	bool found = false;
	const uint32_t h0 = (i + step * n_elements) * 56924617u + 96925573u;
	for (uint32_t j0 = 0; j0 < 10 && !found; j0 += BATCH) {
		uint32_t c[BATCH], id[BATCH];
		bool pass[BATCH];
#if defined(__HIP_DEVICE_COMPILE__)
		#pragma unroll
#endif
		for (uint32_t q = 0; q < BATCH; ++q) {
			const uint32_t h = h0 + (j0 + q) * 19349663u;
			c[q] = POW2 ? (h & (P.n_cells - 1u)) : (h % P.n_cells);
			id[q] = c[q] + level * P.n_cells;
			// above_summary: one bit per word of `above`, set where the word has a cell that fails: a table small enough for the
			// nearest cache, and where hardly any cell fails (the uniform draw: only masked cells do) it answers nearly every lookup
			const uint32_t word = id[q] >> 5;
			if (above_summary && ((above_summary[word >> 5] >> (word & 31u)) & 1u) == 0u) pass[q] = true;
			else pass[q] = above ? ((above[word] >> (id[q] & 31u)) & 1u) != 0u : grid_in[id[q]] > thresh;
		}
#if defined(__HIP_DEVICE_COMPILE__)
		#pragma unroll
#endif
		for (uint32_t q = 0; q < BATCH; ++q) {
			if (!found) { cell = c[q]; idx = id[q]; found = pass[q]; }
		}
	}
	*cell_out = cell;
	*idx_out = idx;
}
template <bool POW2>
SRF_HD void grid_sample_tries(uint32_t i, const Params& P, uint32_t n_elements, uint32_t step, uint32_t level, const float* grid_in, float thresh,
                              const uint32_t* above, uint32_t tries_at_once, uint32_t* cell_out, uint32_t* idx_out, const uint32_t* above_summary = nullptr) {
	if (tries_at_once >= 10u) grid_sample_tries_batched<POW2, 10>(i, P, n_elements, step, level, grid_in, thresh, above, cell_out, idx_out, above_summary);
	else if (tries_at_once >= 5u) grid_sample_tries_batched<POW2, 5>(i, P, n_elements, step, level, grid_in, thresh, above, cell_out, idx_out, above_summary);
	else if (tries_at_once >= 2u) grid_sample_tries_batched<POW2, 2>(i, P, n_elements, step, level, grid_in, thresh, above, cell_out, idx_out, above_summary);
	else grid_sample_tries_batched<POW2, 1>(i, P, n_elements, step, level, grid_in, thresh, above, cell_out, idx_out, above_summary);
}

// above: optional table of the comparison grid_in[idx] > thresh, one bit per cell (bit idx & 31 of word idx >> 5),
// 32 times smaller than the grid, so that the random lookups below mostly stay in the caches
SRF_HD void grid_sample_point(uint32_t i, const Params& P, uint32_t n_elements, Pcg32 rng, uint32_t step,
                              const float* grid_in, float thresh, Vec3* position, uint32_t* index, const uint32_t* above = nullptr,
                              const PcgSkip* skip = nullptr, uint32_t tries_at_once = 1,
                             const uint64_t* skip16_m = nullptr, const uint64_t* skip16_p = nullptr, const uint32_t* above_summary = nullptr) {
	if (skip16_m) pcg_advance_skip16(rng, i * 4u, skip16_m, skip16_p);
	else if (skip) pcg_advance_u32(rng, i * 4u, *skip);
	else pcg_advance(rng, (uint64_t)(uint32_t)(i * 4u));
	// (uint32_t)(f * C) % C with f in [0, 1): the product is at most C, so the remainder only matters when it is C itself
	const uint32_t scaled = (uint32_t)(pcg_next_float(rng) * (float)P.n_cascades);
	const uint32_t level = scaled >= P.n_cascades ? scaled - P.n_cascades : scaled;
	// the remainder by the cell count is a mask when that is a power of two (every grid the library accepts for ERP has one;
	// an integer division costs some forty instructions, and there are up to ten here)
	const bool pow2 = (P.n_cells & (P.n_cells - 1u)) == 0u;
	uint32_t cell = 0, idx = 0;
	if (pow2) grid_sample_tries<true>(i, P, n_elements, step, level, grid_in, thresh, above, tries_at_once, &cell, &idx, above_summary);
	else grid_sample_tries<false>(i, P, n_elements, step, level, grid_in, thresh, above, tries_at_once, &cell, &idx, above_summary);
	const uint32_t x = morton3d_invert(cell), y = morton3d_invert(cell >> 1), z = morton3d_invert(cell >> 2);
	const float jx = pcg_next_float(rng), jy = pcg_next_float(rng), jz = pcg_next_float(rng);
	Vec3 pos = mk3(((float)x + jx) / (float)P.grid_size[0] - 0.5f, ((float)y + jy) / (float)P.grid_size[1] - 0.5f,
	               ((float)z + jz) / (float)P.grid_size[2] - 0.5f);
	switch (P.griddist_type) {
	case SRF_GRID_WARPED_EXP:
		pos = shift3(scale3(pos, srf_exp2i(-(int)(P.n_cascades - level - 1))), 0.5f);
		break;
	case SRF_GRID_WARPED_RECIPROCAL:
		pos = shift3(scale3(pos, 1.f / (float)(P.n_cascades - level)), 0.5f);
		break;
	case SRF_GRID_METRIC_EXP:
		pos = shift3(scale3(pos, (float)P.aabb_scale * srf_exp2i(-(int)(P.n_cascades - level - 1))), 0.5f);
		pos = warp_position(P, pos);
		break;
	case SRF_GRID_METRIC_RECIPROCAL:
		pos = shift3(scale3(pos, (float)P.aabb_scale / (float)(P.n_cascades - level)), 0.5f);
		pos = warp_position(P, pos);
		break;
	}
	*position = pos;
	*index = idx;
}

SRF_HD void grid_sample_body(uint32_t i, const Params& P, uint32_t n_elements, Pcg32 rng, uint32_t step,
                             const float* grid_in, float thresh, float* positions, uint32_t* indices, const uint32_t* above = nullptr,
                             const PcgSkip* skip = nullptr, uint32_t tries_at_once = 1,
                             const uint64_t* skip16_m = nullptr, const uint64_t* skip16_p = nullptr, const uint32_t* above_summary = nullptr) {
	Vec3 pos;
	uint32_t idx;
	grid_sample_point(i, P, n_elements, rng, step, grid_in, thresh, &pos, &idx, above, skip, tries_at_once, skip16_m, skip16_p, above_summary);
	st3(positions + 3 * (size_t)i, pos);
	indices[i] = idx;
}

// ------------------------------------------------------------------------------------
// occupancy_sampler.cu:552-637 — ray set-up and the counting march of one training ray
// ------------------------------------------------------------------------------------
// The counting march is written as a small state machine per ray so that a wavefront can run
// its lanes' rays phase by phase (all lanes that need a grid probe together, all lanes that are
// stepping through known-empty space together, idle lanes picking up the next ray) instead of
// in lockstep; the order in which phases run never changes what a ray computes.
enum : uint32_t { LANE_IDLE = 0, LANE_PROBE = 1, LANE_STEP = 2 };

// A ray that has used up its probe budget in the lane-per-ray march is parked here, as it stands, and finished by a
// whole wavefront (wide_* below): rays that need a lookup at nearly every step would otherwise keep one lane, and with
// it the wavefront, busy for thousands of memory round trips.
struct ParkedRay {
	uint32_t i, img, j, step, word, cur_w, logged;
	uint32_t mask[3];
	float o[3], d[3];
	float t, t_word, startt;
	float xy[2];
};

struct CountArgs {
	uint32_t n_rays, n_rays_shift;
	DatasetArgs ds;
	const uint8_t* bitfield;
	Pcg32 rng;
	TrainRay* state;
	uint32_t* counts;
	StepLog log;
	SkipTable skip;
	// parking: budget of probes per ray (0 = never park), the queue, its capacity, its fill counter; a wavefront only parks
	// rays once it has no more than park_lanes rays under way
	uint32_t probe_budget, park_lanes;
	ParkedRay* parked;
	uint32_t parked_capacity;
	uint32_t* parked_count;
};

struct CountLane {
	uint32_t phase;
	uint32_t i;             // ray
	Vec3 o, d;
	float t, t_limit, t_word, startt;   // t_word: t at the first sample of the log word being filled
	float xy[2];
	uint32_t img, j, step, word, cur_w;  // cur_w: index of the log word being filled
	uint32_t probes;                     // lookups since the ray began (or since parking it last failed)
	uint32_t mask[3];
	bool logged;
	SkipRay sr;
};

SRF_HD void count_finish(CountLane& L, const CountArgs& A) {
	step_log_flush(A.log, L.i, L.cur_w, L.word, L.t_word, L.logged, L.mask);
	TrainRay st;
	st3(st.o, L.o); st3(st.d, L.d); st.startt = L.startt;
	st.xy[0] = L.xy[0]; st.xy[1] = L.xy[1]; st.img = L.img;
	st.logged = L.logged ? 1u : 0u;
	st.word_mask[0] = L.mask[0]; st.word_mask[1] = L.mask[1]; st.word_mask[2] = L.mask[2];
	A.state[L.i] = st;
	A.counts[L.i] = L.j;
	L.phase = LANE_IDLE;
}

// occupancy_sampler.cu:552-594 — pixel choice, ray through it, jittered start
// occupancy_sampler.cu:556 — image that training ray i is drawn from
SRF_HD uint32_t train_ray_image(uint32_t i, const CountArgs& A) {
	return (uint32_t)((uint32_t)((A.n_rays_shift + i) * A.ds.n_images) / A.n_rays) % A.ds.n_images;
}

// occupancy_sampler.cu:556-575 — image and pixel of training ray i; leaves rng where the ray's start jitter is drawn next
SRF_HD uint32_t train_ray_pixel(uint32_t i, const Params& P, const CountArgs& A, Pcg32& rng, float xy[2]) {
	const DatasetArgs& ds = A.ds;
	const uint32_t img = train_ray_image(i, A);
	rng = A.rng;
	pcg_advance(rng, (uint64_t)(uint32_t)(i * 8u));
	xy[0] = pcg_next_float(rng);
	xy[1] = pcg_next_float(rng);
	if (P.snap_train) {
		for (int a = 0; a < 2; ++a) {
			int32_t px = srf_f2i(xy[a] * (float)ds.res[a]);   // cast<int>().cwiseMax(0).cwiseMin(res - 1)
			px = px < 0 ? 0 : px;
			px = px > ds.res[a] - 1 ? ds.res[a] - 1 : px;
			xy[a] = ((float)px + 0.5f) / (float)ds.res[a];
		}
	}
	return img;
}

// Marching order.  Which lane marches which ray has no effect on any output; rays that travel together take similar
// numbers of probes and steps, which is what a wavefront needs.  Rays are reordered within chunks of RAY_CHUNK
// consecutive indices (consecutive indices already share an image or a few) by a key that brings neighbouring pixels of
// one image together: image relative to the chunk's first, then the Morton code of the pixel's tile on a 16 x 16 tiling.
constexpr uint32_t RAY_CHUNK = 4096;
constexpr uint32_t RAY_CHUNK_BINS = 1024;
SRF_HD uint32_t ray_chunk_key_body(uint32_t i, uint32_t chunk_image, const Params& P, const CountArgs& A) {
	Pcg32 rng;
	float xy[2];
	const uint32_t img = train_ray_pixel(i, P, A, rng, xy);
	uint32_t code[2];
	for (int a = 0; a < 2; ++a) {
		int32_t c = srf_f2i(xy[a] * 16.f);
		c = c < 0 ? 0 : (c > 15 ? 15 : c);
		uint32_t v = (uint32_t)c;                 // spread 4 bits to the even positions
		v = (v | (v << 2)) & 0x33u;
		v = (v | (v << 1)) & 0x55u;
		code[a] = v;
	}
	const uint32_t rel = (img + A.ds.n_images - chunk_image) % A.ds.n_images;
	const uint32_t key = (rel << 8) | code[0] | (code[1] << 1);
	return key < RAY_CHUNK_BINS ? key : RAY_CHUNK_BINS - 1;
}

SRF_HD void count_begin(CountLane& L, uint32_t i, const Params& P, const CountArgs& A) {
	const DatasetArgs& ds = A.ds;
	Pcg32 rng;
	float xy[2];
	const uint32_t img = train_ray_pixel(i, P, A, rng, xy);
	const float* xform = ds.xforms + (size_t)img * 12;
	L.i = i; L.img = img; L.xy[0] = xy[0]; L.xy[1] = xy[1];
	L.j = 0; L.step = 0; L.word = 0; L.cur_w = 0; L.probes = 0;
	L.mask[0] = L.mask[1] = L.mask[2] = 0u;
	L.logged = true;
	L.o = mk3(0.f, 0.f, 0.f); L.d = L.o;
	L.startt = L.t = L.t_limit = L.t_word = 0.f;
	bool eligible = true;
	if (ds.prob) eligible = !(half_bits_to_float(ds.prob[pixel_index(xy, ds.res, img)]) <= 0.f);      // occupancy_sampler.cu:571 keeps a NaN probability
	if (!eligible) { count_finish(L, A); return; }
	ray_through(xform, xy[0], xy[1], ds.res, ds.focal, ds.pp, &L.o, &L.d);
	float tmin, tmax;
	aabb_ray_intersect(P, L.o, L.d, &tmin, &tmax);
	tmin = srf_max(tmin, P.near_distance);
	float startt = tmin;
	startt += calc_dt(P, startt, P.cone_angle_constant) * pcg_next_float(rng);
	L.startt = L.t = L.t_limit = L.t_word = startt;
	L.logged = A.log.bits != nullptr;
	if (A.skip.dist != nullptr && P.use_grid) L.sr = skip_ray_setup(L.o, L.d);
	L.phase = LANE_PROBE;
}

// one step of the chain: occupancy_sampler.cu:629-632 (t += dt; a zero step ends the march)
SRF_HD void count_advance(CountLane& L, const CountArgs& A, float dt) {
	++L.step;
	L.t += dt;
	if (dt == 0.f) count_finish(L, A);
}

// hands the ray over to the wide march; false when the queue is full (the lane then carries on)
SRF_HD bool count_park(CountLane& L, const CountArgs& A) {
#if defined(__HIP_DEVICE_COMPILE__)
	const uint32_t slot = atomicAdd(A.parked_count, 1u);
#else
	const uint32_t slot = (*A.parked_count)++;
#endif
	if (slot >= A.parked_capacity) { L.probes = 0; return false; }
	ParkedRay r;
	r.i = L.i; r.img = L.img; r.j = L.j; r.step = L.step; r.word = L.word; r.cur_w = L.cur_w; r.logged = L.logged ? 1u : 0u;
	r.mask[0] = L.mask[0]; r.mask[1] = L.mask[1]; r.mask[2] = L.mask[2];
	st3(r.o, L.o); st3(r.d, L.d);
	r.t = L.t; r.t_word = L.t_word; r.startt = L.startt;
	r.xy[0] = L.xy[0]; r.xy[1] = L.xy[1];
	A.parked[slot] = r;
	L.phase = LANE_IDLE;
	return true;
}

SRF_HD void count_unpark(CountLane& L, const ParkedRay& r) {
	L.i = r.i; L.img = r.img; L.j = r.j; L.step = r.step; L.word = r.word; L.cur_w = r.cur_w; L.logged = r.logged != 0u;
	L.mask[0] = r.mask[0]; L.mask[1] = r.mask[1]; L.mask[2] = r.mask[2];
	L.o = ld3(r.o); L.d = ld3(r.d);
	L.t = L.t_limit = r.t; L.t_word = r.t_word; L.startt = r.startt;
	L.xy[0] = r.xy[0]; L.xy[1] = r.xy[1];
	L.probes = 0;
	L.phase = LANE_PROBE;
}

// occupancy_sampler.cu:595-628 — a step that looks its cell up
// SPHERE = false compiles the optional sphere bound out (the counting kernel is short of registers; it is built both ways)
template <bool SPHERE = true>
SRF_HD void count_probe(CountLane& L, const Params& P, const CountArgs& A, bool may_park = true) {
	const Vec3 pos = along(L.o, L.d, L.t);
	if (!(aabb_contains(P, pos) && L.j < P.n_max_steps)) { count_finish(L, A); return; }
	if (SPHERE && P.sphere[3] > 0.f) {      // optional sphere bound: no sample outside it, the chain of t as it is
		float t_enter;
		const SphereGate g = sphere_gate(P, L.o, L.d, L.t, &t_enter);
		if (g == SPHERE_BEYOND) { count_finish(L, A); return; }
		if (g == SPHERE_BEFORE) {
			L.t_limit = t_enter;
			count_advance(L, A, calc_dt(P, L.t, P.cone_angle_constant));
			if (L.phase != LANE_IDLE) L.phase = L.t < L.t_limit ? LANE_STEP : LANE_PROBE;
			return;
		}
	}
	if (may_park && A.probe_budget && L.probes >= A.probe_budget && count_park(L, A)) return;
	++L.probes;
	SRF_COUNT_PROBE();
	const Probe s = probe_at(P, P.use_grid ? A.bitfield : nullptr, pos, L.t, P.cone_angle_constant, &A.skip);
	L.t_limit = L.t;   // steps at t' < t_limit are known to find an empty cell
	if (s.occ) {
		++L.j;
		const uint32_t w = L.step >> 5;
		if (w != L.cur_w) {
			step_log_flush(A.log, L.i, L.cur_w, L.word, L.t_word, L.logged, L.mask);
			L.word = 0;
			L.cur_w = w;
		}
		if (!L.word) L.t_word = L.t;
		L.word |= 1u << (L.step & 31u);
	}
	else if (A.skip.dist != nullptr && P.use_grid) L.t_limit = skip_limit(P, A.skip, L.sr, L.o, L.d, L.t, s.radius, s.level);
	count_advance(L, A, s.dt);
	if (L.phase != LANE_IDLE) L.phase = L.t < L.t_limit ? LANE_STEP : LANE_PROBE;
}

// up to K steps through space the last probe proved empty: the same t chain, no lookup, no sample.
// Disparity stepping runs as K predicated iterations without branches (a lane that has reached its
// limit idles through the rest), because per-step control flow costs more than the arithmetic:
// calc_dt's disparity branch without its clamps, valid while t stays where neither t, 1/t nor
// c + 1/t comes near the ends of the normal range and the step is positive; the first step that
// does not qualify goes through calc_dt.
// The disparity chain t' = t + (1/(c + 1/t) - t) in its short form, for t in [t_lo, t_hi] with c < 0:
//  * below t_lo the step c would drown in the rounding of 1/t; from t_lo on, c + 1/t is at least three ulps below
//    1/t, which makes every step positive and calc_dt's clamps idle;
//  * up to t_hi = 0.49/|c| the next value q = 1/(c + 1/t) is below 2t, so q - t is exact and t + (q - t) is q itself:
//    the chain is t' = q;
//  * the reciprocal of t' that the following step needs is one fused Newton step from g = c + 1/t, the number whose
//    reciprocal t' is: r' = g + g*(1 - t'*g).  For every float g this is the correctly rounded 1/RN(1/g) (checked for
//    all 2^23 mantissas; tests/test_disparity_chain.py), so a step costs one hardware reciprocal instead of two.
// Every quotient is the correctly rounded one, so the values are those of calc_dt's divisions.
struct ShortForm { bool usable; float c, t_lo, t_hi; };
SRF_HD ShortForm disparity_short_form(const Params& P) {
	ShortForm f;
	f.c = (1.f / (float)P.n_max_steps) * (1.f / P.far_distance - 1.f / P.near_distance);
	f.t_lo = f.c < 0.f ? srf_max(1e-18f, 9.5367432e-7f / -f.c) : 3e38f;
	f.t_hi = f.c < 0.f ? 0.49f / (1e-18f - f.c) : 0.f;
	f.usable = P.sampling_type == SRF_SAMPLING_DISPARITY && f.t_hi > f.t_lo;
	return f;
}
// t and its reciprocal, carried from step to step
struct ShortChain { float t, r; };
SRF_HD ShortChain short_chain_at(float t) { ShortChain ch; ch.t = t; ch.r = srf_rcp_normal(t); return ch; }
// one step from ch.t in [t_lo, t_hi]
SRF_HD ShortChain short_chain_next(const ShortForm& f, const ShortChain& ch) {
	const float g = f.c + ch.r;
	ShortChain n;
	n.t = srf_rcp_normal(g);
	n.r = srf_fma(srf_fma(-n.t, g, 1.0f), g, g);
	return n;
}

// Many steps at once.  For a float g whose mantissa is below sqrt 2 the reciprocal of its reciprocal (both correctly rounded) is g
// itself (every such mantissa checked: tests/test_disparity_chain.py), so while g = c + r stays in that lower part of a binade
// [B, 2B) the reciprocal the chain carries is g and a step is the addition r <- c + r.  In one binade the floats are the
// multiples m u of u = 2^-23 B, and c + r rounds to (m - q) u with q = |c| / u rounded to the nearest integer: the same q at every
// step, unless |c| / u lies exactly halfway between two integers (the rounding then goes by m's parity).  The loop
//     do r = c + r; while (r > S);
// entered with r > S, therefore runs k = ceil((m - s) / q) times (S = s u, rounded down) and ends at (m - k q) u.
// Asked of the caller: c < 0, r > S, both in the binade whose lowest value is `bin`, S >= (bin - c) (1 + 2^-22) so that the last sum
// still lies in it, and c + r below sqrt 2 * bin.  Returns k with r moved there, or 0 with r untouched where the closed form
// does not hold (the halfway case, a q the mantissa arithmetic does not cover, operands in different binades).
SRF_HD uint32_t short_chain_jump(float c, float bin, float S, float& r) {
	const uint32_t rb = srf_f2u(r), sb = srf_f2u(S), eb = srf_f2u(bin);
	if ((rb & 0x7f800000u) != eb || (sb & 0x7f800000u) != eb || eb < (25u << 23)) return 0u;
	const float inv_u = srf_u2f(((254u + 23u) << 23) - eb);      // 1 / u = 2^23 / bin
	const float cu = -c * inv_u;                                    // |c| in units of u: exact (a power of two times c)
	if (!(cu >= 1.0f && cu < 4194304.0f)) return 0u;
	const float whole = __builtin_floorf(cu), part = cu - whole;    // below 2^22 a float has at least one fractional bit: part is exact
	if (part == 0.5f) return 0u;
	const uint32_t q = (uint32_t)whole + (part > 0.5f ? 1u : 0u);
	const uint32_t m = (rb & 0x007fffffu) | 0x00800000u, s_int = (sb & 0x007fffffu) | 0x00800000u;
	const uint32_t a = m - s_int;                                   // > 0: r > S
	uint32_t k = (uint32_t)((float)a * srf_approx_rcp((float)q));   // a / q to within a few units, then made exact
	while (k * q < a) ++k;
	while (k > 1u && (k - 1u) * q >= a) --k;
	if (k == 0u) k = 1u;
	const uint32_t m_end = m - k * q;
	if (k * q >= m || m_end < 0x00800000u) return 0u;              // (the caller's S rules this out)
	r = srf_u2f(eb | (m_end & 0x007fffffu));
	return k;
}

// does any lane of the wavefront that is executing this (on the host: the one caller) hold the condition?
#if defined(__HIP_DEVICE_COMPILE__)
#define SRF_WAVE_ANY(p) (__ballot(p) != 0ull)
#else
#define SRF_WAVE_ANY(p) (p)
#endif

template <uint32_t K>
SRF_HD void count_steps(CountLane& L, const Params& P, const CountArgs& A) {
	{
		const ShortForm f = disparity_short_form(P);
		const float t_lo = f.t_lo, t_hi = f.t_hi;
		// t only grows, and the burst only takes steps that start below both the lane's limit and the end of the
		// short form's range, so checking the lower end once covers every step of the burst
		if (f.usable) {
			ShortChain ch = short_chain_at(L.t);
			float t = L.t;
			uint32_t n = 0;
			const float lim = srf_min(L.t_limit, t_hi);
			bool go = (t >= t_lo) & (t < lim);
			{
				// the stretch's steps inside the lower part of a binade, all at once (short_chain_jump); what is left (the upper
				// part, the last few steps before the limit, the cases the closed form leaves out) goes through the burst below
				const float g1 = f.c + ch.r;
				const float bin = srf_u2f(srf_f2u(ch.r) & 0x7f800000u);
				const float G = srf_approx_rcp(lim) * 1.000001f;      // r > G implies RN(1/r) < lim (see march_steps)
				const float S = srf_max(G, (bin - f.c) * 1.0000002f);
				if (go & (g1 >= bin) & (g1 < bin * 1.4142134f) & (ch.r > S)) {
					float r = ch.r;
					const uint32_t taken = short_chain_jump(f.c, bin, S, r);
					if (taken) {
						ch.r = r;
						ch.t = srf_rcp_normal(r);
						t = ch.t;
						n = taken;
						go = t < lim;
					}
				}
			}
			// in groups of four; the wavefront leaves as soon as none of its stepping lanes has a step left (after a jump most have not)
			for (uint32_t k0 = 0; k0 < K; k0 += 4u) {
				if (!SRF_WAVE_ANY(go)) break;
#if defined(__HIP_DEVICE_COMPILE__)
				#pragma unroll
#endif
				for (uint32_t k = 0; k < 4u; ++k) {
					ch = short_chain_next(f, ch);      // a lane that has stopped runs on idle: its chain is not looked at again
					const bool ok = go;
					const float tn = ch.t;
					t = ok ? tn : t;
					n += ok ? 1u : 0u;
					go = ok & (tn < lim);
				}
			}
			L.t = t;
			L.step += n;
			if (go) return;
			if (!(L.t < L.t_limit)) { L.phase = LANE_PROBE; return; }
			// a step the short form does not cover
			count_advance(L, A, calc_dt(P, L.t, P.cone_angle_constant));
			if (L.phase != LANE_IDLE) L.phase = L.t < L.t_limit ? LANE_STEP : LANE_PROBE;
			return;
		}
	}
	for (uint32_t k = 0; k < K; ++k) {
		count_advance(L, A, calc_dt(P, L.t, P.cone_angle_constant));
		if (L.phase == LANE_IDLE) return;
		if (!(L.t < L.t_limit)) { L.phase = LANE_PROBE; return; }
	}
}

// ------------------------------------------------------------------------------------
// The wide march: one ray, WIDE_STEPS steps per round.  The step sizes do not depend on what the
// grid holds (occupancy_sampler.cu:629-632: t += dt whatever the cell), so the chain of t can run
// ahead (wide_chain, one lane), the WIDE_STEPS positions are then looked up side by side
// (wide_probe, one lane each) and wide_apply replays the loop's bookkeeping over the results in
// step order: the same ray state as WIDE_STEPS calls of count_probe, without the empty-space table.
// ------------------------------------------------------------------------------------
constexpr uint32_t WIDE_STEPS = 64;
SRF_HD uint64_t low_bits64(uint32_t n) { return n >= 64u ? ~0ull : (1ull << n) - 1ull; }

// t[k] = t before step k (k = 0..WIDE_STEPS); returns the mask of steps of size zero
SRF_HD uint64_t wide_chain(const Params& P, float t0, float* t) {
	const ShortForm f = disparity_short_form(P);
	if (f.usable && t0 >= f.t_lo) {
		// the whole batch in the short form, checked afterwards; inside the short form's range every step is positive
		ShortChain ch = short_chain_at(t0);
#if defined(__HIP_DEVICE_COMPILE__)
		#pragma unroll 8
#endif
		for (uint32_t k = 0; k < WIDE_STEPS; ++k) {
			t[k] = ch.t;
			ch = short_chain_next(f, ch);
		}
		t[WIDE_STEPS] = ch.t;
		// t grows until, past the range, the chain runs through infinity; from there on it is negative for good: a last start
		// that is positive and inside the range says that all of them were
		if (t[WIDE_STEPS - 1] >= f.t_lo && t[WIDE_STEPS - 1] <= f.t_hi) return 0ull;
	}
	uint64_t zero = 0;
	float tk = t0;
	for (uint32_t k = 0; k < WIDE_STEPS; ++k) {
		t[k] = tk;
		const float dt = calc_dt(P, tk, P.cone_angle_constant);
		zero |= dt == 0.f ? 1ull << k : 0ull;
		tk += dt;
	}
	t[WIDE_STEPS] = tk;
	return zero;
}

// the lookup of one position in two halves, so that other work can run while the occupancy byte is on its way
struct WideLookup { uint32_t byte, bit; bool inside; };
template <bool SPHERE = true>
SRF_HD WideLookup wide_lookup(const Params& P, const CountArgs& A, Vec3 o, Vec3 d, float t) {
	WideLookup q;
	const Vec3 pos = along(o, d, t);
	q.inside = aabb_contains(P, pos);
	q.byte = 0xffu; q.bit = 0u;
	if (SPHERE && q.inside && P.sphere[3] > 0.f) {
		float t_enter;
		const SphereGate g = sphere_gate(P, o, d, t, &t_enter);
		if (g == SPHERE_BEYOND) q.inside = false;
		if (g == SPHERE_BEFORE) { q.byte = 0u; return q; }
	}
	if (q.inside && P.use_grid) {
		const Probe s = probe_at(P, nullptr, pos, t, P.cone_angle_constant);   // the cell only
		q.bit = s.idx & 7u;
		q.byte = A.bitfield[(s.idx >> 3) + ((P.n_cells * s.level) >> 3)];
	}
	return q;
}
// bit 0: the position is inside the box; bit 1: its cell is occupied
SRF_HD uint32_t wide_flags(const WideLookup& q) { return !q.inside ? 0u : (((q.byte >> q.bit) & 1u) ? 3u : 1u); }
SRF_HD uint32_t wide_probe(const Params& P, const CountArgs& A, Vec3 o, Vec3 d, float t) { return wide_flags(wide_lookup(P, A, o, d, t)); }

SRF_HD void wide_apply(CountLane& L, const Params& P, const CountArgs& A, const float* t, uint64_t m_inside, uint64_t m_occ, uint64_t m_zero) {
	// the loop runs while the position is inside the box and the sample count is below the cap (occupancy_sampler.cu:595-597)
	uint32_t n = ~m_inside ? (uint32_t)__builtin_ctzll(~m_inside) : WIDE_STEPS;
	bool ended = n < WIDE_STEPS;
	const uint32_t allowed = L.j < P.n_max_steps ? P.n_max_steps - L.j : 0u;
	if (!allowed) { n = 0; ended = true; }
	else if ((uint32_t)__builtin_popcountll(m_occ & low_bits64(n)) >= allowed) {
		// the allowed-th sample fills the ray: the step after it is not taken
		uint64_t m = m_occ & low_bits64(n);
		for (uint32_t a = 1; a < allowed; ++a) m &= m - 1ull;
		const uint32_t last = (uint32_t)__builtin_ctzll(m) + 1u;
		if (last < WIDE_STEPS) { n = last; ended = true; }
	}
	// a step of size zero is taken and ends the march (count_advance)
	const uint64_t z = m_zero & low_bits64(n);
	if (z) { n = (uint32_t)__builtin_ctzll(z) + 1u; ended = true; }
	uint64_t rest = m_occ & low_bits64(n);
	L.j += (uint32_t)__builtin_popcountll(rest);
	// samples into the step log, one aligned 32-step word at a time
	while (rest) {
		const uint32_t k = (uint32_t)__builtin_ctzll(rest);
		const uint32_t w = (L.step + k) >> 5;
		const uint32_t k_end = ((w + 1u) << 5) - L.step;          // first step of the batch beyond word w
		const uint64_t in_word = rest & low_bits64(k_end);
		if (w != L.cur_w) {
			step_log_flush(A.log, L.i, L.cur_w, L.word, L.t_word, L.logged, L.mask);
			L.word = 0;
			L.cur_w = w;
		}
		if (!L.word) L.t_word = t[k];
		L.word |= (uint32_t)(in_word >> k) << ((L.step + k) & 31u);
		rest &= ~in_word;
	}
	L.step += n;
	L.t = L.t_limit = t[n];
	if (ended) count_finish(L, A);
}

// one parked ray from where it stopped to its end, the lanes' work done one after the other
SRF_HD void wide_march_serial(const ParkedRay& r, const Params& P, const CountArgs& A) {
	CountLane L;
	count_unpark(L, r);
	float t[WIDE_STEPS + 1];
	while (L.phase != LANE_IDLE) {
		const uint64_t m_zero = wide_chain(P, L.t, t);
		uint64_t m_inside = 0, m_occ = 0;
		for (uint32_t k = 0; k < WIDE_STEPS; ++k) {
			const uint32_t f = wide_probe(P, A, L.o, L.d, t[k]);
			m_inside |= (uint64_t)(f & 1u) << k;
			m_occ |= (uint64_t)(f >> 1) << k;
		}
		wide_apply(L, P, A, t, m_inside, m_occ, m_zero);
	}
}

// ------------------------------------------------------------------------------------
// occupancy_sampler.cu:552-637 — ray set-up and the counting march of one training ray, start to end
// ------------------------------------------------------------------------------------
SRF_HD void train_count_body(uint32_t i, const Params& P, const CountArgs& A) {
	CountLane L;
	L.phase = LANE_IDLE;
	count_begin(L, i, P, A);
	while (L.phase != LANE_IDLE) {
		if (L.phase == LANE_PROBE) count_probe(L, P, A);
		else count_steps<8>(L, P, A);
	}
}

// occupancy_sampler.cu:634-642 — a ray is kept when it has samples and they fit under n_coords
SRF_HD uint32_t train_keep_flag(uint32_t count, uint32_t base, uint32_t n_coords) {
	return (count != 0u && !(base + count > n_coords)) ? 1u : 0u;
}

// where the per-sample side outputs (t, dt, cell) of the writing march go
struct DirectSink {
	float* sample_t; float* sample_dt; uint32_t* sample_cell;
	SRF_HD void put(size_t k, float t, float dt, uint32_t cell) const {
		if (sample_t) sample_t[k] = t;
		if (sample_dt) sample_dt[k] = dt;
		if (sample_cell) sample_cell[k] = cell;
	}
};
constexpr uint32_t WINDOW_EMPTY = 0xffffffffu;   // mark of a staging slot that no ray has written

// occupancy_sampler.cu:644-688 — second march of a kept ray, writing its samples.  In pieces, so that a wavefront can
// spread the per-sample work of its rays evenly over its lanes: the ray's own outputs, the replay of the step log
// (which only finds the t of every sample), what is computed and stored per sample, and the march that looks the
// grid up again for rays without a log.
struct WriteRay { Vec3 o, d, wdir; uint32_t numsteps, base; float startt; };

// occupancy_sampler.cu:644-664 — ray, target colour and sample range of kept ray i
SRF_HD WriteRay train_write_ray(uint32_t i, const DatasetArgs& ds, const TrainRay& st, const uint32_t* counts, const uint32_t* base, const uint32_t* ray_index,
                                float* rays_out, float* rays_rgba, uint32_t* numsteps_out) {
	WriteRay R;
	R.numsteps = counts[i]; R.base = base[i]; R.startt = st.startt;
	const uint32_t r = ray_index[i];
	R.o = ld3(st.o); R.d = ld3(st.d);
	st3(rays_out + 6 * (size_t)r, R.o);
	st3(rays_out + 6 * (size_t)r + 3, R.d);
	Float4 target = mk4(0.f, 0.f, 0.f, 0.f);
	if (ds.images) {
		const uint16_t* px = ds.images + pixel_index(st.xy, ds.res, st.img) * 4;
		target = mk4(half_bits_to_float(px[0]), half_bits_to_float(px[1]), half_bits_to_float(px[2]), half_bits_to_float(px[3]));
	}
	*(Float4*)(rays_rgba + 4 * (size_t)r) = target;
	numsteps_out[2 * (size_t)r + 0] = R.numsteps;
	numsteps_out[2 * (size_t)r + 1] = R.base;
	R.wdir = warp_direction(R.d);
	return R;
}

// the t chain inside the logged runs only; emit(j, t) for sample j of the ray, in order, until it returns false
template <class Emit>
SRF_HD void train_write_replay(uint32_t i, const Params& P, const TrainRay& st, uint32_t cap, const StepLog& log, const Emit& emit) {
	const float cone = P.cone_angle_constant;
	const ShortForm f = disparity_short_form(P);
	uint32_t j = 0;
#if defined(__HIP_DEVICE_COMPILE__)
	#pragma unroll
#endif
	for (uint32_t g = 0; g < 3; ++g) {      // unrolled: the mask words stay in registers
		uint32_t m = st.word_mask[g];
		// a word's bits and the t at its first sample are requested while the word before it is walked
		uint32_t next_bits = 0u;
		float next_t = 0.f;
		if (m) {
			const uint32_t w = g * 32u + (uint32_t)__builtin_ctz(m);
			next_bits = log.bits[(size_t)w * log.stride + i];
			next_t = log.t0[(size_t)w * log.stride + i];
		}
		while (m) {
			m &= m - 1u;
			uint32_t word = next_bits;
			float t = next_t;
			if (m) {
				const uint32_t w = g * 32u + (uint32_t)__builtin_ctz(m);
				next_bits = log.bits[(size_t)w * log.stride + i];
				next_t = log.t0[(size_t)w * log.stride + i];
			}
			word >>= (uint32_t)__builtin_ctz(word);
			const bool short_form = f.usable && t >= f.t_lo;   // t only grows; the upper end is checked per step
			ShortChain ch = short_chain_at(short_form ? t : 1.f);
			while (word && j < cap) {
				if (word & 1u) {
					if (!emit(j, t)) return;
					++j;
				}
				word >>= 1;
				if (short_form && t <= f.t_hi) { ch = short_chain_next(f, ch); t = ch.t; }
				else t += calc_dt(P, t, cone);      // beyond the short form's range for good: t only grows
			}
		}
	}
}

// occupancy_sampler.cu:665-683 — what a sample at t stores: warped position, step, warped direction, and the side outputs
SRF_HD void train_write_sample(const Params& P, Vec3 o, Vec3 d, Vec3 wdir, float t, size_t k, float* coords_out, const DirectSink& out) {
	const float cone = P.cone_angle_constant;
	const float dt = calc_dt(P, t, cone);
	const Probe s = probe_at(P, nullptr, along(o, d, t), t, cone);
	if (coords_out) {
		float* c = coords_out + 7 * k;
		st3(c, s.w); c[3] = dt; st3(c + 4, wdir);
	}
	out.put(k, t, dt, s.idx + s.level * P.n_cells);
}

// a ray without a usable log: the march of the first pass again, lookups included
SRF_HD void train_write_march(const Params& P, const uint8_t* bitfield, const WriteRay& R, uint32_t cap, float* coords_out, const DirectSink& out) {
	const float cone = P.cone_angle_constant;
	uint32_t j = 0;
	float t = R.startt;
	for (;;) {
		const Vec3 pos = along(R.o, R.d, t);
		if (!(aabb_contains(P, pos) && j < cap)) break;
		if (P.sphere[3] > 0.f) {
			float t_enter;
			const SphereGate g = sphere_gate(P, R.o, R.d, t, &t_enter);
			if (g == SPHERE_BEYOND) break;
			if (g == SPHERE_BEFORE) {
				const float dt = calc_dt(P, t, cone);
				t += dt;
				if (dt == 0.f) break;
				continue;
			}
		}
		const Probe s = probe_at(P, P.use_grid ? bitfield : nullptr, pos, t, cone);
		if (s.occ) {
			const size_t k = (size_t)R.base + j;
			if (coords_out) {
				float* c = coords_out + 7 * k;
				st3(c, s.w); c[3] = s.dt; st3(c + 4, R.wdir);
			}
			out.put(k, t, s.dt, s.idx + s.level * P.n_cells);
			++j;
		}
		t += s.dt;
		if (s.dt == 0.f) break;
	}
}

SRF_HD uint32_t train_write_cap(const Params& P, uint32_t numsteps) { return P.use_grid ? numsteps : P.n_max_steps; }

// one ray, start to end
SRF_HD void train_write_body(uint32_t i, const Params& P, const DatasetArgs& ds, const uint8_t* bitfield,
                             const TrainRay* state, const uint32_t* counts, const uint32_t* base, const uint32_t* keep, const uint32_t* ray_index,
                             float* rays_out, float* rays_rgba, uint32_t* numsteps_out,
                             float* coords_out, const DirectSink& sink, StepLog log) {
	if (!keep[i]) return;
	const TrainRay st = state[i];
	const WriteRay R = train_write_ray(i, ds, st, counts, base, ray_index, rays_out, rays_rgba, numsteps_out);
	const uint32_t cap = train_write_cap(P, R.numsteps);
	if (log.bits && st.logged) {
		train_write_replay(i, P, st, cap, log, [&](uint32_t j, float t) {
			train_write_sample(P, R.o, R.d, R.wdir, t, (size_t)R.base + j, coords_out, sink);
			return true;
		});
		return;
	}
	train_write_march(P, bitfield, R, cap, coords_out, sink);
}

// ------------------------------------------------------------------------------------
// occupancy_sampler.cu:691-736 — the payload of pixel (x, y)
// ------------------------------------------------------------------------------------
struct PixelArgs { int32_t res[2]; float focal[2]; float pp[2]; Camera cam; float offset[2]; };

SRF_HD void pixel_ray(const PixelArgs& A, uint32_t x, uint32_t y, Vec3* o, Vec3* d) {
	const float u = ((float)(int32_t)x + A.offset[0]) / (float)A.res[0], v = ((float)(int32_t)y + A.offset[1]) / (float)A.res[1];
	ray_through(A.cam.m, u, v, A.res, A.focal, A.pp, o, d);
}

SRF_HD void init_ray_body(uint32_t x, uint32_t y, const Params& P, const PixelArgs& A, srf_ray_payload* payloads) {
	Vec3 o, d;
	pixel_ray(A, x, y, &o, &d);
	const uint32_t idx = x + (uint32_t)A.res[0] * y;
	srf_ray_payload& pl = payloads[idx];
	float tmin, tmax;
	aabb_ray_intersect(P, o, d, &tmin, &tmax);
	const float t = srf_max(tmin, 0.05f) + 1e-6f;
	if (aabb_contains(P, mk3(o.x + d.x * t, o.y + d.y * t, o.z + d.z * t))) {
		st3(pl.o, o); st3(pl.d, d);
		pl.t = t; pl.idx = idx; pl.n_steps = 0; pl.alive = 1;
	} else {
		st3(pl.o, o);
		pl.alive = 0;
	}
}

// ------------------------------------------------------------------------------------
// The march the three render kernels share, as a lane state machine like the counting march above.  A probe looks the
// cell at t up and, for an empty one, asks the empty-space table how far nothing can be found; steps then walk t through
// that stretch without lookups (the reference would probe each, find nothing and add its dt,
// occupancy_sampler.cu:762-790, :820-850).  What an occupied cell means is the caller's: hit(L, s) says how the march
// goes on.  A wavefront runs its lanes' phases by majority (srf_march.hip); one lane alone runs them in turn.
// ------------------------------------------------------------------------------------
enum MarchEnd : uint32_t { MARCH_GOES_ON = 0, MARCH_LEFT_BOX = 1, MARCH_ZERO_STEP = 2, MARCH_STOPPED = 3, MARCH_NO_RAY = 4 };
// crawl: how many probes in a row found an empty cell and nothing to skip (the ray runs through occupied surroundings and looks a
// cell up at every step); the last few rays of a wavefront that crawl are handed to the one-ray-per-wavefront march (srf_march.hip)
struct MarchLane { uint32_t phase, crawl; Vec3 o, d; float t, t_limit; SkipRay sr; };

SRF_HD void march_start(MarchLane& L, Vec3 o, Vec3 d, float t, bool skipping) {
	L.o = o; L.d = d;
	L.t = L.t_limit = t;
	L.crawl = 0;
	if (skipping) L.sr = skip_ray_setup(o, d);
	L.phase = LANE_PROBE;
}

template <class Hit>
SRF_HD MarchEnd march_probe(MarchLane& L, const Params& P, const uint8_t* bitfield, const SkipTable& skip, bool skipping, const Hit& hit) {
	const float cone = P.cone_angle_constant;
	const Vec3 pos = along(L.o, L.d, L.t);
	if (!aabb_contains(P, pos)) return MARCH_LEFT_BOX;
	if (P.sphere[3] > 0.f) {      // optional sphere bound: no sample outside it, the chain of t as it is
		float t_enter;
		const SphereGate g = sphere_gate(P, L.o, L.d, L.t, &t_enter);
		if (g == SPHERE_BEYOND) return MARCH_LEFT_BOX;
		if (g == SPHERE_BEFORE) {
			const float dt = calc_dt(P, L.t, cone);
			L.t_limit = t_enter;
			L.t += dt;
			if (dt == 0.f) return MARCH_ZERO_STEP;
			L.phase = L.t < L.t_limit ? LANE_STEP : LANE_PROBE;
			return MARCH_GOES_ON;
		}
	}
	SRF_COUNT_PROBE();
	const Probe s = probe_at(P, bitfield, pos, L.t, cone, &skip);
	L.t_limit = L.t;      // steps at t' < t_limit are known to find an empty cell
	const uint32_t crawled = L.crawl;
	L.crawl = 0;
	if (s.occ) return hit(L, s);
	if (skipping) L.t_limit = skip_limit(P, skip, L.sr, L.o, L.d, L.t, s.radius, s.level);
	L.t += s.dt;
	if (s.dt == 0.f) return MARCH_ZERO_STEP;
	L.phase = L.t < L.t_limit ? LANE_STEP : LANE_PROBE;
	L.crawl = L.phase == LANE_PROBE ? crawled + 1u : 0u;
	return MARCH_GOES_ON;
}

// the steps below t_limit, each lane for itself; the step sizes are count_steps's (the short form of the disparity chain
// where it holds, calc_dt elsewhere), and a step of size zero ends the march.  The plain loop that lanes leave one by one
// (seven vector instructions a step) beats predicated bursts of a fixed length here, where all lanes step before any probes.
//
// Half of the way the chain is plainer still.  For a float g whose mantissa is below sqrt 2, the reciprocal of its reciprocal
// (both correctly rounded) is g itself: RN(1/g) is off by at most half an ulp of a number with mantissa 2/m, which moves its
// reciprocal by less than half an ulp of g when m^2 < 2 (every such mantissa checked: tests/test_disparity_chain.py).  While
// g = c + 1/t stays in that lower part [2^e, sqrt 2 * 2^e) of one binade, the reciprocal the chain carries is therefore g, a
// step is one addition, and t = RN(1/g) is only needed when the stretch ends.  "t < lim" becomes "r > G" with a margin of
// 2^-21 (r > G implies RN(1/r) < lim; what the margin leaves is taken by the chained form, which gives the same values).  As
// g falls, the upper part of a binade (chained steps) and its lower part (additions) take turns, a few hundred steps each.
constexpr uint32_t MARCH_PLAIN_MIN_STEPS = 24;
SRF_HD MarchEnd march_steps(MarchLane& L, const Params& P) {
	const float cone = P.cone_angle_constant;
	const ShortForm f = disparity_short_form(P);
	if (f.usable && L.t >= f.t_lo) {
		const float lim = srf_min(L.t_limit, f.t_hi);
		ShortChain ch = short_chain_at(L.t);
		const float G = srf_approx_rcp(lim) * 1.000001f;      // 1 + 2^-20: the estimate's ulp, the product's rounding and an ulp between t and RN(1/r)
		// a stretch of a few steps is not worth telling the two forms apart: (r - G) / -c estimates its length
		if (!(ch.r - G > -(float)MARCH_PLAIN_MIN_STEPS * f.c)) {
			while (ch.t < lim) ch = short_chain_next(f, ch);
		} else if (ch.t < lim) {
			do {
				const float g1 = f.c + ch.r;
				const float bin = srf_u2f(srf_f2u(g1) & 0x7f800000u);      // 2^e <= g1
				if (g1 > 0.f && g1 < bin * 1.4142134f) {
					// additions while the step still lands at or above 2^e (r > 2^e - c, rounded up) and t is still below lim
					const float S = srf_max(G, (bin - f.c) * 1.0000002f);
					float r = ch.r;
					if (r > S) {
						if (!short_chain_jump(f.c, bin, S, r)) do r = f.c + r; while (r > S);
						ch.r = r;
						ch.t = srf_rcp_normal(r);
					} else {
						ch = short_chain_next(f, ch);      // at the end of the stretch or of the binade's lower part
					}
				} else {
					// chained steps up to where g enters the lower part of its binade: g < sqrt 2 * 2^e, t > 1 / (sqrt 2 * 2^e)
					const float lim_c = srf_min(lim, srf_approx_rcp(bin * 1.4142134f) * 1.000001f);
					do ch = short_chain_next(f, ch); while (ch.t < lim_c);
				}
			} while (ch.t < lim);
		}
		L.t = ch.t;
	}
	while (L.t < L.t_limit) {      // what the short form does not cover
		const float dt = calc_dt(P, L.t, cone);
		L.t += dt;
		if (dt == 0.f) return MARCH_ZERO_STEP;
	}
	L.phase = LANE_PROBE;
	return MARCH_GOES_ON;
}

// what the render marches are given besides the ray
struct MarchGrid {
	Params P; const uint8_t* bitfield; SkipTable skip;
	SRF_HD bool skipping() const { return skip.dist != nullptr && bitfield != nullptr; }
};

// occupancy_sampler.cu:738-797 — jitter the start, then step to the first occupied cell
struct AdvanceMarch {
	MarchGrid G; uint32_t n_rays, spp; srf_ray_payload* payloads;
	struct Lane { MarchLane m; uint32_t i; };
	struct Hit { SRF_HD MarchEnd operator()(MarchLane&, const Probe&) const { return MARCH_STOPPED; } };
	SRF_HD uint32_t lanes() const { return n_rays; }
	SRF_HD void finish(Lane& L, MarchEnd end) const {
		srf_ray_payload& pl = payloads[L.i];
		pl.t = L.m.t;
		if (end != MARCH_STOPPED) pl.alive = 0;
		L.m.phase = LANE_IDLE;
	}
	SRF_HD MarchEnd begin(Lane& L, uint32_t i) const {
		L.i = i;
		L.m.phase = LANE_IDLE;
		const srf_ray_payload& pl = payloads[i];
		if (!pl.alive) return MARCH_NO_RAY;
		float t = pl.t;
		t += ld_random_val01(spp, i * 786433u, 0) * calc_dt(G.P, t, G.P.cone_angle_constant);
		march_start(L.m, ld3(pl.o), ld3(pl.d), t, G.skipping());
		return MARCH_GOES_ON;
	}
	SRF_HD MarchEnd probe(Lane& L) const { return march_probe(L.m, G.P, G.bitfield, G.skip, G.skipping(), Hit()); }
	SRF_HD MarchEnd steps(Lane& L) const { return march_steps(L.m, G.P); }
};

// occupancy_sampler.cu:799-863 — next n_steps occupied samples of a live ray.  A ray that leaves the box or ends on a
// zero step before that keeps its old t and records how many samples it got; an occupied sample's own step is taken
// whatever its size.
struct CoordsMarch {
	MarchGrid G; uint32_t n_rays, n_steps; srf_ray_payload* payloads; float* coords;
	const uint32_t* round = nullptr;      // device words {rays, steps} that replace n_rays and n_steps when the kernel starts (the frame loop paced by the device)
	struct Lane { MarchLane m; uint32_t i, j; Vec3 wdir; };
	struct Hit {
		float* c; uint32_t* j; uint32_t n_steps; Vec3 wdir;
		SRF_HD MarchEnd operator()(MarchLane& L, const Probe& s) const {
			float* q = c + 7 * (size_t)*j;
			st3(q, s.w); q[3] = s.dt; st3(q + 4, wdir);
			++*j;
			L.t += s.dt;
			if (*j == n_steps) return MARCH_STOPPED;
			L.phase = LANE_PROBE;
			return MARCH_GOES_ON;
		}
	};
	SRF_HD uint32_t lanes() const { return n_rays; }
	SRF_HD void finish(Lane& L, MarchEnd end) const {
		srf_ray_payload& pl = payloads[L.i];
		if (end == MARCH_STOPPED) { pl.t = L.m.t; pl.n_steps = n_steps; }
		else pl.n_steps = L.j;
		L.m.phase = LANE_IDLE;
	}
	SRF_HD MarchEnd begin(Lane& L, uint32_t i) const {
		L.i = i; L.j = 0;
		L.m.phase = LANE_IDLE;
		const srf_ray_payload& pl = payloads[i];
		if (!pl.alive) return MARCH_NO_RAY;
		const Vec3 d = ld3(pl.d);
		L.wdir = warp_direction(d);
		march_start(L.m, ld3(pl.o), d, pl.t, G.skipping());
		return n_steps == 0 ? MARCH_STOPPED : MARCH_GOES_ON;
	}
	SRF_HD MarchEnd probe(Lane& L) const {
		Hit hit; hit.c = coords + 7 * (size_t)L.i * n_steps; hit.j = &L.j; hit.n_steps = n_steps; hit.wdir = L.wdir;
		return march_probe(L.m, G.P, G.bitfield, G.skip, G.skipping(), hit);
	}
	SRF_HD MarchEnd steps(Lane& L) const { return march_steps(L.m, G.P); }
};

// one ray from begin to finish, the phases in turn
template <class March>
SRF_HD void march_alone(const March& M, uint32_t i) {
	typename March::Lane L;
	MarchEnd end = M.begin(L, i);
	while (end == MARCH_GOES_ON) end = L.m.phase == LANE_PROBE ? M.probe(L) : M.steps(L);
	if (end != MARCH_NO_RAY) M.finish(L, end);
}

SRF_HD void advance_pos_body(uint32_t i, const Params& P, uint32_t spp, srf_ray_payload* payloads, const uint8_t* bitfield, SkipTable skip) {
	AdvanceMarch M;
	M.G.P = P; M.G.bitfield = bitfield; M.G.skip = skip; M.n_rays = i + 1; M.spp = spp; M.payloads = payloads;
	march_alone(M, i);
}

SRF_HD void generate_coords_body(uint32_t i, const Params& P, uint32_t n_steps, const uint8_t* bitfield, srf_ray_payload* payloads, float* coords, SkipTable skip) {
	CoordsMarch M;
	M.G.P = P; M.G.bitfield = bitfield; M.G.skip = skip; M.n_rays = i + 1; M.n_steps = n_steps; M.payloads = payloads; M.coords = coords;
	march_alone(M, i);
}

// ------------------------------------------------------------------------------------
// Table-lookup stand-in for the network: the sample's cascade cell, recomputed from
// its warped position, selects a row of (r, g, b, sigma).  Not in the reference.
// ------------------------------------------------------------------------------------
struct FieldArgs { const float* table; uint32_t mask; uint32_t seed; };

SRF_HD uint32_t field_row(const Params& P, Vec3 w, const FieldArgs& F) {
	const uint32_t level = level_from_pos(P, w, w);
	const uint32_t cell = cascaded_grid_idx_at(P, w, w, level) + level * P.n_cells;
	return mix32(cell ^ F.seed) & F.mask;
}

template <bool HALF>
SRF_HD void field_eval_body(uint32_t i, const Params& P, const float* coords, const FieldArgs& F, void* out, uint32_t width) {
	const Vec3 w = ld3(coords + 7 * (size_t)i);
	const Float4 row = *(const Float4*)(F.table + 4 * (size_t)field_row(P, w, F));
	net_store<HALF>(out, (size_t)i * width + 0, row.x);
	net_store<HALF>(out, (size_t)i * width + 1, row.y);
	net_store<HALF>(out, (size_t)i * width + 2, row.z);
	net_store<HALF>(out, (size_t)i * width + 3, row.w);
}

// Whole-frame render: the ray of a pixel is generated, advanced and marched to the
// end, compositing every occupied sample as volume_rendering_kernel does
// (ray_marcher.cu:233-273) and finishing with shade_kernel's store (testbed.cu:448-477)
// into a frame buffer that starts from zero.  An occupied sample whose step size is
// zero (t at the far plane, still inside the box) makes the reference's loop re-emit it
// with zero weight until MARCH_ITER runs out (testbed.cu:523) and the still-alive ray is
// never shaded; the pixel is left at zero here as well.
// Lanes are numbered so that the 64 of a wavefront cover an 8 x 8 tile of pixels: neighbours in both directions take
// similar paths through the grid.
struct FusedMarch {
	MarchGrid G; PixelArgs A; FieldArgs F; uint32_t spp; float thr; int to_linear; float* frame; uint32_t* n_samples;
	struct Lane { MarchLane m; uint32_t idx, count; Float4 acc; };
	struct Hit {
		const Params* P; const FieldArgs* F; float thr; Float4* acc; uint32_t* count;
		SRF_HD MarchEnd operator()(MarchLane& L, const Probe& s) const {
			if (s.dt == 0.f) { *acc = mk4(0.f, 0.f, 0.f, 0.f); return MARCH_STOPPED; }
			const Float4 row = *(const Float4*)(F->table + 4 * (size_t)field_row(*P, s.w, *F));
			const float T = 1.f - acc->w;
			const float alpha = 1.f - srf_expf(-row.w * s.dt);
			const float weight = alpha * T;
			acc->x += row.x * weight; acc->y += row.y * weight; acc->z += row.z * weight;
			acc->w += weight;
			++*count;
			if (acc->w > (1.0f - thr)) return MARCH_STOPPED;
			L.t += s.dt;
			L.phase = LANE_PROBE;
			return MARCH_GOES_ON;
		}
	};
	SRF_HD uint32_t tiles_x() const { return ((uint32_t)A.res[0] + 7u) >> 3; }
	SRF_HD uint32_t lanes() const { return tiles_x() * (((uint32_t)A.res[1] + 7u) >> 3) * 64u; }
	SRF_HD void finish(Lane& L, MarchEnd) const {
		Float4 out = mk4(0.f, 0.f, 0.f, 0.f);
		if (L.acc.w > 0.001f) {
			out = L.acc;
			if (to_linear) { out.x = srgb_to_linear(out.x); out.y = srgb_to_linear(out.y); out.z = srgb_to_linear(out.z); }
		}
		*(Float4*)(frame + 4 * (size_t)L.idx) = out;
		if (n_samples) n_samples[L.idx] = L.count;
		L.m.phase = LANE_IDLE;
	}
	SRF_HD MarchEnd begin_pixel(Lane& L, uint32_t x, uint32_t y) const {
		L.idx = x + (uint32_t)A.res[0] * y;
		L.count = 0;
		L.acc = mk4(0.f, 0.f, 0.f, 0.f);
		Vec3 o, d;
		pixel_ray(A, x, y, &o, &d);
		float tmin, tmax;
		aabb_ray_intersect(G.P, o, d, &tmin, &tmax);
		float t = srf_max(tmin, 0.05f) + 1e-6f;
		if (!aabb_contains(G.P, mk3(o.x + d.x * t, o.y + d.y * t, o.z + d.z * t))) return MARCH_LEFT_BOX;
		t += ld_random_val01(spp, L.idx * 786433u, 0) * calc_dt(G.P, t, G.P.cone_angle_constant);
		march_start(L.m, o, d, t, G.skipping());
		return MARCH_GOES_ON;
	}
	SRF_HD MarchEnd begin(Lane& L, uint32_t q) const {
		const uint32_t tile = q >> 6, tx = tiles_x();
		const uint32_t x = (tile % tx) * 8u + (q & 7u), y = (tile / tx) * 8u + ((q >> 3) & 7u);
		L.m.phase = LANE_IDLE;
		return x < (uint32_t)A.res[0] && y < (uint32_t)A.res[1] ? begin_pixel(L, x, y) : MARCH_NO_RAY;
	}
	SRF_HD MarchEnd probe(Lane& L) const {
		Hit hit; hit.P = &G.P; hit.F = &F; hit.thr = thr; hit.acc = &L.acc; hit.count = &L.count;
		return march_probe(L.m, G.P, G.bitfield, G.skip, G.skipping(), hit);
	}
	SRF_HD MarchEnd steps(Lane& L) const { return march_steps(L.m, G.P); }
};

SRF_HD void render_fused_body(uint32_t idx, const Params& P, const PixelArgs& A, uint32_t spp, const uint8_t* bitfield, const FieldArgs& F,
                              float transmittance_threshold, int to_linear, float* frame, uint32_t* n_samples, SkipTable skip) {
	FusedMarch M;
	M.G.P = P; M.G.bitfield = bitfield; M.G.skip = skip; M.A = A; M.F = F; M.spp = spp; M.thr = transmittance_threshold;
	M.to_linear = to_linear; M.frame = frame; M.n_samples = n_samples;
	FusedMarch::Lane L;
	L.m.phase = LANE_IDLE;
	MarchEnd end = M.begin_pixel(L, idx % (uint32_t)A.res[0], idx / (uint32_t)A.res[0]);
	while (end == MARCH_GOES_ON) end = L.m.phase == LANE_PROBE ? M.probe(L) : M.steps(L);
	M.finish(L, end);
}

// ------------------------------------------------------------------------------------
// ray_marcher.cu:9-202 — training compositing, split at the compaction atomic
// ------------------------------------------------------------------------------------
struct LossConst {
	uint32_t n_rays;
	uint32_t n_max_compacted;
	uint32_t out_width;
	int32_t  rgb_act, density_act, loss_type;
	float    loss_scale;               // already divided by n_rays
	float    min_optical_thickness;
	int32_t  use_grid;
	float    bg_in[3];                 // background before srgb_to_linear (the shared random draw already applied)
	float    bg_lin[3];                // srgb_to_linear(bg_in): the same for every ray of a call, so worked out once (loss_const_background)
	float    bg_enc[3];                // linear_to_srgb(bg_lin)
	int32_t  color_space;
	int32_t  train_in_linear;
	float    thr;
	uint32_t dt_stride;
};

// per-ray results of the forward pass kept for the backward pass
struct FwdRay {
	float rgb_ray[3];
	float target[3];
	uint32_t numsteps, base;
};

// ray_marcher.cu:85-86, :94, :100 — the two encodings of the background colour that every ray of a call uses; after bg_in is set
SRF_HD void loss_const_background(LossConst& K) {
	for (int c = 0; c < 3; ++c) { K.bg_lin[c] = srgb_to_linear(K.bg_in[c]); K.bg_enc[c] = linear_to_srgb(K.bg_lin[c]); }
}

// ray_marcher.cu:85-104 — background and ground-truth colour of a ray
SRF_HD void target_and_background(const LossConst& K, Float4 tex, float target[3], float bg[3]) {
	for (int c = 0; c < 3; ++c) { bg[c] = K.bg_lin[c]; target[c] = 0.f; }
	if (K.train_in_linear || K.color_space == SRF_COLOR_LINEAR) {
		const float k = 1 - tex.w;
		target[0] = tex.x + k * bg[0]; target[1] = tex.y + k * bg[1]; target[2] = tex.z + k * bg[2];
		if (!K.train_in_linear) {
			for (int c = 0; c < 3; ++c) { target[c] = linear_to_srgb(target[c]); bg[c] = K.bg_enc[c]; }
		}
	} else if (K.color_space == SRF_COLOR_SRGB) {
		for (int c = 0; c < 3; ++c) bg[c] = K.bg_enc[c];
		if (tex.w > 0) {
			const float k = 1 - tex.w;
			target[0] = linear_to_srgb(tex.x / tex.w) * tex.w + k * bg[0];
			target[1] = linear_to_srgb(tex.y / tex.w) * tex.w + k * bg[1];
			target[2] = linear_to_srgb(tex.z / tex.w) * tex.w + k * bg[2];
		} else { target[0] = bg[0]; target[1] = bg[1]; target[2] = bg[2]; }
	}
}

// ray_marcher.cu:57-109 — forward compositing with early termination
template <bool HALF_IN>
SRF_HD void loss_forward_body(uint32_t i, const LossConst& K, const float* rays_rgba, uint32_t n_active,
                              const uint32_t* ray_coord_indices, const float* dt_arr, const void* net,
                              FwdRay* fwd_i, uint32_t* n_out_i, float* rgb_ray_out) {
	if (i >= n_active) { *n_out_i = 0; return; }
	FwdRay f;
	f.numsteps = ray_coord_indices[2 * (size_t)i];
	f.base = ray_coord_indices[2 * (size_t)i + 1];
	float T = 1.f;
	float r = 0.f, g = 0.f, b = 0.f;
	uint32_t n = 0;
	for (; n < f.numsteps; ++n) {
		if (T < K.thr) break;
		const size_t s = (size_t)f.base + n;
		const float density = act_density(net_load<HALF_IN>(net, s * 4 + 3), K.density_act);
		const float cr = act_rgb(net_load<HALF_IN>(net, s * 4 + 0), K.rgb_act);
		const float cg = act_rgb(net_load<HALF_IN>(net, s * 4 + 1), K.rgb_act);
		const float cb = act_rgb(net_load<HALF_IN>(net, s * 4 + 2), K.rgb_act);
		const float dt = dt_arr[s * K.dt_stride];
		const float alpha = 1.f - srf_expf(-density * dt);
		const float weight = alpha * T;
		r += weight * cr; g += weight * cg; b += weight * cb;
		T *= (1.f - alpha);
	}
	float target[3], bg[3];
	target_and_background(K, *(const Float4*)(rays_rgba + 4 * (size_t)i), target, bg);
	if (n == f.numsteps) { r += T * bg[0]; g += T * bg[1]; b += T * bg[2]; }
	f.rgb_ray[0] = r; f.rgb_ray[1] = g; f.rgb_ray[2] = b;
	f.target[0] = target[0]; f.target[1] = target[1]; f.target[2] = target[2];
	*fwd_i = f;
	*n_out_i = n;
	if (rgb_ray_out) { rgb_ray_out[3 * (size_t)i] = r; rgb_ray_out[3 * (size_t)i + 1] = g; rgb_ray_out[3 * (size_t)i + 2] = b; }
}

// ray_marcher.cu:116-201 — clamp to the compacted capacity, loss, and the gradient pass
template <bool HALF_IN, bool HALF_OUT>
SRF_HD void loss_backward_body(uint32_t i, const LossConst& K, uint32_t n_active, uint32_t* ray_coord_indices,
                               const float* dt_arr, const float* coords, float* compacted_coords,
                               const void* net, void* dloss, float* loss_output, float mean_density,
                               const FwdRay& f, uint32_t n_fwd_i, uint32_t cbase, float* reg_buffer) {
	if (i >= n_active) return;
	uint32_t n = n_fwd_i;
	const uint32_t room = K.n_max_compacted - (K.n_max_compacted < cbase ? K.n_max_compacted : cbase);
	n = room < n ? room : n;
	ray_coord_indices[2 * (size_t)i] = n;
	ray_coord_indices[2 * (size_t)i + 1] = cbase;
	if (n == 0) return;

	float lo[3], gr[3];
	for (int c = 0; c < 3; ++c) loss_channel(K.loss_type, f.target[c], f.rgb_ray[c], &lo[c], &gr[c]);
	if (loss_output) loss_output[i] = (((lo[0] + lo[1]) + lo[2]) / 3.0f) / (float)K.n_rays;
	const float l2_reg = K.rgb_act == SRF_ACT_EXPONENTIAL ? 1e-4f : 0.0f;
	const float l1_reg_density = (K.use_grid && (mean_density < K.min_optical_thickness)) ? 1e-4f : 0.0f;

	if (reg_buffer) {   // ray_marcher.cu:142-166: T stays 1 throughout this loop in the reference
		float sum_w = 0.f, sum_wp = 0.f;
		float* buf = reg_buffer + (size_t)cbase * 2;
		for (uint32_t j = 0; j < n; ++j) {
			const size_t s = (size_t)f.base + j;
			const float dt = dt_arr[s * K.dt_stride];
			const float density = act_density(net_load<HALF_IN>(net, s * 4 + 3), K.density_act);
			const float alpha = 1.f - srf_expf(-density * dt);
			const float weight = alpha * 1.f;
			sum_w += weight;
			sum_wp += weight * (float)(j + 1) / (float)n;
			buf[2 * j] = sum_w; buf[2 * j + 1] = sum_wp;
		}
	}

	float r2 = 0.f, g2 = 0.f, b2 = 0.f;
	float T = 1.f;
	for (uint32_t j = 0; j < n; ++j) {
		const size_t s = (size_t)f.base + j;
		const size_t o = (size_t)cbase + j;
		if (compacted_coords) {
			for (int c = 0; c < 7; ++c) compacted_coords[7 * o + c] = coords[7 * s + c];
		}
		const float dt = dt_arr[s * K.dt_stride];
		const float raw0 = net_load<HALF_IN>(net, s * 4 + 0), raw1 = net_load<HALF_IN>(net, s * 4 + 1);
		const float raw2 = net_load<HALF_IN>(net, s * 4 + 2), raw3 = net_load<HALF_IN>(net, s * 4 + 3);
		const float cr = act_rgb(raw0, K.rgb_act), cg = act_rgb(raw1, K.rgb_act), cb = act_rgb(raw2, K.rgb_act);
		const float density = act_density(raw3, K.density_act);
		const float alpha = 1.f - srf_expf(-density * dt);
		const float weight = alpha * T;
		r2 += weight * cr; g2 += weight * cg; b2 += weight * cb;
		T *= (1.f - alpha);
		const float d0 = K.loss_scale * ((weight * gr[0]) * act_rgb_derivative(raw0, K.rgb_act) + srf_max_zero(l2_reg * raw0));
		const float d1 = K.loss_scale * ((weight * gr[1]) * act_rgb_derivative(raw1, K.rgb_act) + srf_max_zero(l2_reg * raw1));
		const float d2 = K.loss_scale * ((weight * gr[2]) * act_rgb_derivative(raw2, K.rgb_act) + srf_max_zero(l2_reg * raw2));
		const float sx = f.rgb_ray[0] - r2, sy = f.rgb_ray[1] - g2, sz = f.rgb_ray[2] - b2;
		const float dd = act_density_derivative(raw3, K.density_act);
		const float dotv = (gr[0] * (T * cr - sx) + gr[1] * (T * cg - sy)) + gr[2] * (T * cb - sz);
		const float dmlp = dd * (dt * dotv);
		const float d3 = K.loss_scale * dmlp + (raw3 < 0 ? -l1_reg_density : 0.0f);
		net_store<HALF_OUT>(dloss, o * K.out_width + 0, d0);
		net_store<HALF_OUT>(dloss, o * K.out_width + 1, d1);
		net_store<HALF_OUT>(dloss, o * K.out_width + 2, d2);
		net_store<HALF_OUT>(dloss, o * K.out_width + 3, d3);
	}
}

// ------------------------------------------------------------------------------------
// ray_marcher.cu:204-282 — composite this iteration's chunk of samples into a ray's accumulator
// ------------------------------------------------------------------------------------
template <bool HALF_IN>
SRF_HD void volume_rendering_body(uint32_t i, const Params& P, const srf_render_args& A, float thr, srf_ray_payload* payloads,
                                  float* rgba, const float* coords, const void* net) {
	srf_ray_payload& pl = payloads[i];
	if (!pl.alive) return;
	const Vec3 origin = ld3(pl.o);
	const Vec3 fwd = mk3(A.camera_matrix[6], A.camera_matrix[7], A.camera_matrix[8]);
	Float4 acc = *(const Float4*)(rgba + 4 * (size_t)i);
	const uint32_t n = pl.n_steps;
	uint32_t j = 0;
	for (; j < n; ++j) {
		const size_t s = (size_t)i * A.n_steps + j;
		const Vec3 w = ld3(coords + 7 * s);
		const float dt = coords[7 * s + 3];
		const float raw0 = net_load<HALF_IN>(net, s * A.padded_output_width + 0), raw1 = net_load<HALF_IN>(net, s * A.padded_output_width + 1);
		const float raw2 = net_load<HALF_IN>(net, s * A.padded_output_width + 2), raw3 = net_load<HALF_IN>(net, s * A.padded_output_width + 3);
		const float T = 1.f - acc.w;
		const float alpha = 1.f - srf_expf(-act_density(raw3, A.density_activation) * dt);
		const float weight = alpha * T;
		Vec3 c = mk3(act_rgb(raw0, A.rgb_activation), act_rgb(raw1, A.rgb_activation), act_rgb(raw2, A.rgb_activation));
		if (A.render_mode == SRF_RENDER_NORMALS) {
			c = unit3(scale3(w, -act_density_derivative(raw3, A.density_activation)));
		} else if (A.render_mode == SRF_RENDER_DEPTH) {
			const float z = dot3(fwd, sub3(unwarp_position(P, w), origin)) * A.depth_scale;
			c = mk3(z, z, z);
		} else if (A.render_mode == SRF_RENDER_DISTANCE) {
			const float z = len3(sub3(unwarp_position(P, w), origin)) * A.depth_scale;
			c = mk3(z, z, z);
		} else if (A.render_mode == SRF_RENDER_AO) {
			c = mk3(alpha, alpha, alpha);
		}
		acc.x += c.x * weight; acc.y += c.y * weight; acc.z += c.z * weight;
		acc.w += weight;
		if (acc.w > (1.0f - thr)) break;
	}
	if (j < A.n_steps) {
		pl.alive = 0;
		pl.n_steps = j + A.i_steps_offset;
	}
	*(Float4*)(rgba + 4 * (size_t)i) = acc;
}

// testbed.cu:448-477 — blend a finished ray into its pixel
SRF_HD void shade_body(uint32_t i, const float* rgba, const srf_ray_payload* payloads, float* frame, int render_mode, int train_in_linear) {
	Float4 tmp = *(const Float4*)(rgba + 4 * (size_t)i);
	const srf_ray_payload& pl = payloads[i];
	if (render_mode == SRF_RENDER_NORMALS) {
		const Vec3 nn = unit3(mk3(tmp.x, tmp.y, tmp.z));
		tmp.x = (0.5f * nn.x + 0.5f) * tmp.w; tmp.y = (0.5f * nn.y + 0.5f) * tmp.w; tmp.z = (0.5f * nn.z + 0.5f) * tmp.w;
	} else if (render_mode == SRF_RENDER_COST) {
		const float col = (float)pl.n_steps / 128;
		tmp = mk4(col, col, col, 1.0f);
	}
	if (!train_in_linear && render_mode == SRF_RENDER_SHADE) {
		tmp.x = srgb_to_linear(tmp.x); tmp.y = srgb_to_linear(tmp.y); tmp.z = srgb_to_linear(tmp.z);
	}
	Float4* fb = (Float4*)(frame + 4 * (size_t)pl.idx);
	Float4 old = *fb;
	const float k = 1.0f - tmp.w;
	old.x = tmp.x + old.x * k; old.y = tmp.y + old.y * k; old.z = tmp.z + old.z * k; old.w = tmp.w + old.w * k;
	*fb = old;
}

} // namespace srf
