// Training compositing (forward, loss, ordered compaction, backward), one wavefront per item.
//
// The sample buffer is cut into windows of `stride` consecutive samples; an item is the rays whose first sample
// lies in one window (consecutive rays, because a sampler that assigns offsets in ray order lays rays out back to
// back), and its samples are the range from its first ray's first sample to its last ray's end.  One wavefront
// carries an item through every phase on its own, switching between two lane assignments:
//
//   rows   (lane <-> sample)  coalesced loads of rgb-sigma and dt; alpha = 1 - exp(-sigma dt); {alpha, colour}
//                             of every sample goes to the wavefront's LDS window
//   chain  (lane <-> ray)     the reference's loop over the ray's samples in order: termination test,
//                             weight = alpha * T, colour sums, T *= (1 - alpha).  {T before the sample, colour sums
//                             including it} replace the sample's record, and the sample is marked with its ray
//   finish (lane <-> ray)     background, target, loss and its gradient; the item's number of kept samples is
//                             published and chained to its predecessors' (ordered offsets)
//   grads  (lane <-> sample)  gradients from the exact per-sample T and colour prefix, one 16-byte store per
//                             sample at its compacted position
//
// Only the chain is sequential; every value a gradient depends on is produced by the same operations in the same
// order as a one-thread-per-ray loop, so the results are bit-identical to it.  An item whose range exceeds the LDS
// window runs rows and chain chunk by chunk with the rays' running state carried along, once to learn counts,
// colours and loss gradients and a second time to emit gradients.  An item of more than 64 rays, and every item of
// a call whose rays are not laid out in increasing order, is composited one lane per ray straight from memory.
//
// The phases are host/device functions of (lane, shared state, per-lane state) so that a host build can run an
// item phase by phase in plain loops.
#pragma once
#include "srf_composite_fused.h"

// On the device: tells the compiler nothing about a register's value, so that what is derived from it here is computed
// here (and not kept in registers since an earlier phase derived the same).
#if defined(__HIP_DEVICE_COMPILE__)
#define SRF_OPAQUE_U32(x) asm volatile("" : "+v"(x))
#define SRF_OPAQUE_F32(x) asm volatile("" : "+v"(x))
#else
#define SRF_OPAQUE_U32(x) ((void)0)
#define SRF_OPAQUE_F32(x) ((void)0)
#endif

namespace srf {
namespace wv {

constexpr uint32_t LANES = 64;
constexpr uint32_t ROWS = 16;                  // rows of 64 samples a wavefront holds in registers and LDS
constexpr uint32_t WIN = ROWS * LANES;         // 1024 samples
constexpr uint32_t PAD = 8;                    // records past the window, where the chain's clamped reads and writes land
constexpr uint32_t LAST = WIN + PAD - 1;
constexpr uint32_t STRIDE_FIT = WIN - 2 * LANES;   // widest stride whose items still fit the window when the last ray overhangs by up to 128 samples
constexpr uint32_t STRIDE_MIN = 64;
constexpr uint32_t CHAIN_UNROLL = 4;
constexpr uint32_t GROUP = 64;                 // rays per item of a call whose rays are not laid out in order
constexpr uint32_t ITEMS_PER_TICKET = 4;       // one wavefront each; a workgroup takes this many consecutive items at a time

using G = fused::Geometry<LANES, ROWS, false>;
using fused::Args;
using fused::RayOut;
using fused::SlotState;
using fused::NO_OWNER;

struct RayLds2;
struct Lds {
	Float4 S[WIN + PAD];         // rows: {alpha, r, g, b}; after the chain: {T before the sample, colour sums including it}; in the common item's last phases: the gradients
	uint8_t owner[WIN + PAD];    // lane of the ray whose chain took the sample (NO_OWNER: none)
	alignas(16) unsigned char rays[LANES * 40];   // per ray: loss gradient, composited colour, compacted offset, end of the kept samples (RayOut[LANES], or RayLds2 for the common item)
	SRF_HD RayOut* out() { return (RayOut*)rays; }
	SRF_HD const RayOut* out() const { return (const RayOut*)rays; }
	SRF_HD RayLds2& staged() { return *(RayLds2*)rays; }
};

// items a call of n_rays rays can make at most; the stride is widened until the items fit (window_stride)
SRF_HD constexpr uint32_t max_items(uint32_t n_rays) { return n_rays / 16 + 64; }

// Stride of the sample windows, from what the last active ray's record tells: span = its first sample minus ray 0's,
// end = its end minus ray 0's first sample.  About 50 rays per item; while rays are short enough for whole items to fit
// the LDS window the stride leaves room for the last ray's overhang, beyond that (mean length > 96) items take the
// chunked path whatever the stride, so it keeps growing with the rays.  Any value gives the same results.
SRF_HD uint32_t window_stride(uint32_t n_active, uint64_t span, uint64_t end, uint32_t item_cap) {
	if (n_active == 0) return STRIDE_FIT;
	const uint64_t mean = end / n_active;
	uint64_t w = 50 * mean;
	if (mean <= 96) {
		const uint64_t fit = WIN > 3 * mean + 512 ? WIN - 3 * mean : 512;
		w = w < fit ? w : fit;
		w = w < STRIDE_FIT ? w : STRIDE_FIT;
	}
	const uint64_t need = span / item_cap + 1;       // span / stride + 1 <= item_cap
	w = w > need ? w : need;
	w = w > STRIDE_MIN ? w : STRIDE_MIN;
	w = (w + 63) / 64 * 64;
	return w > 0xffffff00ull ? 0xffffff00u : (uint32_t)w;
}

// What every thread of the preparing pass works out from the records of ray 0 and of the last active ray.
struct Windows { uint64_t base0; uint32_t stride, n_items; };
SRF_HD Windows windows_of(uint32_t n_active, const uint32_t* ray_coord_indices, uint32_t item_cap) {
	Windows W; W.base0 = 0; W.stride = STRIDE_FIT; W.n_items = 0;
	if (n_active == 0) return W;
	const uint64_t b0 = ray_coord_indices[1];
	const uint64_t bl = ray_coord_indices[2 * (size_t)(n_active - 1) + 1], nl = ray_coord_indices[2 * (size_t)(n_active - 1)];
	const uint64_t span = bl >= b0 ? bl - b0 : 0;
	W.base0 = b0;
	W.stride = window_stride(n_active, span, span + nl, item_cap);
	W.n_items = (uint32_t)(span / W.stride) + 1;
	return W;
}

// What the preparing pass leaves per item: its rays [r0, r_end) and its samples [s0, s_end) (from its first ray's first
// sample to its last ray's end; an item without rays has r_end == r0 and s_end == s0).
struct ItemDesc { uint32_t r0, s0, r_end, s_end; };

// Ray i of the preparing pass: is it laid out after its predecessor (returns false if not: the call's rays are not in
// order), and which items does it open (every window from the one after its predecessor's to its own) and close (its
// predecessor's window, and the empty ones up to its own; the last ray closes its own).  desc holds item_cap entries.
SRF_HD bool prepare_ray(uint32_t i, uint32_t n_active, const uint32_t* ray_coord_indices, const Windows& W, uint32_t item_cap, ItemDesc* desc) {
	const uint64_t n = ray_coord_indices[2 * (size_t)i], b = ray_coord_indices[2 * (size_t)i + 1];
	uint64_t w_prev = 0, prev_end = 0;
	if (b < W.base0) return false;
	if (i != 0) {
		const uint64_t pn = ray_coord_indices[2 * (size_t)(i - 1)], pb = ray_coord_indices[2 * (size_t)(i - 1) + 1];
		if (b < pb + pn || pb < W.base0) return false;
		w_prev = (pb - W.base0) / W.stride;
		prev_end = pb + pn;
	}
	const uint64_t w_here = (b - W.base0) / W.stride;
	if (w_here >= W.n_items || b + n > 0xffffffffull) return false;     // beyond the last ray's window: not in order
	if (i != 0 && w_here != w_prev) {
		if (w_prev < item_cap) { desc[w_prev].r_end = i; desc[w_prev].s_end = (uint32_t)prev_end; }
		for (uint64_t w = w_prev + 1; w < w_here; ++w) if (w < item_cap) { ItemDesc d; d.r0 = i; d.r_end = i; d.s0 = (uint32_t)b; d.s_end = (uint32_t)b; desc[w] = d; }
	}
	if ((i == 0 || w_here != w_prev) && w_here < item_cap) { desc[w_here].r0 = i; desc[w_here].s0 = (uint32_t)b; }
	if (i == n_active - 1 && w_here < item_cap) { desc[w_here].r_end = n_active; desc[w_here].s_end = (uint32_t)(b + n); }
	return true;
}

// ---- rows: lane <-> sample -----------------------------------------------------------------
// Samples [chunk_lo, chunk_lo + WIN) of an item whose samples start at s0 and number `range`.  A row past the range
// is skipped outright; a lane past it re-reads the range's last sample (its values are not used).
template <bool HALF_IN>
SRF_HD void rows_load(uint32_t lane, const Args& A, uint64_t s0, uint32_t range, uint32_t chunk_lo, SlotState<G, HALF_IN>& st) {
	if (chunk_lo >= range) return;
	const uint32_t here = range - chunk_lo < WIN ? range - chunk_lo : WIN;
	const uint32_t n_rows = (here + LANES - 1) / LANES;
	const uint32_t* net = (const uint32_t*)A.net + (s0 + chunk_lo) * (HALF_IN ? 2 : 4);
	const float* dt = A.dt_arr + (s0 + chunk_lo) * A.K.dt_stride;
	#pragma unroll
	for (uint32_t j = 0; j < ROWS; ++j) {
		if (j < n_rows) {
			const uint32_t q = lane + j * LANES;
			const uint32_t srel = q < here ? q : here - 1;
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

// activations and alpha; {alpha, colour} to LDS, every sample marked as nobody's
template <bool HALF_IN, bool PLAIN>
SRF_HD void rows_alpha(uint32_t lane, const Args& A, Lds& w, uint32_t range, uint32_t chunk_lo, SlotState<G, HALF_IN>& st) {
	if (chunk_lo >= range) return;
	const int rgb_act = PLAIN ? (int)SRF_ACT_NONE : A.K.rgb_act, density_act = PLAIN ? (int)SRF_ACT_NONE : A.K.density_act;
	const uint32_t here = range - chunk_lo < WIN ? range - chunk_lo : WIN;
	const uint32_t n_rows = (here + LANES - 1) / LANES;
	#pragma unroll
	for (uint32_t j = 0; j < ROWS; ++j) {
		const uint32_t q = lane + j * LANES;
		if (j < n_rows && q < here) {
			float v[4];
			fused::unpack_raw<HALF_IN>(st.raw[j], v);
			const float density = act_density(v[3], density_act);
			const float alpha = 1.f - srf_expf(-density * st.dt[j]);
			st.alpha[j] = alpha;
			w.S[q] = mk4(alpha, act_rgb(v[0], rgb_act), act_rgb(v[1], rgb_act), act_rgb(v[2], rgb_act));
			w.owner[q] = (uint8_t)NO_OWNER;
		}
	}
}

// ---- chain: lane <-> ray (ray_marcher.cu:63-79, and again :171-182) -------------------------
struct RayState {
	float T, r, g, b;
	uint32_t cnt;       // samples consumed so far
	uint32_t dead;      // the termination test `T < threshold` has held
};
SRF_HD void ray_reset(RayState& s) { s.T = 1.f; s.r = 0.f; s.g = 0.f; s.b = 0.f; s.cnt = 0; s.dead = 0; }

// the steps of the lane's ray (n samples, the first at position rbase of the item) that lie in the chunk: [*k0, *k1)
SRF_HD void chain_span(uint32_t n, uint32_t rbase, uint32_t chunk_lo, uint32_t* k0, uint32_t* k1) {
	const uint64_t lo = chunk_lo, hi = (uint64_t)chunk_lo + WIN, first = rbase, end = (uint64_t)rbase + n;
	const uint64_t a = first > lo ? first : lo, b = end < hi ? end : hi;
	if (a >= b) { *k0 = 0; *k1 = 0; return; }
	*k0 = (uint32_t)(a - first); *k1 = (uint32_t)(b - first);
}

// One stretch of CHAIN_UNROLL steps, the j-th and following of the lane's steps in this chunk.  A step whose sample
// is not consumed (past the ray's end, or after the termination test has held) runs on an all-zero record, which
// leaves T (times 1) and the colour sums (plus 0) as they are, so the stretch needs no branches; its reads and
// writes land on the padding past the window.  Written so that only T's products and each colour's sums depend on
// one another.
// the stretch's records, read (one stretch can be read while the one before it is worked on: they are different samples)
struct ChainReads { Float4 v[CHAIN_UNROLL]; uint32_t idx[CHAIN_UNROLL]; bool inb[CHAIN_UNROLL]; };
SRF_HD void chain_read(uint32_t j, uint32_t k0, uint32_t k1, uint32_t rbase, uint32_t chunk_lo, const Lds& w, ChainReads& c) {
	#pragma unroll
	for (uint32_t u = 0; u < CHAIN_UNROLL; ++u) {
		const uint32_t k = k0 + j + u;
		c.inb[u] = k < k1;
		c.idx[u] = c.inb[u] ? rbase + k - chunk_lo : LAST;
		c.v[u] = w.S[c.idx[u]];
	}
}
SRF_HD void chain_apply(uint32_t lane, float thr, Lds& w, RayState& s, ChainReads& c) {
	Float4 out[CHAIN_UNROLL];
	#pragma unroll
	for (uint32_t u = 0; u < CHAIN_UNROLL; ++u) {
		if (c.inb[u] && s.T < thr) s.dead = 1u;                    // the reference tests before it consumes (:64)
		const bool alive = c.inb[u] && s.dead == 0u;
		if (!alive) c.v[u] = mk4(0.f, 0.f, 0.f, 0.f);
		const float a = c.v[u].x;
		const float Tb = s.T, wgt = a * s.T;
		s.T *= (1.f - a);
		s.r += wgt * c.v[u].y; s.g += wgt * c.v[u].z; s.b += wgt * c.v[u].w;
		s.cnt += alive ? 1u : 0u;
		out[u] = mk4(Tb, s.r, s.g, s.b);
	}
	#pragma unroll
	for (uint32_t u = 0; u < CHAIN_UNROLL; ++u) {
		w.S[c.idx[u]] = out[u];
		w.owner[c.idx[u]] = (uint8_t)lane;
	}
}
SRF_HD void chain_stretch(uint32_t lane, uint32_t j, uint32_t k0, uint32_t k1, uint32_t rbase, uint32_t chunk_lo, float thr, Lds& w, RayState& s) {
	ChainReads c;
	chain_read(j, k0, k1, rbase, chunk_lo, w, c);
	chain_apply(lane, thr, w, s, c);
}

// host form of the whole chain of one lane over one chunk (the device loops over stretches itself, with the trip
// count of the wavefront's longest lane and an early exit once no lane has a live step left)
SRF_HD void chain_chunk(uint32_t lane, uint32_t n, uint32_t rbase, uint32_t chunk_lo, uint32_t n_steps, float thr, Lds& w, RayState& s) {
	uint32_t k0, k1;
	chain_span(n, rbase, chunk_lo, &k0, &k1);
	for (uint32_t j = 0; j < n_steps; j += CHAIN_UNROLL) chain_stretch(lane, j, k0, k1, rbase, chunk_lo, thr, w, s);
}

// ---- finish: lane <-> ray (ray_marcher.cu:81-109, 128-133) ----------------------------------
// n: the ray's samples on input; i: its index; returns the ray's loss term
SRF_HD float finish_lane(uint32_t lane, uint32_t i, uint32_t n, const Args& A, Lds& w, const RayState& s, Float4 target_rgba) {
	float target[3], bg[3];
	target_and_background(A.K, target_rgba, target, bg);
	float r = s.r, g = s.g, b = s.b;
	if (s.cnt == n) { r += s.T * bg[0]; g += s.T * bg[1]; b += s.T * bg[2]; }
	RayOut& o = w.out()[lane];
	o.c[0] = r; o.c[1] = g; o.c[2] = b;
	float lo[3];
	loss_channel(A.K.loss_type, target[0], r, &lo[0], &o.g[0]);
	loss_channel(A.K.loss_type, target[1], g, &lo[1], &o.g[1]);
	loss_channel(A.K.loss_type, target[2], b, &lo[2], &o.g[2]);
	if (A.rgb_ray_out) { A.rgb_ray_out[3 * (size_t)i] = r; A.rgb_ray_out[3 * (size_t)i + 1] = g; A.rgb_ray_out[3 * (size_t)i + 2] = b; }
	return (((lo[0] + lo[1]) + lo[2]) / 3.0f) / (float)A.K.n_rays;
}

// after the ordered offset of the ray is known (ray_marcher.cu:116-131)
SRF_HD void commit_lane(uint32_t lane, uint32_t i, uint32_t n_fwd, uint32_t rbase, uint32_t cbase, float loss, const Args& A, Lds& w) {
	RayOut& o = w.out()[lane];
	const uint32_t room = A.K.n_max_compacted - (A.K.n_max_compacted < cbase ? A.K.n_max_compacted : cbase);
	const uint32_t n = room < n_fwd ? room : n_fwd;
	o.obase = cbase - rbase;
	o.s_end = rbase + n;
	A.ray_coord_indices[2 * (size_t)i] = n;
	A.ray_coord_indices[2 * (size_t)i + 1] = cbase;
	if (n != 0 && A.loss_output) A.loss_output[i] = loss;
}
// a lane without a ray owns nothing
SRF_HD void commit_none(uint32_t lane, Lds& w) { w.out()[lane].obase = 0; w.out()[lane].s_end = 0; }

// ---- grads: lane <-> sample (ray_marcher.cu:171-201) ----------------------------------------
template <bool HALF_IN, bool HALF_OUT, bool PLAIN>
SRF_HD void rows_grads(uint32_t lane, const Args& A, const Lds& w, uint64_t s0, uint32_t range, uint32_t chunk_lo, const SlotState<G, HALF_IN>& st) {
	if (chunk_lo >= range) return;
	const int rgb_act = PLAIN ? (int)SRF_ACT_NONE : A.K.rgb_act, density_act = PLAIN ? (int)SRF_ACT_NONE : A.K.density_act;
	const float l2_reg = rgb_act == SRF_ACT_EXPONENTIAL ? 1e-4f : 0.0f;
	const float l1_reg_density = (A.K.use_grid && (A.mean_density < A.K.min_optical_thickness)) ? 1e-4f : 0.0f;
	const uint32_t here = range - chunk_lo < WIN ? range - chunk_lo : WIN;
	const uint32_t n_rows = (here + LANES - 1) / LANES;
	#pragma unroll
	for (uint32_t j = 0; j < ROWS; ++j) {
		if (j >= n_rows) continue;
		const uint32_t q = lane + j * LANES;
		if (q >= here) continue;
		const uint32_t r = w.owner[q];
		if (r >= LANES) continue;
		const uint32_t srel = chunk_lo + q;                       // position in the item
		const Float4 og = *(const Float4*)&w.out()[r].g[0];        // g.xyz, obase
		const Float4 oc = *(const Float4*)&w.out()[r].c[0];        // c.xyz, s_end
		if (srel >= srf_f2u(oc.w)) continue;
		const Float4 after = w.S[q];                              // T before the sample, colour sums including it
		const float T_before = after.x;
		float v[4];
		fused::unpack_raw<HALF_IN>(st.raw[j], v);
		const float cr = act_rgb(v[0], rgb_act), cg = act_rgb(v[1], rgb_act), cb = act_rgb(v[2], rgb_act);
		const float weight = st.alpha[j] * T_before;
		const float T = T_before * (1.f - st.alpha[j]);           // the chain's own update (ray_marcher.cu:181)
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
				U2 p; p.x = lo; p.y = hi;
				*((U2*)A.dloss + o) = p;
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
		if (A.compacted_coords) {                                 // ray_marcher.cu:175: the kept samples' coordinates move with them
			const float* src = A.coords + 7 * (s0 + srel);
			float cc[7];
			for (int c = 0; c < 7; ++c) cc[c] = src[c];
			for (int c = 0; c < 7; ++c) A.compacted_coords[7 * o + c] = cc[c];
		}
	}
}

// ---- the common item's row phases ----------------------------------------------------------
// For an item whose samples fit the window in one piece.  Rows are taken four at a time and nothing in them branches on
// the lane: a row (or lane) past the item's samples works on a copy of its last sample, and what it leaves is not used.
// The gradients are staged in the window, in place of the records they are made from, so that only their stores wait
// for the item's compacted offset.
constexpr uint32_t ROW_BATCH = 4;
SRF_HD uint32_t row_batches(uint32_t range) { return (range + ROW_BATCH * LANES - 1) / (ROW_BATCH * LANES); }

// (a sample's network output stays the one 8- or 16-byte value it was loaded as: split into words that live in registers
// of their own, every load would be followed by a wait and a move)
template <bool HALF_IN> struct RawSample { typedef U4 type; };
template <> struct RawSample<true> { typedef U2 type; };
template <bool HALF_IN>
struct RowData {
	typename RawSample<HALF_IN>::type raw[ROWS];
	float dt[ROWS];
};
SRF_HD void unpack_sample(const U2& raw, float v[4]) {
	v[0] = half_bits_to_float((uint16_t)(raw.x & 0xffffu)); v[1] = half_bits_to_float((uint16_t)(raw.x >> 16));
	v[2] = half_bits_to_float((uint16_t)(raw.y & 0xffffu)); v[3] = half_bits_to_float((uint16_t)(raw.y >> 16));
}
SRF_HD void unpack_sample(const U4& raw, float v[4]) { v[0] = srf_u2f(raw.x); v[1] = srf_u2f(raw.y); v[2] = srf_u2f(raw.z); v[3] = srf_u2f(raw.w); }

// per ray, for the staged phases: {loss gradient, -} {composited colour, -} and where its kept samples go
struct RayLds2 {
	Float4 g[LANES];
	Float4 c[LANES];
	U2 place[LANES];      // x: compacted offset of the ray minus the position of its first sample in the item; y: position after its last kept sample
};

// range != 0.  Every row is loaded, whatever the range (a lane past it re-reads the last sample): loads with nothing
// conditional between them, so that nothing waits for one of them before the values are used.  Rows [j0, j0 + n).
template <bool HALF_IN>
SRF_HD void fit_rows_load_some(uint32_t lane, uint32_t j0, uint32_t n, const Args& A, uint64_t s0, uint32_t range, RowData<HALF_IN>& in) {
	// one base per array, the same in every lane, and a 32-bit byte offset per lane and row
	const char* net = (const char*)A.net + s0 * (HALF_IN ? 8 : 16);
	const char* dt = (const char*)(A.dt_arr + s0 * A.K.dt_stride);
	const uint32_t dt_bytes = A.K.dt_stride * 4u;
	#pragma unroll
	for (uint32_t j = j0; j < j0 + n; ++j) {
		const uint32_t q = lane + j * LANES;
		const uint32_t srel = q < range ? q : range - 1;
		in.raw[j] = *(const typename RawSample<HALF_IN>::type*)(net + (uint32_t)(srel * (HALF_IN ? 8u : 16u)));
		in.dt[j] = *(const float*)(dt + (uint32_t)(srel * dt_bytes));
	}
}
template <bool HALF_IN>
SRF_HD void fit_rows_load(uint32_t lane, const Args& A, uint64_t s0, uint32_t range, RowData<HALF_IN>& in) {
	fit_rows_load_some<HALF_IN>(lane, 0, ROWS, A, s0, range, in);
}

template <bool HALF_IN, bool PLAIN>
SRF_HD void fit_rows_alpha(uint32_t lane, const Args& A, Float4* S, uint8_t* owner, uint32_t range, const RowData<HALF_IN>& in, float* alpha_out) {
	const int rgb_act = PLAIN ? (int)SRF_ACT_NONE : A.K.rgb_act, density_act = PLAIN ? (int)SRF_ACT_NONE : A.K.density_act;
	const uint32_t nb = row_batches(range);
	#pragma unroll
	for (uint32_t j0 = 0; j0 < ROWS; j0 += ROW_BATCH) {
		if (j0 / ROW_BATCH < nb) {
			#pragma unroll
			for (uint32_t j = j0; j < j0 + ROW_BATCH; ++j) {
				const uint32_t q = lane + j * LANES;
				float v[4];
				unpack_sample(in.raw[j], v);
				const float density = act_density(v[3], density_act);
				const float alpha = 1.f - srf_expf(-density * in.dt[j]);
				alpha_out[j] = alpha;
				float alpha_rec = alpha;
				SRF_OPAQUE_F32(alpha_rec);      // (a register of its own in the record's four: the kept alpha is not tied to them)
				S[q] = mk4(alpha_rec, act_rgb(v[0], rgb_act), act_rgb(v[1], rgb_act), act_rgb(v[2], rgb_act));
				owner[q] = (uint8_t)NO_OWNER;
			}
		}
	}
}

// ray_marcher.cu:171-195 for every sample that a chain took: the four gradients replace the sample's record
// rows [jb, jb + ROW_BATCH)
template <bool HALF_IN, bool PLAIN>
SRF_HD void fit_rows_grads_some(uint32_t lane, uint32_t jb, const Args& A, Float4* S, const uint8_t* owner, const RayLds2& rl, uint32_t range, const RowData<HALF_IN>& in, const float* alpha) {
	const int rgb_act = PLAIN ? (int)SRF_ACT_NONE : A.K.rgb_act, density_act = PLAIN ? (int)SRF_ACT_NONE : A.K.density_act;
	const float l2_reg = rgb_act == SRF_ACT_EXPONENTIAL ? 1e-4f : 0.0f;
	const float l1_reg_density = (A.K.use_grid && (A.mean_density < A.K.min_optical_thickness)) ? 1e-4f : 0.0f;
	const uint32_t nb = row_batches(range);
	constexpr uint32_t GB = 4;          // rows whose LDS reads are under way together
	#pragma unroll
	for (uint32_t j0 = jb; j0 < jb + ROW_BATCH; j0 += GB) {
		if (j0 / ROW_BATCH < nb) {
			uint32_t r[GB];
			Float4 og[GB], oc[GB], after[GB];
			#pragma unroll
			for (uint32_t u = 0; u < GB; ++u) { const uint32_t o = owner[lane + (j0 + u) * LANES]; r[u] = o < LANES ? o : 0u; }
			#pragma unroll
			for (uint32_t u = 0; u < GB; ++u) { og[u] = rl.g[r[u]]; oc[u] = rl.c[r[u]]; after[u] = S[lane + (j0 + u) * LANES]; }
			#pragma unroll
			for (uint32_t u = 0; u < GB; ++u) {
				const uint32_t j = j0 + u;
				const float T_before = after[u].x;
				float v[4];
				typename RawSample<HALF_IN>::type raw = in.raw[j];
				SRF_OPAQUE_U32(raw.x); SRF_OPAQUE_U32(raw.y);     // (the colours are converted again rather than kept since the first phase)
				unpack_sample(raw, v);
				const float cr = act_rgb(v[0], rgb_act), cg = act_rgb(v[1], rgb_act), cb = act_rgb(v[2], rgb_act);
				const float weight = alpha[j] * T_before;
				const float T = T_before * (1.f - alpha[j]);          // the chain's own update (ray_marcher.cu:181)
				const float d0 = A.K.loss_scale * ((weight * og[u].x) * act_rgb_derivative(v[0], rgb_act) + srf_max_zero(l2_reg * v[0]));
				const float d1 = A.K.loss_scale * ((weight * og[u].y) * act_rgb_derivative(v[1], rgb_act) + srf_max_zero(l2_reg * v[1]));
				const float d2 = A.K.loss_scale * ((weight * og[u].z) * act_rgb_derivative(v[2], rgb_act) + srf_max_zero(l2_reg * v[2]));
				const float sx = oc[u].x - after[u].y, sy = oc[u].y - after[u].z, sz = oc[u].z - after[u].w;
				const float dd = act_density_derivative(v[3], density_act);
				const float dotv = (og[u].x * (T * cr - sx) + og[u].y * (T * cg - sy)) + og[u].z * (T * cb - sz);
				const float dmlp = dd * (in.dt[j] * dotv);
				const float d3 = A.K.loss_scale * dmlp + (v[3] < 0 ? -l1_reg_density : 0.0f);
				S[lane + j * LANES] = mk4(d0, d1, d2, d3);
			}
		}
	}
}

template <bool HALF_IN, bool PLAIN>
SRF_HD void fit_rows_grads(uint32_t lane, const Args& A, Float4* S, const uint8_t* owner, const RayLds2& rl, uint32_t range, const RowData<HALF_IN>& in, const float* alpha) {
	#pragma unroll
	for (uint32_t jb = 0; jb < ROWS; jb += ROW_BATCH) fit_rows_grads_some<HALF_IN, PLAIN>(lane, jb, A, S, owner, rl, range, in, alpha);
}

// the staged gradients of the kept samples go to their compacted positions (records 4 wide: one 16- or 8-byte store a sample)
// (place.x counts from `first`, the compacted position of the item's first kept sample)
template <bool HALF_OUT>
SRF_HD void fit_rows_store(uint32_t lane, const Args& A, const Float4* S, const uint8_t* owner, const RayLds2& rl, uint64_t s0, uint32_t range, uint32_t first) {
	const uint32_t nb = row_batches(range);
	char* out = (char*)A.dloss + (size_t)first * (HALF_OUT ? 8 : 16);
	#pragma unroll
	for (uint32_t j0 = 0; j0 < ROWS; j0 += ROW_BATCH) {
		if (j0 / ROW_BATCH < nb) {
			uint32_t o[ROW_BATCH];
			U2 place[ROW_BATCH];
			Float4 d[ROW_BATCH];
			#pragma unroll
			for (uint32_t u = 0; u < ROW_BATCH; ++u) o[u] = owner[lane + (j0 + u) * LANES];
			#pragma unroll
			for (uint32_t u = 0; u < ROW_BATCH; ++u) { place[u] = rl.place[o[u] < LANES ? o[u] : 0u]; d[u] = S[lane + (j0 + u) * LANES]; }
			#pragma unroll
			for (uint32_t u = 0; u < ROW_BATCH; ++u) {
				const uint32_t q = lane + (j0 + u) * LANES;
				if (o[u] < LANES && q < place[u].y) {
					const uint32_t rel = place[u].x + q;              // < the item's samples
					if (HALF_OUT) {
						U2 p;
						p.x = (uint32_t)float_to_half_bits(d[u].x) | ((uint32_t)float_to_half_bits(d[u].y) << 16);
						p.y = (uint32_t)float_to_half_bits(d[u].z) | ((uint32_t)float_to_half_bits(d[u].w) << 16);
						*(U2*)(out + (uint32_t)(rel * 8u)) = p;
					} else {
						*(Float4*)(out + (uint32_t)(rel * 16u)) = d[u];
					}
					if (A.compacted_coords) {                         // ray_marcher.cu:175: the kept samples' coordinates move with them
						const float* src = A.coords + 7 * (s0 + q);
						float* dst = A.compacted_coords + 7 * ((size_t)first + rel);
						float cc[7];
						for (int c = 0; c < 7; ++c) cc[c] = src[c];
						for (int c = 0; c < 7; ++c) dst[c] = cc[c];
					}
				}
			}
		}
	}
}

// finish_lane and commit_lane for the staged phases
SRF_HD float fit_finish_lane(uint32_t lane, uint32_t i, uint32_t n, const Args& A, RayLds2& rl, const RayState& s, Float4 target_rgba) {
	float target[3], bg[3];
	target_and_background(A.K, target_rgba, target, bg);
	float r = s.r, g = s.g, b = s.b;
	if (s.cnt == n) { r += s.T * bg[0]; g += s.T * bg[1]; b += s.T * bg[2]; }
	float lo[3], gr[3];
	loss_channel(A.K.loss_type, target[0], r, &lo[0], &gr[0]);
	loss_channel(A.K.loss_type, target[1], g, &lo[1], &gr[1]);
	loss_channel(A.K.loss_type, target[2], b, &lo[2], &gr[2]);
	rl.g[lane] = mk4(gr[0], gr[1], gr[2], 0.f);
	rl.c[lane] = mk4(r, g, b, 0.f);
	if (A.rgb_ray_out) { A.rgb_ray_out[3 * (size_t)i] = r; A.rgb_ray_out[3 * (size_t)i + 1] = g; A.rgb_ray_out[3 * (size_t)i + 2] = b; }
	return (((lo[0] + lo[1]) + lo[2]) / 3.0f) / (float)A.K.n_rays;
}
// first: the compacted offset of the item's first ray
SRF_HD void fit_commit_lane(uint32_t lane, uint32_t i, uint32_t n_fwd, uint32_t rbase, uint32_t cbase, uint32_t first, float loss, const Args& A, RayLds2& rl) {
	const uint32_t room = A.K.n_max_compacted - (A.K.n_max_compacted < cbase ? A.K.n_max_compacted : cbase);
	const uint32_t n = room < n_fwd ? room : n_fwd;
	U2 p; p.x = (cbase - first) - rbase; p.y = rbase + n;
	rl.place[lane] = p;
	A.ray_coord_indices[2 * (size_t)i] = n;
	A.ray_coord_indices[2 * (size_t)i + 1] = cbase;
	if (n != 0 && A.loss_output) A.loss_output[i] = loss;
}
SRF_HD void fit_commit_none(uint32_t lane, RayLds2& rl) { U2 p; p.x = 0; p.y = 0; rl.place[lane] = p; }

} // namespace wv
} // namespace srf
