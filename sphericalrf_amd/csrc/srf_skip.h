// Empty-space table for the marching kernels.  The reference marches every step and probes the
// occupancy bitfield at each one (internal/sampler/occupancy_sampler.cu:595-633); the table lets
// a ray prove that a run of its steps cannot hit an occupied cell and advance t through them
// without probing.  The t chain itself is never shortened, so the samples that come out are the
// ones the reference produces, bit for bit.
//
// Layout: the cascaded grid (WarpedSpace_Exp cascades only) is cut into nb^3 blocks per cascade
// that are cubes in warped space (side 2^-(C-1-level) / nb).  dist[level][bz][by][bx] is a
// Chebyshev radius, in units of the finest cascade's block side, such that NO warped position
// within that radius of any point of the block looks up an occupied cell, whichever cascade that
// position selects.  It is rebuilt whenever the bitfield is.
//
// Why one radius covers every cascade: block occupancy is pooled upwards (a block is occupied
// when any of its own cells or any block of the finer cascade inside it is), so a position that
// selects a finer cascade than the block's is covered by the block's own cascade; positions that
// would leave the block's cascade are excluded by clamping the radius at the cascade's edge; and a
// block inherits the radius of the coarser-cascade block that contains it when that is larger.
#pragma once
#include "srf_device.h"

// hook for host builds that tally the radii the march reads
#ifndef SRF_COUNT_RADIUS
#define SRF_COUNT_RADIUS(n, level) ((void)0)
#endif

namespace srf {

constexpr uint32_t SKIP_MAX_BLOCKS = 64;   // per axis
constexpr uint32_t SKIP_MAX_RADIUS = 32;   // in blocks of a block's own cascade

SRF_HD uint32_t ilog2_u32(uint32_t v) { uint32_t r = 0; while (v > 1u) { v >>= 1; ++r; } return r; }

// blocks per axis for a grid, 0 when the table is not built (tiny grids, other cascade layouts)
SRF_HD uint32_t skip_blocks_per_axis(const Params& P) {
	if (!P.use_grid || P.griddist_type != SRF_GRID_WARPED_EXP) return 0;
	if (P.warping_type != SRF_WARP_ERP && P.warping_type != SRF_WARP_SINUSOIDAL) return 0;
	const uint32_t gz = P.grid_size[2];
	if (gz < 16) return 0;
	// blocks of four cells a side; two on small grids, where the coarser table leaves most probes of a ray that runs through
	// occupied surroundings in place (workload 1: 501 of 512 lookups a ray against 103) -- on a 128-grid the finer, 8 x larger
	// table saves a seventh of the lookups and makes a frame a fifth slower
	const uint32_t nb = gz <= 64 ? gz / 2 : gz / 4;
	return nb < SKIP_MAX_BLOCKS ? nb : SKIP_MAX_BLOCKS;
}

SRF_HD SkipTable skip_table_for(const Params& P, const uint16_t* dist) {
	SkipTable t;
	t.nb = skip_blocks_per_axis(P);
	t.dist = t.nb ? dist : nullptr;
	t.sx = t.sy = t.sz = 0; t.side0 = 0.f;
	if (t.nb) {
		t.sx = ilog2_u32(P.grid_size[0] / t.nb);
		t.sy = ilog2_u32(P.grid_size[1] / t.nb);
		t.sz = ilog2_u32(P.grid_size[2] / t.nb);
		t.side0 = srf_exp2i(-(int)(P.n_cascades - 1)) / (float)t.nb;
	}
	return t;
}

// ---- build, step 1: a block is occupied when any of its cells is.  i runs over cascades x blocks.
SRF_HD void skip_block_occupancy_body(uint32_t i, const Params& P, SkipTable T, const uint8_t* bitfield, uint8_t* occ) {
	const uint32_t nb = T.nb, nb3 = nb * nb * nb;
	const uint32_t level = i / nb3, r = i % nb3;
	const uint32_t bx = r % nb, by = (r / nb) % nb, bz = r / (nb * nb);
	const uint32_t c = 1u << T.sz;                      // a c^3 cube of cells is c^3 consecutive Morton indices
	const uint32_t nx = 1u << (T.sx - T.sz), ny = 1u << (T.sy - T.sz);
	const uint32_t bytes = (c * c * c) / 8u;
	const uint8_t* lvl = bitfield + (size_t)level * (P.n_cells / 8u);
	uint32_t any = 0;
	for (uint32_t a = 0; a < nx; ++a)
		for (uint32_t b = 0; b < ny; ++b) {
			const uint32_t m = morton3d((bx << T.sx) + a * c, (by << T.sy) + b * c, bz << T.sz);
			const uint8_t* p = lvl + m / 8u;
			for (uint32_t k = 0; k < bytes; ++k) any |= p[k];
		}
	occ[i] = any ? 1 : 0;
}

// ---- build, step 2 (cascade by cascade, finest first): pool the finer cascade's blocks into the
// coarser blocks that contain them.  i runs over the (nb/2)^3 central blocks of `level` (>= 1).
SRF_HD void skip_pool_body(uint32_t i, SkipTable T, uint32_t level, uint8_t* occ) {
	const uint32_t nb = T.nb, h = nb / 2;
	const uint32_t px = i % h, py = (i / h) % h, pz = i / (h * h);
	uint32_t any = 0;
	for (uint32_t k = 0; k < 8; ++k) any |= occ[skip_index(nb, level - 1, 2 * px + (k & 1u), 2 * py + ((k >> 1) & 1u), 2 * pz + (k >> 2))];
	if (any) occ[skip_index(nb, level, px + nb / 4, py + nb / 4, pz + nb / 4)] = 1;
}

// ---- build, step 3: Chebyshev distance to the nearest occupied block of the same cascade, one
// axis at a time.  The first axis reads the occupancy flags (occupied -> 0, empty -> SKIP_MAX_RADIUS),
// the others the previous axis' result.  out(b) = min over offsets k along the axis of max(in(b+k), |k|).
SRF_HD uint32_t skip_axis_read(const uint8_t* in, size_t i, bool flags) { const uint32_t v = in[i]; return flags ? (v ? 0u : SKIP_MAX_RADIUS) : v; }
SRF_HD void skip_distance_axis_body(uint32_t i, SkipTable T, uint32_t axis, const uint8_t* in, uint8_t* out) {
	const bool flags = axis == 0;
	const uint32_t nb = T.nb, nb3 = nb * nb * nb;
	const uint32_t r = i % nb3;
	uint32_t co[3] = { r % nb, (r / nb) % nb, r / (nb * nb) };
	const uint32_t stride = axis == 0 ? 1u : (axis == 1 ? nb : nb * nb);
	const uint32_t at = co[axis];
	uint32_t best = skip_axis_read(in, i, flags);
	for (uint32_t k = 1; k < best; ++k) {
		if (at >= k) { const uint32_t v = skip_axis_read(in, i - k * stride, flags); const uint32_t m = v > k ? v : k; best = m < best ? m : best; }
		if (at + k < nb) { const uint32_t v = skip_axis_read(in, i + k * stride, flags); const uint32_t m = v > k ? v : k; best = m < best ? m : best; }
	}
	out[i] = (uint8_t)best;
}

// ---- build, step 4: radius per block.  n = distance (in blocks) to the nearest occupied block;
// every cascade but the outermost also stops at its own edge; the radius is (n - 1) block sides,
// and a block takes the best radius among itself and the coarser blocks that contain it.
SRF_HD void skip_combine_body(uint32_t i, const Params& P, SkipTable T, const uint8_t* n_blocks, uint16_t* dist) {
	const uint32_t nb = T.nb, nb3 = nb * nb * nb;
	uint32_t level = i / nb3;
	const uint32_t r = i % nb3;
	uint32_t bx = r % nb, by = (r / nb) % nb, bz = r / (nb * nb);
	uint32_t best = 0;
	for (; level < P.n_cascades; ++level) {
		uint32_t n = n_blocks[skip_index(nb, level, bx, by, bz)];
		if (level + 1 < P.n_cascades) {
			uint32_t e = bx < nb - 1 - bx ? bx : nb - 1 - bx;
			const uint32_t ey = by < nb - 1 - by ? by : nb - 1 - by, ez = bz < nb - 1 - bz ? bz : nb - 1 - bz;
			e = e < ey ? e : ey; e = e < ez ? e : ez;
			n = n < e + 1 ? n : e + 1;
		}
		if (n > 0) { const uint32_t rad = (n - 1) << level; best = rad > best ? rad : best; }
		bx = (bx >> 1) + nb / 4; by = (by >> 1) + nb / 4; bz = (bz >> 1) + nb / 4;
	}
	dist[i] = (uint16_t)best;
}

// ------------------------------------------------------------------------------------
// use: per-ray constants and the per-probe bound on t
// ------------------------------------------------------------------------------------
struct SkipRay {
	float t_c;        // parameter of the ray's closest approach to the warp centre (0.5,0.5,0.5)
	float inv_speed;  // 1 / |d|
	float cut_lo, cut_hi;   // the ray crosses the azimuth branch cut (y = 0.5, x < 0.5) inside [cut_lo, cut_hi]; +huge when it does not
	float b_lo, b_hi;       // lower and upper bound of the ray's distance of closest approach to the centre
	Vec3  oc;         // o - centre
};

SRF_HD SkipRay skip_ray_setup(Vec3 o, Vec3 d) {
	SkipRay R;
	R.oc = shift3(o, -0.5f);
	const float dd = (d.x * d.x + d.y * d.y) + d.z * d.z;
	const float speed = srf_sqrt(dd);
	R.inv_speed = speed > 0.f ? 1.f / speed : 0.f;
	const float od = (R.oc.x * d.x + R.oc.y * d.y) + R.oc.z * d.z;
	R.t_c = dd > 0.f ? -od / dd : 0.f;
	// closest approach b: b^2 = |oc|^2 - (oc.d)^2 / |d|^2, a difference of like-sized numbers, hence the error allowance
	const float oc2 = dot3(R.oc, R.oc);
	const float b2 = dd > 0.f ? oc2 - od * od / dd : oc2;
	const float err = 8e-6f * oc2 + 1e-12f;
	R.b_hi = srf_sqrt(srf_max(b2, 0.f) + err) * 1.0005f;
	R.b_lo = srf_sqrt(srf_max(b2 - err, 0.f)) * 0.9995f;
	R.cut_lo = R.cut_hi = 3.0e38f;
	if (d.y != 0.f) {
		const float t_cut = -R.oc.y / d.y;
		const float x_cross = R.oc.x + t_cut * d.x;
		if (x_cross < 1e-3f) {   // also taken for NaN-free borderline crossings near the polar axis
			const float m = 1e-4f * (1.f + srf_abs(t_cut)) + (1e-4f + 2e-6f * srf_abs(R.oc.y)) / srf_abs(d.y);
			R.cut_lo = t_cut - m;
			R.cut_hi = t_cut + m;
		}
		if (!(x_cross == x_cross)) { R.cut_lo = -3.0e38f; R.cut_hi = 3.0e38f; }   // undecidable: never skip
	}
	return R;
}

// Path length along which no component of the sinusoidal warp can change by more than rho, when the
// distance to the warp centre stays >= m and |sin(elevation)| <= s_phi over that length.  A point moving
// on a line turns around the centre at b / r^2 radians per unit length (b: the line's closest approach),
// at most 1 / r.  Per unit of turning angle, elevation/pi changes by at most 1/pi and
// azimuth * cos(elevation) / (2 pi) by at most (1 + pi |sin(elevation)|) / (2 pi)  (|cos dtheta| <= dOmega,
// |theta sin(phi) dphi| <= pi |sin(phi)| dOmega); the radial component changes by at most 1/2 per unit
// length inside the unit sphere and 1 / (2 r^2) outside.
SRF_HD float skip_safe_length(const SkipRay& R, float rho, float s_phi, float m) {
	if (!(m > 1e-6f)) return 0.f;
	const float inv_m = srf_approx_rcp(m), inv_m2 = inv_m * inv_m;
	const float omega = srf_min(R.b_hi * inv_m2, inv_m);
	const float rate_x = omega * (1.f + 3.1415927f * s_phi) * 0.15915494f;
	const float rate_y = omega * 0.31830989f;
	const float rate_z = 0.5f * srf_min(1.f, inv_m2);
	const float rate = srf_max(rate_x, srf_max(rate_y, rate_z));
	return rho * srf_approx_rcp(rate);
}

// Largest t' such that every step with t <= t'' < t' is known to look up an empty cell, given an
// unoccupied probe at t that read radius n (table units) for its block of cascade `level`.  Returns t when nothing
// can be skipped.
// Parameter stretch dt such that the warped position of o + t'' d stays within rho (every component) of the one at t
// for all t <= t'' <= t + dt, as long as the ray does not cross the azimuth branch cut in between.
SRF_HD float skip_stretch(const SkipRay& R, Vec3 d, float t, float rho) {
	const Vec3 p = mk3(R.oc.x + t * d.x, R.oc.y + t * d.y, R.oc.z + t * d.z);
	const float mag = srf_approx_sqrt(dot3(p, p));
	// inside the ball of radius rho the elevation moves by at most pi * rho
	const float s_phi = srf_min(1.f, srf_abs(p.z) * srf_approx_rcp(mag) + 3.1415927f * rho + 1e-3f);
	// smallest distance to the centre over the stretch: moving away it is the current one; moving closer, the
	// stretch computed for the current distance bounds how far the distance can drop, and the stretch is recomputed for that
	float len = skip_safe_length(R, rho, s_phi, mag);
	if (t < R.t_c) len = skip_safe_length(R, rho, s_phi, srf_max(R.b_lo, mag - len));
	return 0.9f * len * R.inv_speed;
}

SRF_HD float skip_limit(const Params& P, const SkipTable& T, const SkipRay& R, Vec3 o, Vec3 d, float t, uint32_t n, uint32_t level) {
	SRF_COUNT_RADIUS(n, level);
	if (n == 0u) return t;
	if (!(t < R.cut_lo || t > R.cut_hi)) return t;
	float lim = t + skip_stretch(R, d, t, (float)n * T.side0);
	if (t < R.cut_lo && lim > R.cut_lo) lim = R.cut_lo;
	// the march stops at the first step outside the box: positions are monotone in t per axis, so
	// when both ends of the stretch are inside every step between them is
	if (!(lim > t) || !aabb_contains(P, along(o, d, lim))) return t;
	return lim;
}

} // namespace srf
