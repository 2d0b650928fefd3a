// Device-side building blocks of the sampling / marching / compositing kernels.
// Everything here is `__host__ __device__` so the same bodies can also be compiled
// by a host compiler for bounds-checked runs of the per-ray logic.
//
// Arithmetic follows the reference's device helpers operation by operation
// (file:line cited per function); implicit fused multiply-adds are disabled at
// compile time, so a*b+c below always means a rounded product followed by a
// rounded sum.
#pragma once
#include <stdint.h>
#include <stddef.h>
#include "srf_elem.h"
#include "../../include/srf_hip.h"

namespace srf {

// ------------------------------------------------------------------------------------
// kernel-side copy of the sampler's public members (occupancy_sampler.h:88-122)
// ------------------------------------------------------------------------------------
struct Params {
	int32_t  warping_type;
	int32_t  griddist_type;
	int32_t  sampling_type;
	int32_t  use_grid;
	float    aabb_min[3];
	float    aabb_max[3];
	uint32_t aabb_scale;
	uint32_t grid_size[3];
	uint32_t n_cascades;
	uint32_t n_max_steps;
	float    cone_angle_constant;
	float    min_cone_stepsize;
	float    max_cone_stepsize;
	float    near_distance;
	float    far_distance;
	int32_t  snap_train;
	int32_t  snap_render;
	float    min_optical_thickness;
	float    ema_decay;
	uint32_t n_cells;          // grid_size[0]*grid_size[1]*grid_size[2]
	float    sphere[4];        // optional bound of the marches: centre and radius, radius <= 0 = none (not in the reference)
};

struct Vec3 { float x, y, z; };
SRF_HD Vec3 mk3(float x, float y, float z) { Vec3 v; v.x = x; v.y = y; v.z = z; return v; }
SRF_HD Vec3 ld3(const float* p) { return mk3(p[0], p[1], p[2]); }
SRF_HD void st3(float* p, Vec3 v) { p[0] = v.x; p[1] = v.y; p[2] = v.z; }
SRF_HD Vec3 add3(Vec3 a, Vec3 b) { return mk3(a.x + b.x, a.y + b.y, a.z + b.z); }
SRF_HD Vec3 sub3(Vec3 a, Vec3 b) { return mk3(a.x - b.x, a.y - b.y, a.z - b.z); }
SRF_HD Vec3 scale3(Vec3 a, float s) { return mk3(a.x * s, a.y * s, a.z * s); }
SRF_HD Vec3 shift3(Vec3 a, float s) { return mk3(a.x + s, a.y + s, a.z + s); }
SRF_HD float dot3(Vec3 a, Vec3 b) { return (a.x * b.x + a.y * b.y) + a.z * b.z; }
SRF_HD float len3(Vec3 a) { return srf_sqrt(dot3(a, a)); }
SRF_HD Vec3 unit3(Vec3 a) {
	const float q = dot3(a, a);
	if (q > 0.f) { const float n = srf_sqrt(q); return mk3(a.x / n, a.y / n, a.z / n); }
	return a;
}
// point on a ray: o + t*d per component
SRF_HD Vec3 along(Vec3 o, Vec3 d, float t) { return mk3(o.x + t * d.x, o.y + t * d.y, o.z + t * d.z); }

SRF_HD float clamp_f(float v, float lo, float hi) { return v < lo ? lo : (hi < v ? hi : v); }
SRF_HD int32_t clamp_i(int32_t v, int32_t lo, int32_t hi) { return v < lo ? lo : (hi < v ? hi : v); }
SRF_HD float logistic_f(float x) { return 1.0f / (1.0f + srf_expf(-x)); }
SRF_HD float logit_f(float x) { return -srf_logf(1.0f / (srf_min(srf_max(x, 1e-9f), 1.0f - 1e-9f)) - 1.0f); }

// ------------------------------------------------------------------------------------
// binary16 <-> binary32
// ------------------------------------------------------------------------------------
SRF_HD float half_bits_to_float(uint16_t h) {
#if defined(__HIP_DEVICE_COMPILE__)
	_Float16 v;
	__builtin_memcpy(&v, &h, 2);
	return (float)v;
#else
	const uint32_t s = (uint32_t)(h & 0x8000u) << 16;
	const uint32_t e = (h >> 10) & 0x1fu;
	uint32_t m = h & 0x3ffu;
	if (e == 31) return srf_u2f(s | 0x7f800000u | (m << 13));
	if (e != 0) return srf_u2f(s | ((e + 112u) << 23) | (m << 13));
	// zero / subnormal: m * 2^-24 is exact in binary32
	const float mag = (float)m * 5.9604644775390625e-8f;
	return srf_u2f(s | srf_f2u(mag));
#endif
}

SRF_HD uint16_t float_to_half_bits(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
	// The value converted is the binary32 result already rounded: without this the compiler may merge the multiplication that
	// produced it with the conversion into one mixed-precision instruction that rounds once, which is not what the host does.
	asm volatile("" : "+v"(f));
	const _Float16 v = (_Float16)f;   // round to nearest even
	uint16_t h;
	__builtin_memcpy(&h, &v, 2);
	return h;
#else
	const uint32_t u = srf_f2u(f);
	const uint32_t s = (u >> 16) & 0x8000u;
	const uint32_t a = u & 0x7fffffffu;
	if (a > 0x7f800000u) return (uint16_t)(s | 0x7e00u | ((a >> 13) & 0x3ffu));
	if (a >= 0x477ff000u) return (uint16_t)(s | 0x7c00u);
	if (a < 0x33000001u) return (uint16_t)s;
	const int32_t e = (int32_t)(a >> 23) - 127;
	const uint32_t m = (a & 0x7fffffu) | 0x800000u;
	const int sh = e < -14 ? 13 + (-14 - e) : 13;
	uint32_t q = m >> sh;
	const uint32_t rem = m & ((1u << sh) - 1u), halfway = 1u << (sh - 1);
	if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
	const uint32_t r = e < -14 ? q : (((uint32_t)(e + 15) - 1u) << 10) + q;
	return (uint16_t)(s | r);
#endif
}

// network record element i, stored as binary16 or binary32
template <bool HALF>
SRF_HD float net_load(const void* p, size_t i) {
	if (HALF) return half_bits_to_float(((const uint16_t*)p)[i]);
	return ((const float*)p)[i];
}
template <bool HALF>
SRF_HD void net_store(void* p, size_t i, float v) {
	if (HALF) ((uint16_t*)p)[i] = float_to_half_bits(v);
	else ((float*)p)[i] = v;
}

// ------------------------------------------------------------------------------------
// tiny-cuda-nn primitives the path relies on (public upstream definitions):
// morton3D / morton3D_invert, pcg32.  Call sites: occupancy_sampler.cu:141-143,
// 280-284, 448; random_val.cuh:6.
// ------------------------------------------------------------------------------------
SRF_HD uint32_t spread3(uint32_t v) {   // bit k of a 10-bit value moves to bit 3k
	v = (v | (v << 16)) & 0xFF0000FFu;
	v = (v | (v << 8)) & 0x0F00F00Fu;
	v = (v | (v << 4)) & 0xC30C30C3u;
	v = (v | (v << 2)) & 0x49249249u;
	return v;
}
SRF_HD uint32_t morton3d(uint32_t x, uint32_t y, uint32_t z) { return spread3(x) | (spread3(y) << 1) | (spread3(z) << 2); }
SRF_HD uint32_t morton3d_invert(uint32_t x) {
	x &= 0x49249249u;
	x = (x | (x >> 2)) & 0xc30c30c3u;
	x = (x | (x >> 4)) & 0x0f00f00fu;
	x = (x | (x >> 8)) & 0xff0000ffu;
	x = (x | (x >> 16)) & 0x0000ffffu;
	return x;
}

struct Pcg32 { uint64_t state, inc; };
SRF_HD uint32_t pcg_next_uint(Pcg32& r) {
	const uint64_t old = r.state;
	r.state = old * 0x5851f42d4c957f2dULL + r.inc;
	const uint32_t xs = (uint32_t)(((old >> 18u) ^ old) >> 27u);
	const uint32_t rot = (uint32_t)(old >> 59u);
	return (xs >> rot) | (xs << ((~rot + 1u) & 31u));
}
SRF_HD float pcg_next_float(Pcg32& r) { return srf_u2f((pcg_next_uint(r) >> 9) | 0x3f800000u) - 1.0f; }
SRF_HD void pcg_advance(Pcg32& r, uint64_t delta) {
	uint64_t cur_mult = 0x5851f42d4c957f2dULL, cur_plus = r.inc, acc_mult = 1u, acc_plus = 0u;
	while (delta > 0) {
		if (delta & 1) { acc_mult *= cur_mult; acc_plus = acc_plus * cur_mult + cur_plus; }
		cur_plus = (cur_mult + 1) * cur_plus;
		cur_mult *= cur_mult;
		delta >>= 1;
	}
	r.state = acc_mult * r.state + acc_plus;
}
// The same skip-ahead from a table of the generator's 2^b-step maps (state -> m[b]*state + p[b]), which depend on the
// stream constant only: one multiply-add per set bit of delta instead of three multiplies per bit.
struct PcgSkip { uint64_t m[32], p[32]; };
SRF_HD void pcg_skip_table(const Pcg32& r, PcgSkip& T) {
	uint64_t mult = 0x5851f42d4c957f2dULL, plus = r.inc;
	for (int b = 0; b < 32; ++b) { T.m[b] = mult; T.p[b] = plus; plus = (mult + 1) * plus; mult *= mult; }
}
SRF_HD void pcg_advance_u32(Pcg32& r, uint32_t delta, const PcgSkip& T) {
	for (uint32_t b = 0; delta != 0u; ++b, delta >>= 1) if (delta & 1u) r.state = T.m[b] * r.state + T.p[b];
}
// Skip-ahead in eight hexadecimal digits: entry [16 d + k] of the tables is the generator's map for k * 16^d steps
// (state -> m * state + p), so a 32-bit distance is eight multiply-adds.  pcg_skip16_entry computes one entry the plain way.
SRF_HD void pcg_skip16_entry(const Pcg32& r, uint32_t entry, uint64_t* m, uint64_t* p) {
	uint64_t delta = (uint64_t)(entry & 15u) << (4u * (entry >> 4));
	uint64_t cur_mult = 0x5851f42d4c957f2dULL, cur_plus = r.inc, acc_mult = 1u, acc_plus = 0u;
	while (delta > 0) {
		if (delta & 1) { acc_mult *= cur_mult; acc_plus = acc_plus * cur_mult + cur_plus; }
		cur_plus = (cur_mult + 1) * cur_plus;
		cur_mult *= cur_mult;
		delta >>= 1;
	}
	*m = acc_mult; *p = acc_plus;
}
SRF_HD void pcg_advance_skip16(Pcg32& r, uint32_t delta, const uint64_t* m, const uint64_t* p) {
	for (uint32_t d = 0; d < 8; ++d) {
		const uint32_t e = 16u * d + ((delta >> (4u * d)) & 15u);
		r.state = m[e] * r.state + p[e];
	}
}
SRF_HD void pcg_seed(Pcg32& r, uint64_t initstate, uint64_t initseq) {
	r.state = 0u;
	r.inc = (initseq << 1u) | 1u;
	pcg_next_uint(r);
	r.state += initstate;
	pcg_next_uint(r);
}

// ------------------------------------------------------------------------------------
// random_val.cuh:137-273 — scrambled Sobol.  Only dimensions 0 and 1 are used on
// this path; their direction numbers have closed forms (dimension 0: single bits,
// i.e. bit reversal; dimension 1: v[k] = v[k-1] ^ (v[k-1] >> 1) from 0x80000000).
// ------------------------------------------------------------------------------------
SRF_HD uint32_t reverse_bits32(uint32_t x) {
	x = (((x & 0xaaaaaaaau) >> 1) | ((x & 0x55555555u) << 1));
	x = (((x & 0xccccccccu) >> 2) | ((x & 0x33333333u) << 2));
	x = (((x & 0xf0f0f0f0u) >> 4) | ((x & 0x0f0f0f0fu) << 4));
	x = (((x & 0xff00ff00u) >> 8) | ((x & 0x00ff00ffu) << 8));
	return (x >> 16) | (x << 16);
}
SRF_HD uint32_t sobol01(uint32_t index, uint32_t dim) {
	if (dim == 0) return reverse_bits32(index);
	uint32_t X = 0, v = 0x80000000u;
	for (uint32_t bit = 0; bit < 32; ++bit) {
		if ((index >> bit) & 1u) X ^= v;
		v ^= v >> 1;
	}
	return X;
}
SRF_HD uint32_t hash_combine(uint32_t seed, uint32_t v) { return seed ^ (v + (seed << 6) + (seed >> 2)); }
SRF_HD uint32_t lk_permute(uint32_t x, uint32_t seed) {
	x += seed;
	x ^= x * 0x6c50b47cu;
	x ^= x * 0xb82f1e52u;
	x ^= x * 0xc7afe638u;
	x ^= x * 0x8d22f6e6u;
	return x;
}
SRF_HD uint32_t owen_scramble(uint32_t x, uint32_t seed) { return reverse_bits32(lk_permute(reverse_bits32(x), seed)); }
SRF_HD float ld_random_val01(uint32_t index, uint32_t seed, uint32_t dim) {   // random_val.cuh:262-266, dim in {0,1}
	index = owen_scramble(index, seed);
	return (float)owen_scramble(sobol01(index, dim), hash_combine(seed, dim)) * 2.3283064365386963e-10f;
}
// random_val.cuh:268-273 — offset inside the pixel; a per-launch constant
SRF_HD void ld_random_pixel_offset(uint32_t spp, float out[2]) {
	for (uint32_t a = 0; a < 2; ++a) {
		const float base = ld_random_val01(0, 0xdeadbeefu, a);
		const float cur = ld_random_val01(spp, 0xdeadbeefu, a);
		const float v = 0.5f - base + cur;
		out[a] = v - __builtin_floorf(v);
	}
}

// ------------------------------------------------------------------------------------
// bounding_box.h:145-191
// ------------------------------------------------------------------------------------
SRF_HD void aabb_ray_intersect(const Params& P, Vec3 o, Vec3 d, float* tmin_out, float* tmax_out) {
	float tmin = (P.aabb_min[0] - o.x) / d.x, tmax = (P.aabb_max[0] - o.x) / d.x;
	if (tmin > tmax) { const float s = tmin; tmin = tmax; tmax = s; }
	float tymin = (P.aabb_min[1] - o.y) / d.y, tymax = (P.aabb_max[1] - o.y) / d.y;
	if (tymin > tymax) { const float s = tymin; tymin = tymax; tymax = s; }
	if ((tmin > tymax) || (tymin > tmax)) { *tmin_out = 100000.0f; *tmax_out = 100000.0f; return; }
	if (tymin > tmin) tmin = tymin;
	if (tymax < tmax) tmax = tymax;
	float tzmin = (P.aabb_min[2] - o.z) / d.z, tzmax = (P.aabb_max[2] - o.z) / d.z;
	if (tzmin > tzmax) { const float s = tzmin; tzmin = tzmax; tzmax = s; }
	if ((tmin > tzmax) || (tzmin > tmax)) { *tmin_out = 100000.0f; *tmax_out = 100000.0f; return; }
	if (tzmin > tmin) tmin = tzmin;
	if (tzmax < tmax) tmax = tzmax;
	*tmin_out = tmin; *tmax_out = tmax;
}
SRF_HD bool aabb_contains(const Params& P, Vec3 p) {
	return p.x >= P.aabb_min[0] && p.x <= P.aabb_max[0] && p.y >= P.aabb_min[1] && p.y <= P.aabb_max[1] &&
	       p.z >= P.aabb_min[2] && p.z <= P.aabb_max[2];
}

// The stretch [t0, t1] of a ray inside a sphere, from the quadratic |o + t d - c|^2 = r^2 written around the ray's closest
// approach: t_mid = -(m.d)/(d.d), half = sqrt((m.d)^2 - (d.d)(m.m - r^2))/(d.d), m = o - c.  A ray whose line misses the
// sphere (or a direction of length zero) has no stretch.  Not in the reference, which bounds rays by the box alone.
struct SphereSpan { float t0, t1; bool hit; };
SRF_HD SphereSpan sphere_ray_span(const float sphere[4], Vec3 o, Vec3 d) {
	const Vec3 m = sub3(o, ld3(sphere));
	const float a = dot3(d, d), b = dot3(m, d), c = dot3(m, m) - sphere[3] * sphere[3];
	const float disc = b * b - a * c;
	SphereSpan sp;
	sp.hit = a > 0.f && disc >= 0.f;
	sp.t0 = sp.t1 = 0.f;
	if (sp.hit) {
		const float half = srf_sqrt(disc) / a, mid = -b / a;
		sp.t0 = mid - half; sp.t1 = mid + half;
	}
	return sp;
}
// where a march at t stands against the optional sphere: before it (nothing to find until *t_enter), inside, or past it for good
enum SphereGate : uint32_t { SPHERE_INSIDE = 0, SPHERE_BEFORE = 1, SPHERE_BEYOND = 2 };
SRF_HD SphereGate sphere_gate(const Params& P, Vec3 o, Vec3 d, float t, float* t_enter) {
	const SphereSpan sp = sphere_ray_span(P.sphere, o, d);
	if (!sp.hit || t > sp.t1) return SPHERE_BEYOND;
	if (t < sp.t0) { *t_enter = sp.t0; return SPHERE_BEFORE; }
	return SPHERE_INSIDE;
}

// ------------------------------------------------------------------------------------
// occupancy_sampler.cu:287-331 — step size
// ------------------------------------------------------------------------------------
SRF_HD float calc_dt(const Params& P, float t, float cone_angle) {
	const float ds = 1.f / (float)P.n_max_steps;
	if (P.sampling_type == SRF_SAMPLING_DISPARITY) {
		const float g_far = 1.f / P.far_distance, g_near = 1.f / P.near_distance, g0 = srf_rcp(t);
		const float g1 = ds * (g_far - g_near) + g0;
		const float t1 = srf_rcp(g1);
		float dt = t1 - t;
		if (dt < 0.f) dt = t >= P.far_distance ? 0.f : P.far_distance - t;
		return dt;
	}
	if (P.sampling_type == SRF_SAMPLING_ORIGINAL) return clamp_f(t * cone_angle, P.min_cone_stepsize, P.max_cone_stepsize);
	if (P.sampling_type == SRF_SAMPLING_LOG) {
		const float g_far = srf_logf(P.far_distance), g_near = srf_logf(P.near_distance), g0 = srf_logf(t);
		const float g1 = ds * (g_far - g_near) + g0;
		float t1 = srf_expf(g1);
		t1 = t1 < P.far_distance ? t1 : P.far_distance;
		return t1 - t;
	}
	return 0.f;
}

// ------------------------------------------------------------------------------------
// common_device.h:375-453 — position warp.  The reference's ERP case has no break
// and falls into SinusoidalProjection, which overwrites its result: both values
// select the sinusoidal formula.  Mixed precision as in the source: the float
// products are widened to double by the M_1_PI factor and narrowed on store.
// ------------------------------------------------------------------------------------
SRF_HD Vec3 warp_sinusoidal(Vec3 pos) {
	const Vec3 p = shift3(pos, -0.5f);
	const float mag = len3(p);
	const float inv = srf_rcp(mag);   // 1.f / mag, same rounding
	const float theta = srf_atan2f(p.y, p.x);
	const float phi = srf_asinf(p.z * inv);
	float rad = (mag <= 1.f) ? mag : (2.f - inv);
	rad *= 0.5f;
	const float tc = theta * srf_cosf(phi);
	Vec3 w;
	w.x = (float)((double)tc * SRF_M_1_PI_D * 0.5 + 0.5);
	w.y = (float)((double)phi * SRF_M_1_PI_D + 0.5);
	w.z = rad;
	return w;
}

SRF_HD Vec3 warp_position(const Params& P, Vec3 pos) {
	switch (P.warping_type) {
	case SRF_WARP_ERP:
	case SRF_WARP_SINUSOIDAL:
		return warp_sinusoidal(pos);
	case SRF_WARP_NGP:
		return mk3((pos.x - P.aabb_min[0]) / (P.aabb_max[0] - P.aabb_min[0]),
		           (pos.y - P.aabb_min[1]) / (P.aabb_max[1] - P.aabb_min[1]),
		           (pos.z - P.aabb_min[2]) / (P.aabb_max[2] - P.aabb_min[2]));
	case SRF_WARP_MIPNERF360: {
		const Vec3 x = scale3(shift3(pos, -0.5f), 2.f);
		const float m = len3(x), mi = 1.f / m;
		const Vec3 z = (m <= 1.f) ? x : scale3(x, (2.f - mi) * mi);
		return shift3(scale3(z, 0.25f), 0.5f);
	}
	case SRF_WARP_DONERF: {
		const float dmax = len3(mk3(P.aabb_max[0] - P.aabb_min[0], P.aabb_max[1] - P.aabb_min[1], P.aabb_max[2] - P.aabb_min[2]));
		const Vec3 x = shift3(pos, -0.5f);
		const float m = len3(x);
		Vec3 z = x;
		if (m != 0.f) { const float s = srf_sqrt(m * dmax); z = mk3(x.x / s, x.y / s, x.z / s); }
		return shift3(scale3(z, 0.5f), 0.5f);
	}
	case SRF_WARP_SIGMOID:
		return mk3(logistic_f(pos.x - 0.5f), logistic_f(pos.y - 0.5f), logistic_f(pos.z - 0.5f));
	}
	return mk3(0.f, 0.f, 0.f);
}

// common_device.h:455-526 — inverse warp (ERP falls through to the sinusoidal inverse likewise)
SRF_HD Vec3 unwarp_position(const Params& P, Vec3 w) {
	switch (P.warping_type) {
	case SRF_WARP_ERP:
	case SRF_WARP_SINUSOIDAL: {
		const float phi = (float)((double)(w.y - 0.5f) * SRF_M_PI_D);
		const float theta = (float)((double)((w.x - 0.5f) * 2.f) * SRF_M_PI_D / (double)srf_cosf(phi));
		float rad = w.z * 2.f;
		rad = (rad <= 1.f) ? rad : 1.f / (2.f - rad);
		float sp, cp, st, ct;
		srf_sincosf(phi, &sp, &cp);
		srf_sincosf(theta, &st, &ct);
		return shift3(mk3((rad * cp) * ct, (rad * cp) * st, rad * sp), 0.5f);
	}
	case SRF_WARP_NGP:
		return mk3(P.aabb_min[0] + w.x * (P.aabb_max[0] - P.aabb_min[0]),
		           P.aabb_min[1] + w.y * (P.aabb_max[1] - P.aabb_min[1]),
		           P.aabb_min[2] + w.z * (P.aabb_max[2] - P.aabb_min[2]));
	case SRF_WARP_MIPNERF360: {
		const Vec3 z = scale3(shift3(w, -0.5f), 4.f);
		const float m = len3(z), mi = 1.f / m;
		const Vec3 x = (m <= 1.f) ? z : scale3(z, (1.f / (2.f - m)) * mi);
		return shift3(scale3(x, 0.5f), 0.5f);
	}
	case SRF_WARP_DONERF: {
		const float dmax = len3(mk3(P.aabb_max[0] - P.aabb_min[0], P.aabb_max[1] - P.aabb_min[1], P.aabb_max[2] - P.aabb_min[2]));
		const Vec3 z = scale3(shift3(w, -0.5f), 2.f);
		return shift3(scale3(scale3(z, len3(z)), dmax), 0.5f);
	}
	case SRF_WARP_SIGMOID:
		return mk3(logit_f(w.x) + 0.5f, logit_f(w.y) + 0.5f, logit_f(w.z) + 0.5f);
	}
	return mk3(0.f, 0.f, 0.f);
}

SRF_HD Vec3 warp_direction(Vec3 d) { return scale3(shift3(d, 1.f), 0.5f); }   // common_device.h:528-530

// ------------------------------------------------------------------------------------
// occupancy_sampler.cu:349-469 — cascade of a point, its cell and its bit.  One
// grid size per warped axis (all equal in the reference).
// ------------------------------------------------------------------------------------
SRF_HD float centred_max(float a, float b, float c) {
	float m = srf_abs(a);
	const float ab = srf_abs(b), ac = srf_abs(c);
	if (ab > m) m = ab;
	if (ac > m) m = ac;
	return m;
}

SRF_HD uint32_t level_from_pos(const Params& P, Vec3 pos, Vec3 w) {
	const bool warped = P.griddist_type == SRF_GRID_WARPED_EXP || P.griddist_type == SRF_GRID_WARPED_RECIPROCAL;
	const bool expo = P.griddist_type == SRF_GRID_WARPED_EXP || P.griddist_type == SRF_GRID_METRIC_EXP;
	float m;
	if (warped) m = centred_max(w.x - 0.5f, w.y - 0.5f, w.z - 0.5f);
	else m = centred_max((pos.x - 0.5f) / (P.aabb_max[0] - P.aabb_min[0]), (pos.y - 0.5f) / (P.aabb_max[1] - P.aabb_min[1]),
	                     (pos.z - 0.5f) / (P.aabb_max[2] - P.aabb_min[2]));
	m *= 2.f;
	uint32_t mip = 0;
	for (; mip + 1 < P.n_cascades; ++mip) {
		const float bound = expo ? srf_exp2i(-1 - (int)mip) : 1.f / (float)(mip + 2);
		if (m > bound) break;
	}
	return P.n_cascades - mip - 1;
}

SRF_HD uint32_t cascaded_grid_idx_at(const Params& P, Vec3 pos, Vec3 w, uint32_t level) {
	const bool warped = P.griddist_type == SRF_GRID_WARPED_EXP || P.griddist_type == SRF_GRID_WARPED_RECIPROCAL;
	const bool expo = P.griddist_type == SRF_GRID_WARPED_EXP || P.griddist_type == SRF_GRID_METRIC_EXP;
	Vec3 p;
	if (warped) p = shift3(w, -0.5f);
	else {
		p = shift3(pos, -0.5f);
		p = mk3(p.x / (P.aabb_max[0] - P.aabb_min[0]), p.y / (P.aabb_max[1] - P.aabb_min[1]), p.z / (P.aabb_max[2] - P.aabb_min[2]));
	}
	const float zoom = expo ? srf_exp2i((int)(P.n_cascades - level - 1)) : (float)(P.n_cascades - level);
	p = shift3(scale3(p, zoom), 0.5f);
	const int32_t ix = clamp_i(srf_f2i(p.x * (float)P.grid_size[0]), 0, (int32_t)P.grid_size[0] - 1);
	const int32_t iy = clamp_i(srf_f2i(p.y * (float)P.grid_size[1]), 0, (int32_t)P.grid_size[1] - 1);
	const int32_t iz = clamp_i(srf_f2i(p.z * (float)P.grid_size[2]), 0, (int32_t)P.grid_size[2] - 1);
	return morton3d((uint32_t)ix, (uint32_t)iy, (uint32_t)iz);
}

// The two functions above for the WarpedSpace_Exp grid in fewer instructions, with identical results:
//  * the first mip with m > 2^(-1-mip) is read off the exponent of m = 2*max|w-0.5| (m = f*2^e, f in [0.5,1):
//    mip = -e, plus one when f == 0.5 because the comparison is strict); NaN compares false everywhere -> last mip
//  * truncation followed by an integer clamp to [0, N-1] equals a float clamp to [0, N-1] followed by
//    truncation (values in (-1,0) truncate to 0, values in (N-1, N) to N-1, NaN clamps to 0)
SRF_HD uint32_t level_warped_exp(const Params& P, Vec3 w) {
	const float m = centred_max(w.x - 0.5f, w.y - 0.5f, w.z - 0.5f) * 2.f;
	const uint32_t last = P.n_cascades - 1;
	if (!(m == m)) return 0;   // mip = last
	const uint32_t u = srf_f2u(m);
	const int32_t e = (int32_t)(u >> 23);                 // biased exponent; m >= 0
	int32_t mip = 126 - e + ((u & 0x007fffffu) == 0u ? 1 : 0);
	if (e == 0) mip = (int32_t)last;                       // zero and subnormals are below every threshold
	mip = mip < 0 ? 0 : (mip > (int32_t)last ? (int32_t)last : mip);
	return last - (uint32_t)mip;
}

SRF_HD void cell_warped_exp(const Params& P, Vec3 w, uint32_t level, uint32_t* cx, uint32_t* cy, uint32_t* cz) {
	const float zoom = srf_exp2i((int)(P.n_cascades - level - 1));
	const float px = (w.x - 0.5f) * zoom + 0.5f, py = (w.y - 0.5f) * zoom + 0.5f, pz = (w.z - 0.5f) * zoom + 0.5f;
	const float fx = srf_min(srf_max(px * (float)P.grid_size[0], 0.f), (float)(P.grid_size[0] - 1));
	const float fy = srf_min(srf_max(py * (float)P.grid_size[1], 0.f), (float)(P.grid_size[1] - 1));
	const float fz = srf_min(srf_max(pz * (float)P.grid_size[2], 0.f), (float)(P.grid_size[2] - 1));
	*cx = (uint32_t)fx; *cy = (uint32_t)fy; *cz = (uint32_t)fz;
}
SRF_HD uint32_t grid_idx_warped_exp(const Params& P, Vec3 w, uint32_t level) {
	uint32_t x, y, z;
	cell_warped_exp(P, w, level, &x, &y, &z);
	return morton3d(x, y, z);
}

SRF_HD bool bit_at(const uint8_t* bitfield, const Params& P, uint32_t idx, uint32_t level) {
	return (bitfield[(idx >> 3) + ((P.n_cells * level) >> 3)] >> (idx & 7u)) & 1u;
}

// empty-space table (built and explained in srf_skip.h): per cascade nb^3 blocks, each with a radius in units of side0
struct SkipTable {
	const uint16_t* dist;   // NULL: no skipping
	uint32_t nb;            // blocks per axis and cascade
	uint32_t sx, sy, sz;    // cell coordinate >> s = block coordinate
	float    side0;         // block side of cascade 0 in warped units
};

SRF_HD size_t skip_index(uint32_t nb, uint32_t level, uint32_t bx, uint32_t by, uint32_t bz) {
	return (((size_t)level * nb + bz) * nb + by) * nb + bx;
}

// what one marching step looks at: cell and occupancy of the point o + t*d, and (with a table) the empty-space radius of
// the cell's block, requested together with the occupancy byte so that the two memory round trips overlap
struct Probe { Vec3 w; float dt; uint32_t level; uint32_t idx; bool occ; uint32_t radius; };
SRF_HD Probe probe_at(const Params& P, const uint8_t* bitfield, Vec3 pos, float t, float cone_angle, const SkipTable* table = nullptr) {
	Probe s;
	size_t table_index = (size_t)-1;
	s.dt = calc_dt(P, t, cone_angle);
	s.w = warp_position(P, pos);
	if (P.griddist_type == SRF_GRID_WARPED_EXP) {
		s.level = level_warped_exp(P, s.w);
		uint32_t cx, cy, cz;
		cell_warped_exp(P, s.w, s.level, &cx, &cy, &cz);
		s.idx = morton3d(cx, cy, cz);
		if (table && table->dist && bitfield) table_index = skip_index(table->nb, s.level, cx >> table->sx, cy >> table->sy, cz >> table->sz);
	} else {
		s.level = level_from_pos(P, pos, s.w);
		s.idx = cascaded_grid_idx_at(P, pos, s.w, s.level);
	}
	// both loads are issued before either result is used
	const uint32_t byte = bitfield ? bitfield[(s.idx >> 3) + ((P.n_cells * s.level) >> 3)] : 0xffu;
	s.radius = table_index != (size_t)-1 ? table->dist[table_index] : 0u;
	s.occ = ((byte >> (s.idx & 7u)) & 1u) != 0u;
	return s;
}

// ------------------------------------------------------------------------------------
// common_device.h:143-165 — camera ray through a pixel (offset: ld_random_pixel_offset,
// evaluated once per launch on the host)
// ------------------------------------------------------------------------------------
struct Camera { float m[12]; };   // column-major 3x4
SRF_HD Vec3 cam_rotate(const float* m, Vec3 v) {
	return mk3((m[0] * v.x + m[3] * v.y) + m[6] * v.z, (m[1] * v.x + m[4] * v.y) + m[7] * v.z, (m[2] * v.x + m[5] * v.y) + m[8] * v.z);
}
SRF_HD void ray_through(const float* cam, float u, float v, const int32_t res[2], const float focal[2], const float pp[2], Vec3* o, Vec3* d) {
	*o = mk3(cam[9], cam[10], cam[11]);
	const Vec3 dir = mk3((u - pp[0]) * (float)res[0] / focal[0], (v - pp[1]) * (float)res[1] / focal[1], 1.0f);
	*d = unit3(cam_rotate(cam, dir));
}

// ------------------------------------------------------------------------------------
// common_device.h:70-100 and :320-370 — colour curves and output activations
// ------------------------------------------------------------------------------------
SRF_HD float srgb_to_linear(float s) { return s <= 0.04045f ? s / 12.92f : srf_powf((s + 0.055f) / 1.055f, 2.4f); }
SRF_HD float linear_to_srgb(float l) { return l < 0.0031308f ? 12.92f * l : 1.055f * srf_powf(l, 0.41666f) - 0.055f; }

SRF_HD float act_rgb(float v, int act) {
	if (act == SRF_ACT_NONE) return v;
	if (act == SRF_ACT_RELU) return v > 0.0f ? v : 0.0f;
	if (act == SRF_ACT_LOGISTIC) return logistic_f(v);
	if (act == SRF_ACT_EXPONENTIAL) return srf_expf(clamp_f(v, -10.0f, 10.0f));
	return 0.0f;
}
SRF_HD float act_rgb_derivative(float v, int act) {
	if (act == SRF_ACT_NONE) return 1.0f;
	if (act == SRF_ACT_RELU) return v > 0.0f ? 1.0f : 0.0f;
	if (act == SRF_ACT_LOGISTIC) { const float d = logistic_f(v); return d * (1 - d); }
	if (act == SRF_ACT_EXPONENTIAL) return srf_expf(clamp_f(v, -10.0f, 10.0f));
	return 0.0f;
}
SRF_HD float act_density(float v, int act) {
	if (act == SRF_ACT_NONE) return v;
	if (act == SRF_ACT_RELU) return v > 0.0f ? v : 0.0f;
	if (act == SRF_ACT_LOGISTIC) return logistic_f(v);
	if (act == SRF_ACT_EXPONENTIAL) return srf_expf(v);
	return 0.0f;
}
SRF_HD float act_density_derivative(float v, int act) {
	if (act == SRF_ACT_NONE) return 1.0f;
	if (act == SRF_ACT_RELU) return v > 0.0f ? 1.0f : 0.0f;
	if (act == SRF_ACT_LOGISTIC) { const float d = logistic_f(v); return d * (1 - d); }
	if (act == SRF_ACT_EXPONENTIAL) return srf_expf(clamp_f(v, -15.0f, 15.0f));
	return 0.0f;
}

// ------------------------------------------------------------------------------------
// loss.cu:18-98 — per-channel loss value and derivative w.r.t. the prediction
// ------------------------------------------------------------------------------------
SRF_HD void loss_channel(int type, float target, float pred, float* loss, float* grad) {
	const float d = pred - target;
	switch (type) {
	case SRF_LOSS_RELATIVEL2: { const float f = 1.0f / (pred * pred + 1e-2f); *loss = d * d * f; *grad = 2.0f * d * f; } return;
	case SRF_LOSS_L1: *loss = srf_abs(d); *grad = srf_copysign(1.0f, d); return;
	case SRF_LOSS_MAPE: { const float f = 1.0f / (srf_abs(pred) + 1e-2f); *loss = srf_abs(d) * f; *grad = srf_copysign(f, d); } return;
	case SRF_LOSS_SMAPE: { const float f = 1.0f / (0.5f * (srf_abs(pred) + srf_abs(target)) + 1e-2f); *loss = srf_abs(d) * f; *grad = srf_copysign(f, d); } return;
	case SRF_LOSS_SMOOTHL1: {
		const float alpha = 0.1f, ad = srf_abs(d);
		*loss = ad > alpha ? (ad - 0.5f * alpha) : (0.5f / alpha * d * d);
		*grad = ad > alpha ? (d > 0 ? 1.0f : -1.0f) : (d / alpha);
	} return;
	case SRF_LOSS_LOGL1: { const float q = srf_abs(d) + 1.0f; *loss = srf_logf(q); *grad = srf_copysign(1.0f / q, d); } return;
	default: *loss = d * d; *grad = 2.0f * d; return;
	}
}

// 32-bit mix used by the table-lookup stand-in for the network
SRF_HD uint32_t mix32(uint32_t h) {
	h ^= h >> 16; h *= 0x7feb352du; h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 16;
	return h;
}

} // namespace srf
