// Elementary functions with ONE definition shared by host and device code.
//
// Cell indices and early-termination counts are integers decided by the
// results of sqrt / division / atan2 / asin / cos / exp.  glibc's libm and the
// ROCm device library are each accurate but not bit-identical to one another,
// so every transcendental used on the sampling / compositing path is defined
// here as an explicit sequence of IEEE-754 binary32 operations (+, -, *, /,
// sqrt, fma, round-to-nearest-even) that both gcc (x86-64) and hipcc (gfx950)
// evaluate identically when implicit contraction is disabled
// (-ffp-contract=off on both compilers).  Polynomial coefficients for
// exp/log/sin/cos/asin are the classic Cephes single-precision sets; atan uses
// a degree-7 (in x^2) minimax fit on [0,1] (max error ~1.1 ulp).
//
// Replaces, for this path, the CUDA intrinsics the reference calls:
//   __expf            internal/render/ray_marcher.cu:71,149,179,245
//   atan2f/asinf/cosf internal/utils/common_device.h:437-443
//   sinf/cosf         internal/utils/common_device.h:510-518
//   __logf/__expf     internal/sampler/occupancy_sampler.cu:320-322
//   std::pow          internal/utils/common_device.h:70-100
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define SRF_HD __host__ __device__ inline
#else
#define SRF_HD inline
#endif

SRF_HD float srf_u2f(uint32_t u) { float f; __builtin_memcpy(&f, &u, 4); return f; }
SRF_HD uint32_t srf_f2u(float f) { uint32_t u; __builtin_memcpy(&u, &f, 4); return u; }
SRF_HD float srf_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
SRF_HD float srf_sqrt(float x) { return __builtin_sqrtf(x); }
SRF_HD float srf_abs(float x) { return __builtin_fabsf(x); }
SRF_HD float srf_rint(float x) { return __builtin_rintf(x); }
SRF_HD float srf_copysign(float m, float s) { return __builtin_copysignf(m, s); }
// fminf/fmaxf semantics of C (a NaN operand yields the other operand).
SRF_HD float srf_min(float a, float b) { return __builtin_fminf(a, b); }
SRF_HD float srf_max(float a, float b) { return __builtin_fmaxf(a, b); }
// max(0, x) with +0 for either zero and for NaN.  fmaxf leaves the sign of max(+0, -0) open (host libraries and GPU
// instructions differ); CUDA's, which the reference's fmaxf(0.0f, x) goes through, orders -0 below +0.
SRF_HD float srf_max_zero(float x) { return x > 0.0f ? x : 0.0f; }

// float -> int32 with truncation toward zero; NaN -> 0 and saturation at the
// int32 range (what a GPU convert instruction does; a bare C cast is undefined
// for those inputs on the host).
SRF_HD int32_t srf_f2i(float x) {
	if (!(x == x)) return 0;
	if (x >= 2147483648.0f) return 2147483647;
	if (x <= -2147483648.0f) return (int32_t)(-2147483647 - 1);
	return (int32_t)x;
}

// 2^e as a float for -126 <= e <= 127 (scalbnf(1.f, e) on that range).
SRF_HD float srf_exp2i(int e) { return srf_u2f((uint32_t)(e + 127) << 23); }

#define SRF_PI_F      3.14159274101257324f   /* fl(pi)   */
#define SRF_PIO2_F    1.57079637050628662f   /* fl(pi/2) */
#define SRF_PIO4_F    0.785398185253143311f  /* fl(pi/4) */
#define SRF_M_1_PI_D  0.318309886183790671537767526745028724  /* double 1/pi, as M_1_PI */
#define SRF_M_PI_D    3.14159265358979323846                  /* double pi,  as M_PI   */

// e^x.  x <= -86 returns 0 (true value < 4.5e-38), x > 88 returns +inf.
SRF_HD float srf_expf(float x) {
	if (!(x == x)) return x;
	if (x <= -86.0f) return 0.0f;
	if (x > 88.0f) return srf_u2f(0x7f800000u);
	const float k = srf_rint(x * 1.44269504088896341f);
	float r = srf_fma(k, -0.693359375f, x);
	r = srf_fma(k, 2.12194440e-4f, r);
	const float z = r * r;
	float p = 1.9875691500e-4f;
	p = srf_fma(p, r, 1.3981999507e-3f);
	p = srf_fma(p, r, 8.3334519073e-3f);
	p = srf_fma(p, r, 4.1665795894e-2f);
	p = srf_fma(p, r, 1.6666665459e-1f);
	p = srf_fma(p, r, 5.0000001201e-1f);
	p = srf_fma(p, z, r);
	p = p + 1.0f;
	const int32_t ki = (int32_t)k;   // in [-124, 127]; p in (0.70, 1.42)
	return srf_u2f(srf_f2u(p) + ((uint32_t)ki << 23));
}

// natural log for x > 0 (normal floats); x <= 0 returns -inf, NaN propagates.
SRF_HD float srf_logf(float x) {
	if (!(x == x)) return x;
	if (x <= 0.0f) return srf_u2f(0xff800000u);
	uint32_t u = srf_f2u(x);
	int32_t e = 0;
	if (u < 0x00800000u) { x = x * 8388608.0f; u = srf_f2u(x); e = -23; }   // subnormal input
	if (u >= 0x7f800000u) return x;                                          // +inf
	e += (int32_t)(u >> 23) - 126;
	float m = srf_u2f((u & 0x007fffffu) | 0x3f000000u);    // [0.5, 1)
	if (m < 0.707106781186547524f) { e -= 1; m = m + m - 1.0f; } else { m = m - 1.0f; }
	const float z = m * m;
	float y = 7.0376836292e-2f;
	y = srf_fma(y, m, -1.1514610310e-1f);
	y = srf_fma(y, m, 1.1676998740e-1f);
	y = srf_fma(y, m, -1.2420140846e-1f);
	y = srf_fma(y, m, 1.4249322787e-1f);
	y = srf_fma(y, m, -1.6668057665e-1f);
	y = srf_fma(y, m, 2.0000714765e-1f);
	y = srf_fma(y, m, -2.4999993993e-1f);
	y = srf_fma(y, m, 3.3333331174e-1f);
	y = y * m * z;
	const float fe = (float)e;
	y = srf_fma(fe, -2.12194440e-4f, y);
	y = srf_fma(z, -0.5f, y);
	float r = m + y;
	r = srf_fma(fe, 0.693359375f, r);
	return r;
}

// x^y for x >= 0 as exp(y*log(x)); x <= 0 returns 0 (the sRGB curves only call
// it on non-negative arguments).
SRF_HD float srf_powf(float x, float y) {
	if (!(x > 0.0f)) return (x == x) ? 0.0f : x;
	return srf_expf(y * srf_logf(x));
}

// kernels on |x| <= pi/4
SRF_HD float srf_sin_k(float x) {
	const float z = x * x;
	float p = -1.9515295891e-4f;
	p = srf_fma(p, z, 8.3321608736e-3f);
	p = srf_fma(p, z, -1.6666654611e-1f);
	return srf_fma(p * z, x, x);
}
SRF_HD float srf_cos_k(float x) {
	const float z = x * x;
	float p = 2.443315711809948e-5f;
	p = srf_fma(p, z, -1.388731625493765e-3f);
	p = srf_fma(p, z, 4.166664568298827e-2f);
	p = p * z * z;
	p = srf_fma(z, -0.5f, p);
	return p + 1.0f;
}

// sin and cos with three-term Cody-Waite reduction by pi/4 octants; intended
// for |x| < ~8000 (beyond that the reduction loses bits, the result stays in
// [-1, 1]).
SRF_HD void srf_sincosf(float x, float* s_out, float* c_out) {
	if (!(x == x) || srf_abs(x) > 3.0e38f) { *s_out = x - x; *c_out = x - x; return; }
	float a = srf_abs(x);
	if (a > 8388608.0f) a = 0.0f;  // no fractional bits left: define as angle 0
	uint32_t j = (uint32_t)(a * 1.27323954473516f);   // a * 4/pi
	j += (j & 1u);
	const float y = (float)j;
	float r = srf_fma(y, -0.78515625f, a);
	r = srf_fma(y, -2.4187564849853515625e-4f, r);
	r = srf_fma(y, -3.77489497744594108e-8f, r);
	const uint32_t q = (j >> 1) & 3u;   // quadrant
	const float sk = srf_sin_k(r), ck = srf_cos_k(r);
	float s, c;
	switch (q) {
		case 0:  s = sk;  c = ck;  break;
		case 1:  s = ck;  c = -sk; break;
		case 2:  s = -sk; c = -ck; break;
		default: s = -ck; c = sk;  break;
	}
	*s_out = (x < 0.0f) ? -s : s;
	*c_out = c;
}
// 1/x, correctly rounded.  Host: the IEEE quotient.  Device: for finite x whose reciprocal lies well inside the
// normal range, the hardware estimate (within an ulp) refined by one fused Newton step: the residual 1 - x*r is
// exact, and r + r*(1 - x*r) rounds to the true quotient; anything else takes the IEEE quotient.
// Equality with the IEEE quotient is checked on the device for every mantissa.
// srf_rcp_normal: the caller guarantees 1e-30 < |x| < 1e30
SRF_HD float srf_rcp_normal(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
	const float r = __builtin_amdgcn_rcpf(x);
	const float e = srf_fma(-x, r, 1.0f);
	return srf_fma(e, r, r);
#else
	return 1.0f / x;
#endif
}
SRF_HD float srf_rcp(float x) {
	const float a = srf_abs(x);
	if (a > 1.0e-30f && a < 1.0e30f) return srf_rcp_normal(x);
	return 1.0f / x;
}

// Approximate 1/x and sqrt(x) (about an ulp on the device) for bounds that carry their own safety margin;
// never used where a result reaches an output.
SRF_HD float srf_approx_rcp(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
	return __builtin_amdgcn_rcpf(x);
#else
	return 1.0f / x;
#endif
}
SRF_HD float srf_approx_sqrt(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
	return __builtin_amdgcn_sqrtf(x);
#else
	return srf_sqrt(x);
#endif
}

SRF_HD float srf_sinf(float x) { float s, c; srf_sincosf(x, &s, &c); return s; }
// cos alone: the same reduction, evaluating only the kernel the quadrant selects (bit-identical to srf_sincosf's cosine)
SRF_HD float srf_cosf(float x) {
	if (!(x == x) || srf_abs(x) > 3.0e38f) return x - x;
	float a = srf_abs(x);
	if (a > 8388608.0f) a = 0.0f;
	uint32_t j = (uint32_t)(a * 1.27323954473516f);
	j += (j & 1u);
	const float y = (float)j;
	float r = srf_fma(y, -0.78515625f, a);
	r = srf_fma(y, -2.4187564849853515625e-4f, r);
	r = srf_fma(y, -3.77489497744594108e-8f, r);
	const uint32_t q = (j >> 1) & 3u;
	const float k = (q & 1u) ? srf_sin_k(r) : srf_cos_k(r);
	return (q == 1u || q == 2u) ? -k : k;
}

// asin on [-1, 1]; arguments whose magnitude exceeds 1 (possible by one
// rounding in z * (1/r)) are clamped to +-1 instead of producing NaN.
SRF_HD float srf_asinf(float x) {
	if (!(x == x)) return x;
	float a = srf_abs(x);
	if (a > 1.0f) a = 1.0f;
	float z, s;
	const bool big = a > 0.5f;
	if (big) { z = 0.5f * (1.0f - a); s = srf_sqrt(z); }
	else     { s = a; z = a * a; }
	float p = 4.2163199048e-2f;
	p = srf_fma(p, z, 2.4181311049e-2f);
	p = srf_fma(p, z, 4.5470025998e-2f);
	p = srf_fma(p, z, 7.4953002686e-2f);
	p = srf_fma(p, z, 1.6666752422e-1f);
	float r = srf_fma(p * z, s, s);
	if (big) { r = r + r; r = SRF_PIO2_F - r; }
	return srf_copysign(r, x);
}

// atan on [0, 1]
SRF_HD float srf_atan01(float a) {
	const float z = a * a;
	float p = 2.920690924e-03f;
	p = srf_fma(p, z, -1.636792347e-02f);
	p = srf_fma(p, z, 4.321185127e-02f);
	p = srf_fma(p, z, -7.552213967e-02f);
	p = srf_fma(p, z, 1.066600457e-01f);
	p = srf_fma(p, z, -1.421105564e-01f);
	p = srf_fma(p, z, 1.999377310e-01f);
	p = srf_fma(p, z, -3.333315253e-01f);
	return srf_fma(a * z, p, a);
}

// atan2(y, x) in (-pi, pi]; atan2(0, 0) = 0 (signed like y).
SRF_HD float srf_atan2f(float y, float x) {
	if (!(x == x) || !(y == y)) return x + y;
	const float ax = srf_abs(x), ay = srf_abs(y);
	const float mx = ax > ay ? ax : ay;
	const float mn = ax > ay ? ay : ax;
	float a;
	if (mx == 0.0f) a = 0.0f;
	else if (mn == mx) a = 1.0f;     // also covers inf/inf
	else a = mn / mx;                // inf denominators give 0
	float r = srf_atan01(a);
	if (ay > ax) r = SRF_PIO2_F - r;
	if (x < 0.0f) r = SRF_PI_F - r;
	return srf_copysign(r, y);
}
