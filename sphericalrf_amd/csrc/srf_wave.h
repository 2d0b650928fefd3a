// 64-lane wavefront and workgroup primitives (device only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace srf {

constexpr uint32_t WAVE = 64;

__device__ inline uint32_t lane_id() { return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

// inclusive prefix sum across the 64 lanes of a wave
__device__ inline uint32_t wave_inclusive_scan_u32(uint32_t v) {
	const uint32_t lane = lane_id();
	#pragma unroll
	for (uint32_t d = 1; d < WAVE; d <<= 1) {
		const uint32_t up = (uint32_t)__shfl_up((int)v, d, WAVE);
		if (lane >= d) v += up;
	}
	return v;
}

__device__ inline uint32_t wave_sum_u32(uint32_t v) {
	#pragma unroll
	for (uint32_t d = WAVE / 2; d > 0; d >>= 1) v += (uint32_t)__shfl_xor((int)v, d, WAVE);
	return v;
}

__device__ inline uint32_t wave_max_u32(uint32_t v) {
	#pragma unroll
	for (uint32_t d = WAVE / 2; d > 0; d >>= 1) { const uint32_t o = (uint32_t)__shfl_xor((int)v, d, WAVE); v = o > v ? o : v; }
	return v;
}

// ---- the same reductions without the LDS crossbar -----------------------------------------------
// __shfl* compile to ds_bpermute, which queues behind the workgroup's LDS traffic and comes back after an LDS round trip; six of
// them in a row cost a busy kernel more than a thousand cycles.  These use the vector unit's lane shuffles (DPP) inside rows of 16
// lanes and scalar reads of single lanes across rows.  To be called with all 64 lanes active.
template <int CTRL, bool BOUND_ZERO>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
	return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, BOUND_ZERO);
}
__device__ __forceinline__ uint32_t lane_value_u32(uint32_t v, uint32_t uniform_lane) {
	return (uint32_t)__builtin_amdgcn_readlane((int)v, (int)__builtin_amdgcn_readfirstlane((int)uniform_lane));
}
// the sum of all 64 lanes, the same in every lane
__device__ __forceinline__ uint32_t wave_sum_fast(uint32_t v) {
	v += dpp_u32<0xb1, false>(v);       // quad_perm [1,0,3,2]
	v += dpp_u32<0x4e, false>(v);       // quad_perm [2,3,0,1]
	v += dpp_u32<0x141, false>(v);      // row_half_mirror
	v += dpp_u32<0x140, false>(v);      // row_mirror: every lane holds its row's sum
	return (lane_value_u32(v, 0) + lane_value_u32(v, 16)) + (lane_value_u32(v, 32) + lane_value_u32(v, 48));
}
__device__ __forceinline__ uint32_t wave_max_fast(uint32_t v) {
	uint32_t o;
	o = dpp_u32<0xb1, false>(v); v = o > v ? o : v;
	o = dpp_u32<0x4e, false>(v); v = o > v ? o : v;
	o = dpp_u32<0x141, false>(v); v = o > v ? o : v;
	o = dpp_u32<0x140, false>(v); v = o > v ? o : v;
	const uint32_t a = lane_value_u32(v, 0), b = lane_value_u32(v, 16), c = lane_value_u32(v, 32), d = lane_value_u32(v, 48);
	const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
	return ab > cd ? ab : cd;
}
// inclusive prefix sum over the 64 lanes
__device__ __forceinline__ uint32_t wave_inclusive_scan_fast(uint32_t v) {
	v += dpp_u32<0x111, true>(v);       // row_shr 1, 2, 4, 8 with zeros shifted in: the scan inside every row
	v += dpp_u32<0x112, true>(v);
	v += dpp_u32<0x114, true>(v);
	v += dpp_u32<0x118, true>(v);
	const uint32_t t0 = lane_value_u32(v, 15), t1 = lane_value_u32(v, 31), t2 = lane_value_u32(v, 47);
	const uint32_t lane = lane_id();
	return v + (lane >= 16 ? t0 : 0u) + (lane >= 32 ? t1 : 0u) + (lane >= 48 ? t2 : 0u);
}
// the value of the lane below (lane 0 gets 0)
__device__ __forceinline__ uint32_t lane_below_u32(uint32_t v) { return dpp_u32<0x138, true>(v); }     // wave_shr 1

// sum over a workgroup of THREADS threads (multiple of 64); lds holds THREADS/64 words.
// Every thread receives the total.
template <uint32_t THREADS>
__device__ inline uint32_t block_sum_u32(uint32_t v, uint32_t* lds) {
	constexpr uint32_t NW = THREADS / WAVE;
	const uint32_t w = threadIdx.x / WAVE;
	const uint32_t s = wave_sum_u32(v);
	if (lane_id() == 0) lds[w] = s;
	__syncthreads();
	uint32_t total = 0;
	#pragma unroll
	for (uint32_t k = 0; k < NW; ++k) total += lds[k];
	__syncthreads();
	return total;
}

// exclusive prefix sum over a workgroup in thread order; lds holds THREADS/64 + 1 words.
template <uint32_t THREADS>
__device__ inline uint32_t block_exclusive_scan_u32(uint32_t v, uint32_t* lds, uint32_t* total_out) {
	constexpr uint32_t NW = THREADS / WAVE;
	const uint32_t w = threadIdx.x / WAVE;
	const uint32_t incl = wave_inclusive_scan_u32(v);
	if (lane_id() == WAVE - 1) lds[w] = incl;
	__syncthreads();
	uint32_t before = 0, total = 0;
	#pragma unroll
	for (uint32_t k = 0; k < NW; ++k) {
		const uint32_t s = lds[k];
		if (k < w) before += s;
		total += s;
	}
	__syncthreads();
	*total_out = total;
	return before + incl - v;
}

} // namespace srf
