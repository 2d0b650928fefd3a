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
