// A whole frame through the stepwise entry points, and the display post-process that follows it
// (Testbed::render_frame, internal/testbed.cu:479-606; CudaRenderBuffer::accumulate / tonemap, internal/utils/render_buffer.cu:46-235).
#include "srf_internal.h"
#include "srf_bodies.h"

namespace srf {

// render_buffer.cu:46-85 — running mean of the frames of one view; the frame enters in the buffer's colour space
__global__ void __launch_bounds__(256) k_accumulate(uint32_t n_pixels, const Float4* __restrict__ frame, Float4* __restrict__ acc, float sample_count, int32_t color_space) {
	const uint32_t i = blockIdx.x * 256u + threadIdx.x;
	if (i < n_pixels) acc[i] = accumulate_body(frame[i], acc[i], sample_count, color_space);
}

// render_buffer.cu:142-178 — exposure, background, tone curve, output encoding
__global__ void __launch_bounds__(256) k_tonemap(uint32_t n_pixels, TonemapArgs A, const Float4* __restrict__ acc, Float4* __restrict__ out) {
	const uint32_t i = blockIdx.x * 256u + threadIdx.x;
	if (i < n_pixels) out[i] = tonemap_body(acc[i], A);
}

// stand-in for the network's input gradient: a second table row, centred on zero, replaces the sample's position
__global__ void __launch_bounds__(256) k_field_input_gradient(Params P, uint32_t n, float* __restrict__ coords, FieldArgs F) {
	const uint32_t i = blockIdx.x * 256u + threadIdx.x;
	if (i >= n) return;
	float* c = coords + 7 * (size_t)i;
	const Float4 row = *(const Float4*)(F.table + 4 * (size_t)field_row(P, ld3(c), F));
	c[0] = row.x - 0.5f; c[1] = row.y - 0.5f; c[2] = row.z - 0.5f;
}

} // namespace srf

using namespace srf;

extern "C" {

int srf_field_inference(void* user, uint32_t n_elements, const float* coords, void* rgbsigma, int32_t dtype, uint32_t padded_output_width, void* stream) {
	const srf_field_inference_ctx* c = (const srf_field_inference_ctx*)user;
	SRF_REQUIRE(c && c->sampler && c->field, "srf_field_inference: NULL context");
	return srf_field_eval(c->sampler, c->field, n_elements, coords, rgbsigma, dtype, padded_output_width, stream);
}

int srf_field_input_gradient(void* user, uint32_t n_elements, float* coords, void* stream) {
	const srf_field_inference_ctx* c = (const srf_field_inference_ctx*)user;
	SRF_REQUIRE(c && c->sampler && c->field && c->field->table, "srf_field_input_gradient: NULL context");
	SRF_REQUIRE(c->field->table_size && !(c->field->table_size & (c->field->table_size - 1)), "srf_field_input_gradient: table_size must be a power of two");
	SRF_REQUIRE(c->sampler->P.griddist_type == SRF_GRID_WARPED_EXP || c->sampler->P.griddist_type == SRF_GRID_WARPED_RECIPROCAL, "srf_field_input_gradient: needs a warped-space grid type");
	if (n_elements == 0) return SRF_OK;
	SRF_REQUIRE(coords, "srf_field_input_gradient: NULL buffer");
	const FieldArgs F{c->field->table, c->field->table_size - 1, c->field->seed ^ 0x9e3779b9u};
	hipLaunchKernelGGL(k_field_input_gradient, dim3(div_up(n_elements, 256)), dim3(256), 0, (hipStream_t)stream, c->sampler->P, n_elements, coords, F);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int srf_render_frame(srf_sampler_t* s, srf_marcher_t* m, const srf_frame_args* a, srf_inference_fn inference, void* user,
                     float* frame_buffer, uint32_t* n_iterations, void* stream) {
	SRF_REQUIRE(s && m && a && inference && frame_buffer, "srf_render_frame: NULL argument");
	SRF_REQUIRE(a->resolution[0] > 0 && a->resolution[1] > 0, "srf_render_frame: resolution must be positive");
	SRF_REQUIRE(a->padded_output_width >= 4, "srf_render_frame: padded_output_width must be >= 4");
	SRF_REQUIRE(a->network_output_dtype == SRF_DTYPE_F16 || a->network_output_dtype == SRF_DTYPE_F32, "srf_render_frame: unknown dtype");
	SRF_REQUIRE(a->render_mode >= SRF_RENDER_AO && a->render_mode <= SRF_RENDER_COST, "srf_render_frame: unknown render mode");
	if (a->render_mode == SRF_RENDER_NORMALS && !a->input_gradient)
		SRF_FAIL(SRF_ERR_UNSUPPORTED, "srf_render_frame: Normals mode composites the density's input gradient (internal/testbed.cu:558-560); args->input_gradient must supply it");
	hipStream_t st = (hipStream_t)stream;
	const uint32_t n_pixels = (uint32_t)a->resolution[0] * (uint32_t)a->resolution[1];
	constexpr uint32_t MIN_STEPS = 1, MAX_STEPS = 8, MARCH_ITER = 10000;       // testbed.h: MIN/MAX_STEPS_INBETWEEN_COMPACTION, MARCH_ITER
	// testbed.cu:488-499: two ray buffers that take turns, the buffer of finished rays, coordinates and network output of one round
	const size_t pay_bytes = align_up((size_t)n_pixels * sizeof(srf_ray_payload), 256), col_bytes = align_up((size_t)n_pixels * 16, 256);
	const size_t coord_bytes = align_up((size_t)n_pixels * MAX_STEPS * 7 * sizeof(float), 256);
	const size_t net_bytes = align_up((size_t)n_pixels * MAX_STEPS * a->padded_output_width * (a->network_output_dtype == SRF_DTYPE_F16 ? 2 : 4), 256);
	int rc = m->frame_ws.reserve(3 * pay_bytes + 3 * col_bytes + coord_bytes + net_bytes + 256);
	if (rc != SRF_OK) return rc;
	if (!m->frame_counter_host) {
		SRF_HIP(hipHostMalloc((void**)&m->frame_counter_host, 64, hipHostMallocMapped));
		void* dev = nullptr;
		if (hipHostGetDevicePointer(&dev, m->frame_counter_host, 0) == hipSuccess) m->frame_word_dev = (unsigned long long*)((char*)dev + 8);
		else (void)hipGetLastError();
		*(volatile unsigned long long*)(m->frame_counter_host + 2) = 0ull;
	}
	char* w = (char*)m->frame_ws.ptr;
	srf_ray_payload* pay[2] = {(srf_ray_payload*)w, (srf_ray_payload*)(w + pay_bytes)};
	srf_ray_payload* hit_pay = (srf_ray_payload*)(w + 2 * pay_bytes);
	float* col[2] = {(float*)(w + 3 * pay_bytes), (float*)(w + 3 * pay_bytes + col_bytes)};
	float* hit_col = (float*)(w + 3 * pay_bytes + 2 * col_bytes);
	float* coords = (float*)(w + 3 * pay_bytes + 3 * col_bytes);
	void* rgbsigma = w + 3 * pay_bytes + 3 * col_bytes + coord_bytes;
	uint32_t* counters = (uint32_t*)(w + 3 * pay_bytes + 3 * col_bytes + coord_bytes + net_bytes);     // [0] alive, [1] hit

	// testbed.cu:502-518
	rc = fill_u32(frame_buffer, (size_t)n_pixels * 4, 0u, st);
	if (rc != SRF_OK) return rc;
	rc = srf_sampler_generate_rays_from_camera_matrix(s, a->resolution, a->focal_length, a->principal_point, a->camera_matrix, pay[0], a->spp, st);
	if (rc != SRF_OK) return rc;
	rc = fill_u32(col[0], (size_t)n_pixels * 4, 0u, st);
	if (rc != SRF_OK) return rc;
	rc = fill_u32(counters + 1, 1, 0u, st);
	if (rc != SRF_OK) return rc;

	srf_render_args ra;
	ra.padded_output_width = a->padded_output_width;
	ra.density_activation = a->density_activation; ra.rgb_activation = a->rgb_activation; ra.render_mode = a->render_mode;
	for (int k = 0; k < 12; ++k) ra.camera_matrix[k] = a->camera_matrix[k];
	ra.depth_scale = a->depth_scale;
	ra.network_output_dtype = a->network_output_dtype;

	uint32_t offset = 1, dbi = 0, n_alive = n_pixels, iters = 0;
	while (offset < MARCH_ITER) {       // testbed.cu:526-597
		const uint32_t prev = dbi % 2, cur = (dbi + 1) % 2;
		++dbi;
		const uint32_t stamp = ++m->frame_stamp;
		rc = compact_rays(m, n_alive, pay[prev], col[prev], pay[cur], col[cur], hit_pay, hit_col, counters, counters + 1, true, st, m->frame_word_dev, stamp);
		if (rc != SRF_OK) return rc;
		// the host decides the size of the next round, as the reference does (:540-541).  The compaction's last block stores the
		// count, stamped with this call's number, straight into host memory; the host watches that word instead of queueing a copy
		// and waiting for the stream to drain.  Should the word not arrive although the stream has run dry, the copy does it.
		bool seen = false;
		if (m->frame_word_dev) {
			const volatile unsigned long long* word = (const volatile unsigned long long*)(m->frame_counter_host + 2);
			for (uint32_t spins = 1; !seen; ++spins) {
				const unsigned long long v = *word;
				if ((uint32_t)(v >> 32) == stamp) { n_alive = (uint32_t)v; seen = true; break; }
				if ((spins & 0xfffu) == 0u && hipStreamQuery(st) != hipErrorNotReady) {
					const unsigned long long v2 = *word;
					if ((uint32_t)(v2 >> 32) == stamp) { n_alive = (uint32_t)v2; seen = true; }
					break;
				}
			}
			(void)hipGetLastError();
		}
		if (!seen) {
			SRF_HIP(hipMemcpyAsync(m->frame_counter_host, counters, 4, hipMemcpyDeviceToHost, st));
			SRF_HIP(hipStreamSynchronize(st));
			n_alive = *m->frame_counter_host;
		}
		if (n_alive == 0) break;
		++iters;
		uint32_t n_steps = n_pixels / n_alive;
		n_steps = n_steps < MIN_STEPS ? MIN_STEPS : (n_steps > MAX_STEPS ? MAX_STEPS : n_steps);
		rc = srf_sampler_generate_coords_from_rays(s, n_alive, n_steps, pay[cur], coords, st);
		if (rc != SRF_OK) return rc;
		rc = inference(user, n_alive * n_steps, coords, rgbsigma, a->network_output_dtype, a->padded_output_width, st);
		if (rc != SRF_OK) { if (rc > 0) SRF_FAIL(SRF_ERR_INVALID, "srf_render_frame: the inference callback returned %d", rc); return rc; }
		if (a->render_mode == SRF_RENDER_NORMALS) {       // testbed.cu:558-560
			rc = a->input_gradient(a->input_gradient_user, n_alive * n_steps, coords, st);
			if (rc != SRF_OK) { if (rc > 0) SRF_FAIL(SRF_ERR_INVALID, "srf_render_frame: the input gradient callback returned %d", rc); return rc; }
		}
		ra.n_rays = n_alive; ra.n_steps = n_steps; ra.i_steps_offset = offset;
		rc = srf_marcher_volume_rendering(m, s, &ra, pay[cur], col[cur], coords, rgbsigma, st);
		if (rc != SRF_OK) return rc;
		offset += n_steps;
	}
	SRF_HIP(hipMemcpyAsync(m->frame_counter_host, counters + 1, 4, hipMemcpyDeviceToHost, st));
	SRF_HIP(hipStreamSynchronize(st));
	const uint32_t n_hit = *m->frame_counter_host;
	rc = srf_shade(n_hit, hit_col, hit_pay, frame_buffer, a->render_mode, m->cfg.train_in_linear_color, st);     // testbed.cu:603-611
	if (rc != SRF_OK) return rc;
	if (n_iterations) *n_iterations = iters;
	return SRF_OK;
}

int srf_frame_accumulate(const int32_t resolution[2], const float* frame_buffer, float* accumulate_buffer, uint32_t spp, int32_t color_space, void* stream) {
	SRF_REQUIRE(resolution && frame_buffer && accumulate_buffer, "srf_frame_accumulate: NULL argument");
	SRF_REQUIRE(resolution[0] > 0 && resolution[1] > 0, "srf_frame_accumulate: resolution must be positive");
	SRF_REQUIRE(color_space >= SRF_COLOR_LINEAR && color_space <= SRF_COLOR_VISPOSNEG, "srf_frame_accumulate: unknown colour space");
	const uint32_t n = (uint32_t)resolution[0] * (uint32_t)resolution[1];
	// render_buffer.cu:214-216: the first frame of a view starts from an empty buffer
	if (spp == 0) { const int rc = fill_u32(accumulate_buffer, (size_t)n * 4, 0u, (hipStream_t)stream); if (rc != SRF_OK) return rc; }
	hipLaunchKernelGGL(k_accumulate, dim3(div_up(n, 256)), dim3(256), 0, (hipStream_t)stream, n, (const Float4*)frame_buffer, (Float4*)accumulate_buffer, (float)spp, color_space);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

int srf_frame_tonemap(const int32_t resolution[2], float exposure, const float background_color[4], const float* accumulate_buffer,
                      int32_t color_space, int32_t output_color_space, int32_t tonemap_curve, float* out_rgba, void* stream) {
	SRF_REQUIRE(resolution && background_color && accumulate_buffer && out_rgba, "srf_frame_tonemap: NULL argument");
	SRF_REQUIRE(resolution[0] > 0 && resolution[1] > 0, "srf_frame_tonemap: resolution must be positive");
	SRF_REQUIRE(color_space >= SRF_COLOR_LINEAR && color_space <= SRF_COLOR_VISPOSNEG && output_color_space >= SRF_COLOR_LINEAR && output_color_space <= SRF_COLOR_VISPOSNEG,
	            "srf_frame_tonemap: unknown colour space");
	SRF_REQUIRE(tonemap_curve >= SRF_TONEMAP_IDENTITY && tonemap_curve <= SRF_TONEMAP_REINHARD, "srf_frame_tonemap: unknown tonemap curve");
	const uint32_t n = (uint32_t)resolution[0] * (uint32_t)resolution[1];
	TonemapArgs A;
	A.scale = srf_powf(2.0f, exposure);
	for (int c = 0; c < 4; ++c) A.background[c] = background_color[c];
	A.color_space = color_space; A.output_color_space = output_color_space; A.curve = tonemap_curve;
	hipLaunchKernelGGL(k_tonemap, dim3(div_up(n, 256)), dim3(256), 0, (hipStream_t)stream, n, A, (const Float4*)accumulate_buffer, (Float4*)out_rgba);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

} // extern "C"
