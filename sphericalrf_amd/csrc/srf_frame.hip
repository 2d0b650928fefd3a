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

// the first round's words: every pixel's ray enters the first compaction, which starts at i_steps_offset 1 (testbed.cu:521-524)
__global__ void k_round_words_init(RoundWords* w, uint32_t n_pixels) {
	RoundWords v;
	v.n_alive = n_pixels; v.n_steps = 0; v.offset = 0; v.n_elements = 0; v.next_offset = 1; v.rounds = 0; v.pad[0] = v.pad[1] = 0;
	w[0] = v;
	v.n_alive = 0;
	w[1] = v;
}

// stand-in for the network's input gradient: a second table row, centred on zero, replaces the sample's position
__global__ void __launch_bounds__(256) k_field_input_gradient(Params P, uint32_t n, float* __restrict__ coords, FieldArgs F, const uint32_t* __restrict__ n_dev) {
	if (n_dev) n = *n_dev;
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
	return srf_field_input_gradient_counted(user, nullptr, n_elements, coords, stream);
}

int srf_field_inference_counted(void* user, const uint32_t* n_elements_dev, uint32_t max_elements, const float* coords, void* rgbsigma,
                                int32_t dtype, uint32_t padded_output_width, void* stream) {
	const srf_field_inference_ctx* c = (const srf_field_inference_ctx*)user;
	SRF_REQUIRE(c && c->sampler && c->field, "srf_field_inference_counted: NULL context");
	return srf_field_eval_counted(c->sampler, c->field, n_elements_dev, max_elements, coords, rgbsigma, dtype, padded_output_width, stream);
}

int srf_field_input_gradient_counted(void* user, const uint32_t* n_elements_dev, uint32_t n_elements, float* coords, void* stream) {
	const srf_field_inference_ctx* c = (const srf_field_inference_ctx*)user;
	SRF_REQUIRE(c && c->sampler && c->field && c->field->table, "srf_field_input_gradient: NULL context");
	SRF_REQUIRE(c->field->table_size && !(c->field->table_size & (c->field->table_size - 1)), "srf_field_input_gradient: table_size must be a power of two");
	SRF_REQUIRE(c->sampler->P.griddist_type == SRF_GRID_WARPED_EXP || c->sampler->P.griddist_type == SRF_GRID_WARPED_RECIPROCAL, "srf_field_input_gradient: needs a warped-space grid type");
	if (n_elements == 0) return SRF_OK;
	SRF_REQUIRE(coords, "srf_field_input_gradient: NULL buffer");
	const FieldArgs F{c->field->table, c->field->table_size - 1, c->field->seed ^ 0x9e3779b9u};
	hipLaunchKernelGGL(k_field_input_gradient, dim3(div_up(n_elements, 256)), dim3(256), 0, (hipStream_t)stream, c->sampler->P, n_elements, coords, F, n_elements_dev);
	SRF_LAUNCH_CHECK();
	return SRF_OK;
}

// testbed.cu:488-499: two ray buffers that take turns, the buffer of finished rays, coordinates and network output of one round; then the
// loop's counters and the round words of the paced loop
struct FrameBuffers {
	srf_ray_payload* pay[2]; srf_ray_payload* hit_pay; float* col[2]; float* hit_col; float* coords; void* rgbsigma; uint32_t* counters; RoundWords* round;
};

static int frame_prepare(srf_sampler_t* s, srf_marcher_t* m, const srf_frame_args* a, const void* inference, float* frame_buffer, hipStream_t st, const char* who,
                         FrameBuffers* B, srf_render_args* ra) {
	SRF_REQUIRE(s && m && a && inference && frame_buffer, "%s: NULL argument", who);
	SRF_REQUIRE(a->resolution[0] > 0 && a->resolution[1] > 0, "%s: resolution must be positive", who);
	SRF_REQUIRE(a->padded_output_width >= 4, "%s: padded_output_width must be >= 4", who);
	SRF_REQUIRE(a->network_output_dtype == SRF_DTYPE_F16 || a->network_output_dtype == SRF_DTYPE_F32, "%s: unknown dtype", who);
	SRF_REQUIRE(a->render_mode >= SRF_RENDER_AO && a->render_mode <= SRF_RENDER_COST, "%s: unknown render mode", who);
	const uint32_t n_pixels = (uint32_t)a->resolution[0] * (uint32_t)a->resolution[1];
	const size_t pay_bytes = align_up((size_t)n_pixels * sizeof(srf_ray_payload), 256), col_bytes = align_up((size_t)n_pixels * 16, 256);
	const size_t coord_bytes = align_up((size_t)n_pixels * FRAME_MAX_STEPS * 7 * sizeof(float), 256);
	const size_t net_bytes = align_up((size_t)n_pixels * FRAME_MAX_STEPS * a->padded_output_width * (a->network_output_dtype == SRF_DTYPE_F16 ? 2 : 4), 256);
	int rc = m->frame_ws.reserve(3 * pay_bytes + 3 * col_bytes + coord_bytes + net_bytes + 512);
	if (rc != SRF_OK) return rc;
	if (!m->frame_counter_host) {
		SRF_HIP(hipHostMalloc((void**)&m->frame_counter_host, 64, hipHostMallocMapped));
		void* dev = nullptr;
		if (hipHostGetDevicePointer(&dev, m->frame_counter_host, 0) == hipSuccess) m->frame_word_dev = (unsigned long long*)((char*)dev + 8);
		else (void)hipGetLastError();
		*(volatile unsigned long long*)(m->frame_counter_host + 2) = 0ull;
	}
	char* w = (char*)m->frame_ws.ptr;
	B->pay[0] = (srf_ray_payload*)w; B->pay[1] = (srf_ray_payload*)(w + pay_bytes);
	B->hit_pay = (srf_ray_payload*)(w + 2 * pay_bytes);
	B->col[0] = (float*)(w + 3 * pay_bytes); B->col[1] = (float*)(w + 3 * pay_bytes + col_bytes);
	B->hit_col = (float*)(w + 3 * pay_bytes + 2 * col_bytes);
	B->coords = (float*)(w + 3 * pay_bytes + 3 * col_bytes);
	B->rgbsigma = w + 3 * pay_bytes + 3 * col_bytes + coord_bytes;
	B->counters = (uint32_t*)(w + 3 * pay_bytes + 3 * col_bytes + coord_bytes + net_bytes);     // [0] alive, [1] hit
	B->round = (RoundWords*)(B->counters + 64);

	// testbed.cu:502-518
	rc = fill_u32(frame_buffer, (size_t)n_pixels * 4, 0u, st);
	if (rc != SRF_OK) return rc;
	rc = srf_sampler_generate_rays_from_camera_matrix(s, a->resolution, a->focal_length, a->principal_point, a->camera_matrix, B->pay[0], a->spp, st);
	if (rc != SRF_OK) return rc;
	rc = fill_u32(B->col[0], (size_t)n_pixels * 4, 0u, st);
	if (rc != SRF_OK) return rc;
	rc = fill_u32(B->counters + 1, 1, 0u, st);
	if (rc != SRF_OK) return rc;

	ra->padded_output_width = a->padded_output_width;
	ra->density_activation = a->density_activation; ra->rgb_activation = a->rgb_activation; ra->render_mode = a->render_mode;
	for (int k = 0; k < 12; ++k) ra->camera_matrix[k] = a->camera_matrix[k];
	ra->depth_scale = a->depth_scale;
	ra->network_output_dtype = a->network_output_dtype;
	ra->n_rays = ra->n_steps = ra->i_steps_offset = 0;
	return SRF_OK;
}

// the count that the compaction stamped `stamp` stored into host memory, if it has arrived
static bool frame_word_seen(const srf_marcher_t* m, uint32_t stamp, uint32_t* count) {
	const unsigned long long v = *(const volatile unsigned long long*)(m->frame_counter_host + 2);
	if ((uint32_t)(v >> 32) != stamp) return false;
	*count = (uint32_t)v;
	return true;
}

int srf_render_frame(srf_sampler_t* s, srf_marcher_t* m, const srf_frame_args* a, srf_inference_fn inference, void* user,
                     float* frame_buffer, uint32_t* n_iterations, void* stream) {
	hipStream_t st = (hipStream_t)stream;
	FrameBuffers B;
	srf_render_args ra;
	int rc = frame_prepare(s, m, a, (const void*)inference, frame_buffer, st, "srf_render_frame", &B, &ra);
	if (rc != SRF_OK) return rc;
	if (a->render_mode == SRF_RENDER_NORMALS && !a->input_gradient)
		SRF_FAIL(SRF_ERR_UNSUPPORTED, "srf_render_frame: Normals mode composites the density's input gradient (internal/testbed.cu:558-560); args->input_gradient must supply it");
	const uint32_t n_pixels = (uint32_t)a->resolution[0] * (uint32_t)a->resolution[1];
	uint32_t offset = 1, dbi = 0, n_alive = n_pixels, iters = 0;
	while (offset < FRAME_MARCH_ITER) {       // testbed.cu:526-597
		const uint32_t prev = dbi % 2, cur = (dbi + 1) % 2;
		++dbi;
		const uint32_t stamp = ++m->frame_stamp;
		rc = compact_rays(m, n_alive, B.pay[prev], B.col[prev], B.pay[cur], B.col[cur], B.hit_pay, B.hit_col, B.counters, B.counters + 1, true, st, m->frame_word_dev, stamp);
		if (rc != SRF_OK) return rc;
		// the host decides the size of the next round, as the reference does (:540-541).  The compaction's last block stores the
		// count, stamped with this call's number, straight into host memory; the host watches that word instead of queueing a copy
		// and waiting for the stream to drain.  Should the word not arrive although the stream has run dry, the copy does it.
		bool seen = false;
		if (m->frame_word_dev) {
			for (uint32_t spins = 1; !seen; ++spins) {
				seen = frame_word_seen(m, stamp, &n_alive);
				if (!seen && (spins & 0xfffu) == 0u && hipStreamQuery(st) != hipErrorNotReady) {
					seen = frame_word_seen(m, stamp, &n_alive);
					break;
				}
			}
			(void)hipGetLastError();
		}
		if (!seen) {
			SRF_HIP(hipMemcpyAsync(m->frame_counter_host, B.counters, 4, hipMemcpyDeviceToHost, st));
			SRF_HIP(hipStreamSynchronize(st));
			n_alive = *m->frame_counter_host;
		}
		if (n_alive == 0) break;
		++iters;
		uint32_t n_steps = n_pixels / n_alive;
		n_steps = n_steps < FRAME_MIN_STEPS ? FRAME_MIN_STEPS : (n_steps > FRAME_MAX_STEPS ? FRAME_MAX_STEPS : n_steps);
		rc = srf_sampler_generate_coords_from_rays(s, n_alive, n_steps, B.pay[cur], B.coords, st);
		if (rc != SRF_OK) return rc;
		rc = inference(user, n_alive * n_steps, B.coords, B.rgbsigma, a->network_output_dtype, a->padded_output_width, st);
		if (rc != SRF_OK) { if (rc > 0) SRF_FAIL(SRF_ERR_INVALID, "srf_render_frame: the inference callback returned %d", rc); return rc; }
		if (a->render_mode == SRF_RENDER_NORMALS) {       // testbed.cu:558-560
			rc = a->input_gradient(a->input_gradient_user, n_alive * n_steps, B.coords, st);
			if (rc != SRF_OK) { if (rc > 0) SRF_FAIL(SRF_ERR_INVALID, "srf_render_frame: the input gradient callback returned %d", rc); return rc; }
		}
		ra.n_rays = n_alive; ra.n_steps = n_steps; ra.i_steps_offset = offset;
		rc = srf_marcher_volume_rendering(m, s, &ra, B.pay[cur], B.col[cur], B.coords, B.rgbsigma, st);
		if (rc != SRF_OK) return rc;
		offset += n_steps;
	}
	SRF_HIP(hipMemcpyAsync(m->frame_counter_host, B.counters + 1, 4, hipMemcpyDeviceToHost, st));
	SRF_HIP(hipStreamSynchronize(st));
	const uint32_t n_hit = *m->frame_counter_host;
	rc = srf_shade(n_hit, B.hit_col, B.hit_pay, frame_buffer, a->render_mode, m->cfg.train_in_linear_color, st);     // testbed.cu:603-611
	if (rc != SRF_OK) return rc;
	if (n_iterations) *n_iterations = iters;
	return SRF_OK;
}

int srf_render_frame_paced(srf_sampler_t* s, srf_marcher_t* m, const srf_frame_args* a, srf_inference_counted_fn inference, void* user,
                           srf_input_gradient_counted_fn input_gradient, void* input_gradient_user,
                           float* frame_buffer, uint32_t* n_iterations, void* stream) {
	hipStream_t st = (hipStream_t)stream;
	FrameBuffers B;
	srf_render_args ra;
	int rc = frame_prepare(s, m, a, (const void*)inference, frame_buffer, st, "srf_render_frame_paced", &B, &ra);
	if (rc != SRF_OK) return rc;
	if (a->render_mode == SRF_RENDER_NORMALS && !input_gradient)
		SRF_FAIL(SRF_ERR_UNSUPPORTED, "srf_render_frame_paced: Normals mode composites the density's input gradient (internal/testbed.cu:558-560); input_gradient must supply it");
	SRF_REQUIRE(m->frame_word_dev, "srf_render_frame_paced: host memory that the device can write is not available; use srf_render_frame");
	const uint32_t n_pixels = (uint32_t)a->resolution[0] * (uint32_t)a->resolution[1];
	hipLaunchKernelGGL(k_round_words_init, dim3(1), dim3(1), 0, st, B.round, n_pixels);
	SRF_LAUNCH_CHECK();
	// How far the host may run ahead of the last count it has seen.  Every round past the end of the frame costs six launches that
	// return at once; every round the host is NOT ahead costs the device an idle gap.
	constexpr uint32_t RUN_AHEAD = 4;
	const uint32_t first_stamp = m->frame_stamp + 1;
	uint32_t bound = n_pixels;         // no more rays than this are alive (the last count seen; counts only fall)
	uint32_t seen_rounds = 0;          // rounds whose count has been seen
	uint32_t launched = 0;
	bool finished = false;
	while (!finished && launched < FRAME_MARCH_ITER) {      // (the device ends the loop by the offset, as testbed.cu:526 does; this only bounds the host)
		// what has arrived so far: the newest stamp of this frame
		for (uint32_t spins = 1;; ++spins) {
			const unsigned long long v = *(const volatile unsigned long long*)(m->frame_counter_host + 2);
			const uint32_t k = (uint32_t)(v >> 32) - first_stamp;
			if (k < launched && k + 1 > seen_rounds) { seen_rounds = k + 1; bound = (uint32_t)v; }
			if (bound == 0 && seen_rounds) { finished = true; break; }
			if (launched - seen_rounds < RUN_AHEAD) break;
			if ((spins & 0xfffu) == 0u && hipStreamQuery(st) != hipErrorNotReady) {      // the stream has run dry: the words of everything launched are there, or never come
				(void)hipGetLastError();
				const unsigned long long v2 = *(const volatile unsigned long long*)(m->frame_counter_host + 2);
				if ((uint32_t)(v2 >> 32) - first_stamp + 1 == launched) { seen_rounds = launched; bound = (uint32_t)v2; finished = bound == 0; break; }
				SRF_FAIL(SRF_ERR_HIP, "srf_render_frame_paced: the count of round %u never reached host memory", launched);
			}
		}
		if (finished) break;
		const uint32_t prev = launched % 2, cur = (launched + 1) % 2;
		const RoundWords* in = B.round + prev;
		RoundWords* out = B.round + cur;
		const uint32_t stamp = ++m->frame_stamp;
		rc = compact_rays_paced(m, bound, n_pixels, in, out, B.pay[prev], B.col[prev], B.pay[cur], B.col[cur], B.hit_pay, B.hit_col, B.counters + 1, st, m->frame_word_dev, stamp);
		if (rc != SRF_OK) return rc;
		++launched;
		rc = generate_coords_paced(s, bound, out, B.pay[cur], B.coords, st);
		if (rc != SRF_OK) return rc;
		// n_alive * n_steps never exceeds the number of pixels (n_steps is at most n_pixels / n_alive, or 1)
		const uint32_t max_elements = bound <= n_pixels / FRAME_MAX_STEPS ? bound * FRAME_MAX_STEPS : n_pixels;
		rc = inference(user, &out->n_elements, max_elements, B.coords, B.rgbsigma, a->network_output_dtype, a->padded_output_width, st);
		if (rc != SRF_OK) { if (rc > 0) SRF_FAIL(SRF_ERR_INVALID, "srf_render_frame_paced: the inference callback returned %d", rc); return rc; }
		if (a->render_mode == SRF_RENDER_NORMALS) {       // testbed.cu:558-560
			rc = input_gradient(input_gradient_user, &out->n_elements, max_elements, B.coords, st);
			if (rc != SRF_OK) { if (rc > 0) SRF_FAIL(SRF_ERR_INVALID, "srf_render_frame_paced: the input gradient callback returned %d", rc); return rc; }
		}
		rc = volume_rendering_paced(m, s, &ra, bound, out, B.pay[cur], B.col[cur], B.coords, B.rgbsigma, st);
		if (rc != SRF_OK) return rc;
	}
	rc = shade_counted(n_pixels, B.counters + 1, B.hit_col, B.hit_pay, frame_buffer, a->render_mode, m->cfg.train_in_linear_color, st);     // testbed.cu:603-611
	if (rc != SRF_OK) return rc;
	if (n_iterations) {
		SRF_HIP(hipMemcpyAsync(m->frame_counter_host, &B.round[launched % 2].rounds, 4, hipMemcpyDeviceToHost, st));
		SRF_HIP(hipStreamSynchronize(st));
		*n_iterations = *m->frame_counter_host;
	}
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
