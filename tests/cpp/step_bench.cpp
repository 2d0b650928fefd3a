// Torch-free driver of one training step (march + compositing forward/backward) through include/srf_hip.hpp,
// for timing and for profiler runs (a process that holds nothing but this library's kernels and a few fill kernels).
//
//   step_bench <workload file> [--steps K] [--warmup W] [--rays N] [--cap C] [--only march|composite|render|grid] [--verify] [--copy-check]
//              [--cell-order] [--steady]
//
// --only render times whole frames of the workload file's cameras through srf_render_frame_fused instead (any workload).
// --only grid times the occupancy-grid maintenance of the workload's grid (Testbed::train's calls, internal/testbed.cu:343-372):
// sample_positions_from_grid, update_grid with one table density per point, update_grid_bitfield; one uniform point per cell as
// in the reference's first 256 steps, or with --steady a quarter of the cells each way; --cell-order draws the points in cell order.
//
// The workload file (written by sphericalrf_amd.scene.write_workload_file) holds the sampler configuration, the
// cameras, the occupancy bitfield and a table of (r, g, b, sigma) rows; per-sample network output and per-ray targets
// are drawn from the table by an integer hash of the sample / ray index, so every run sees the same inputs.
// It plays the role the reference's Testbed::train_nerf_step plays (internal/testbed.cu:308-418): same call order,
// same buffer sizing, the network replaced by the table.
// Prints one JSON line: sizes, milliseconds per entry point (HIP events on the stream the calls are enqueued on).
// --verify also runs the one-thread-per-ray compositing implementation on the same inputs and compares every output bit.
// --copy-check ends with three launches of a plain copy of 256 MiB (k_plain_copy reads 2^28 bytes and writes 2^28 bytes), so that
// a profiler's HBM byte counters of the same run can be scaled by what they read for a kernel of known traffic.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "srf_hip.hpp"

#define HIP_OK(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) { std::fprintf(stderr, "%s: %s\n", #expr, hipGetErrorString(e_)); std::exit(2); } } while (0)

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
	x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
	return x;
}

// reads n 16-byte words and writes them elsewhere: a kernel whose HBM traffic is known
__global__ void __launch_bounds__(256) k_plain_copy(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n) {
	for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

// float grid holding 1 where the bitfield has a bit and 0 elsewhere
__global__ void k_expand_bits(const uint8_t* __restrict__ bits, float* __restrict__ grid, uint32_t n_cells) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n_cells) grid[i] = ((bits[i >> 3] >> (i & 7u)) & 1u) ? 1.0f : 0.0f;
}

// network output of sample s: row hash(s) of the table, as 4 halfs
__global__ void k_fill_network_output(const float* __restrict__ table, uint32_t table_mask, uint32_t seed, uint32_t n, __half* __restrict__ out) {
	const uint32_t s = blockIdx.x * blockDim.x + threadIdx.x;
	if (s >= n) return;
	const float4 row = ((const float4*)table)[mix32(s ^ seed) & table_mask];
	__half* o = out + 4 * (size_t)s;
	o[0] = __float2half(row.x); o[1] = __float2half(row.y); o[2] = __float2half(row.z); o[3] = __float2half(row.w);
}

// density of grid point i: the sigma column of row hash(i) of the table, as a half
__global__ void k_fill_point_density(const float* __restrict__ table, uint32_t table_mask, uint32_t seed, uint32_t n, __half* __restrict__ out) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i < n) out[i] = __float2half(table[4 * (size_t)(mix32(i ^ seed) & table_mask) + 3]);
}

// target colour of ray i: uniform in [0, 1), alpha 1
__global__ void k_fill_targets(uint32_t seed, uint32_t n, float* __restrict__ out) {
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	if (i >= n) return;
	float4 v;
	v.x = (float)(mix32(3u * i + seed) >> 8) * (1.0f / 16777216.0f);
	v.y = (float)(mix32(3u * i + 1u + seed) >> 8) * (1.0f / 16777216.0f);
	v.z = (float)(mix32(3u * i + 2u + seed) >> 8) * (1.0f / 16777216.0f);
	v.w = 1.0f;
	((float4*)out)[i] = v;
}

struct Workload {
	srf_sampler_config cfg;
	uint32_t n_cameras;
	int32_t  res[2];
	float    focal[2];
	std::vector<float> cameras;
	std::vector<uint8_t> bitfield;
	std::vector<float> table;
};

static bool read_exact(FILE* f, void* p, size_t n) { return std::fread(p, 1, n, f) == n; }

static Workload load_workload(const char* path) {
	FILE* f = std::fopen(path, "rb");
	if (!f) { std::fprintf(stderr, "cannot open %s\n", path); std::exit(2); }
	Workload w;
	char magic[8];
	uint32_t cfg_bytes = 0, n_bits_bytes = 0, table_rows = 0;
	bool ok = read_exact(f, magic, 8) && std::memcmp(magic, "SRFWLD01", 8) == 0;
	ok = ok && read_exact(f, &cfg_bytes, 4) && cfg_bytes == sizeof(srf_sampler_config) && read_exact(f, &w.cfg, sizeof(w.cfg));
	ok = ok && read_exact(f, &w.n_cameras, 4) && read_exact(f, w.res, 8) && read_exact(f, w.focal, 8);
	if (ok) { w.cameras.resize((size_t)w.n_cameras * 12); ok = read_exact(f, w.cameras.data(), w.cameras.size() * 4); }
	ok = ok && read_exact(f, &n_bits_bytes, 4);
	if (ok) { w.bitfield.resize(n_bits_bytes); ok = read_exact(f, w.bitfield.data(), n_bits_bytes); }
	ok = ok && read_exact(f, &table_rows, 4) && table_rows > 0 && (table_rows & (table_rows - 1)) == 0;
	if (ok) { w.table.resize((size_t)table_rows * 4); ok = read_exact(f, w.table.data(), w.table.size() * 4); }
	std::fclose(f);
	if (!ok) { std::fprintf(stderr, "%s is not a workload file of this build\n", path); std::exit(2); }
	return w;
}

template <class T> static T* dev_alloc(size_t n) { T* p = nullptr; HIP_OK(hipMalloc((void**)&p, n * sizeof(T))); HIP_OK(hipMemset(p, 0, n * sizeof(T))); return p; }

struct Timer {
	hipEvent_t a, b;
	Timer() { HIP_OK(hipEventCreate(&a)); HIP_OK(hipEventCreate(&b)); }
	void start(hipStream_t s) { HIP_OK(hipEventRecord(a, s)); }
	float stop(hipStream_t s) { HIP_OK(hipEventRecord(b, s)); HIP_OK(hipEventSynchronize(b)); float ms = 0; HIP_OK(hipEventElapsedTime(&ms, a, b)); return ms; }
};

int main(int argc, char** argv) {
	if (argc < 2) { std::fprintf(stderr, "usage: step_bench <workload file> [--steps K] [--warmup W] [--rays N] [--cap C] [--only march|composite|render|grid] [--verify] [--copy-check] [--cell-order] [--steady]\n"); return 2; }
	uint32_t steps = 10, warmup = 2, n_rays = 1u << 20, cap = 1u << 24;
	bool verify = false, copy_check = false, cell_order = false, steady = false;
	std::string only;
	for (int i = 2; i < argc; ++i) {
		const std::string a = argv[i];
		auto next = [&]() -> const char* { if (i + 1 >= argc) { std::fprintf(stderr, "%s needs a value\n", a.c_str()); std::exit(2); } return argv[++i]; };
		if (a == "--steps") steps = (uint32_t)std::atoi(next());
		else if (a == "--warmup") warmup = (uint32_t)std::atoi(next());
		else if (a == "--rays") n_rays = (uint32_t)std::atoi(next());
		else if (a == "--cap") cap = (uint32_t)std::atoi(next());
		else if (a == "--only") only = next();
		else if (a == "--verify") verify = true;
		else if (a == "--copy-check") copy_check = true;
		else if (a == "--cell-order") cell_order = true;
		else if (a == "--steady") steady = true;
		else { std::fprintf(stderr, "unknown option %s\n", a.c_str()); return 2; }
	}
	const Workload w = load_workload(argv[1]);
	hipStream_t st = nullptr;   // the default stream: every call below is enqueued on it

	try {
		srf::OccupancySampler sampler(w.cfg);
		const srf_sampler_info info = sampler.members();
		if ((size_t)info.n_total_elements != w.bitfield.size() * 8) { std::fprintf(stderr, "bitfield size does not match the grid\n"); return 2; }
		// the bitfield enters the way a snapshot does (internal/testbed.cu:167-168): as a float grid, then update_grid_bitfield
		uint8_t* d_bits = dev_alloc<uint8_t>(w.bitfield.size());
		HIP_OK(hipMemcpy(d_bits, w.bitfield.data(), w.bitfield.size(), hipMemcpyHostToDevice));
		float* d_grid = dev_alloc<float>(info.n_total_elements);
		hipLaunchKernelGGL(k_expand_bits, dim3((info.n_total_elements + 255) / 256), dim3(256), 0, st, d_bits, d_grid, info.n_total_elements);
		sampler.set_density_grid(d_grid, st);
		sampler.update_grid_bitfield(st);
		HIP_OK(hipStreamSynchronize(st));
		HIP_OK(hipFree(d_grid));
		{
			std::vector<uint8_t> back(w.bitfield.size());
			HIP_OK(hipMemcpy(back.data(), sampler.density_grid_bitfield(), back.size(), hipMemcpyDeviceToHost));
			if (std::memcmp(back.data(), w.bitfield.data(), back.size()) != 0) { std::fprintf(stderr, "rebuilt bitfield differs from the file's\n"); return 1; }
		}
		HIP_OK(hipFree(d_bits));

		srf_marcher_config mc = srf::RayMarcher::default_config();
		mc.train_with_random_bg_color = 0;
		mc.train_in_linear_color = 1;
		mc.transmittance_threshold = 1e-4f;
		srf::RayMarcher marcher(mc);

		if (only == "grid") {
			sampler.set_grid_sample_order(cell_order);
			srf_pcg32 grid_rng{0x853c49e6748fea9bULL, 0xda3e39cb94b95bdbULL};
			const float pp[2] = {0.5f, 0.5f};
			sampler.init(1, w.res, w.focal, pp, nullptr, grid_rng, st);       // a grid without a camera mask starts from zero (occupancy_sampler.cu:946-978)
			const uint32_t n_total = info.n_total_elements;
			const uint32_t n_uni = steady ? n_total / 4 : n_total, n_non = steady ? n_total / 4 : 0u, n_points = n_uni + n_non;
			float* pos = dev_alloc<float>((size_t)n_points * 3);
			uint32_t* idx = dev_alloc<uint32_t>(n_points);
			__half* dens = dev_alloc<__half>(n_points);
			float* d_table = dev_alloc<float>(w.table.size());
			HIP_OK(hipMemcpy(d_table, w.table.data(), w.table.size() * 4, hipMemcpyHostToDevice));
			hipLaunchKernelGGL(k_fill_point_density, dim3((n_points + 255) / 256), dim3(256), 0, st, d_table, (uint32_t)(w.table.size() / 4 - 1), 49u, n_points, dens);
			HIP_OK(hipStreamSynchronize(st));
			Timer tm;
			double ms[3] = {0, 0, 0};
			for (uint32_t k = 0; k < warmup + steps; ++k) {
				tm.start(st);
				sampler.sample_positions_from_grid(n_uni, n_non, pos, idx, st);
				const float t0 = tm.stop(st);
				tm.start(st);
				sampler.update_grid(n_points, 1, dens, SRF_DTYPE_F16, idx, SRF_ACT_NONE, st);
				const float t1 = tm.stop(st);
				tm.start(st);
				sampler.update_grid_bitfield(st);
				const float t2 = tm.stop(st);
				if (k >= warmup) { ms[0] += t0; ms[1] += t1; ms[2] += t2; }
			}
			if (copy_check) {
				const size_t n16 = (size_t)1 << 24;
				uint4* src = dev_alloc<uint4>(n16);
				uint4* dst = dev_alloc<uint4>(n16);
				HIP_OK(hipMemset(src, 1, n16 * 16));
				for (int k = 0; k < 3; ++k) hipLaunchKernelGGL(k_plain_copy, dim3(16384), dim3(256), 0, st, (const uint4*)src, dst, n16);
				HIP_OK(hipStreamSynchronize(st));
			}
			std::printf("{\"cells\": %u, \"points\": %u, \"cell_order\": %s, \"steady_state\": %s, \"steps\": %u, \"sample_positions_ms\": %.4f, \"update_grid_ms\": %.4f, "
			            "\"update_grid_bitfield_ms\": %.4f, \"update_grid_gbs\": %.1f, \"bitfield_gbs\": %.1f}\n", n_total, n_points, cell_order ? "true" : "false",
			            steady ? "true" : "false", steps, ms[0] / steps, ms[1] / steps, ms[2] / steps, 12.0 * n_total / (ms[1] / steps * 1e-3) / 1e9,
			            4.125 * n_total / (ms[2] / steps * 1e-3) / 1e9);
			return 0;
		}

		if (only == "render") {
			// frames of the workload's cameras in turn through the one-launch frame, the table standing in for the network
			const uint32_t n_pixels = (uint32_t)w.res[0] * (uint32_t)w.res[1];
			float* frame = dev_alloc<float>((size_t)n_pixels * 4);
			uint32_t* n_samples = dev_alloc<uint32_t>(n_pixels);
			float* d_table = dev_alloc<float>(w.table.size());
			HIP_OK(hipMemcpy(d_table, w.table.data(), w.table.size() * 4, hipMemcpyHostToDevice));
			srf_field field{d_table, (uint32_t)(w.table.size() / 4), 1000u};
			const float pp[2] = {0.5f, 0.5f};
			Timer tm;
			double ms = 0;
			for (uint32_t k = 0; k < warmup + steps; ++k) {
				tm.start(st);
				const int rc = srf_render_frame_fused(sampler.handle(), marcher.handle(), &field, w.res, w.focal, pp, &w.cameras[(size_t)(k % w.n_cameras) * 12], 0, frame, n_samples, st);
				if (rc != SRF_OK) { std::fprintf(stderr, "srf_render_frame_fused: %s\n", srf_last_error()); return 1; }
				const float t = tm.stop(st);
				if (k >= warmup) ms += t;
			}
			std::vector<uint32_t> ns(n_pixels);
			HIP_OK(hipMemcpy(ns.data(), n_samples, (size_t)n_pixels * 4, hipMemcpyDeviceToHost));
			unsigned long long total = 0;
			for (uint32_t v : ns) total += v;
			std::printf("{\"frames\": %u, \"resolution\": [%d, %d], \"render_ms\": %.4f, \"composited_samples_last_frame\": %llu}\n", steps, w.res[0], w.res[1], ms / steps, total);
			return 0;
		}

		float* d_cams = dev_alloc<float>(w.cameras.size());
		HIP_OK(hipMemcpy(d_cams, w.cameras.data(), w.cameras.size() * 4, hipMemcpyHostToDevice));
		srf_dataset ds{};
		ds.n_images = w.n_cameras;
		ds.image_resolution[0] = w.res[0]; ds.image_resolution[1] = w.res[1];
		ds.focal_length[0] = w.focal[0]; ds.focal_length[1] = w.focal[1];
		ds.principal_point[0] = 0.5f; ds.principal_point[1] = 0.5f;
		ds.xforms = d_cams;

		float* rays = dev_alloc<float>((size_t)n_rays * 6);
		float* rays_rgba = dev_alloc<float>((size_t)n_rays * 4);
		uint32_t* ray_idx = dev_alloc<uint32_t>((size_t)n_rays * 2);
		uint32_t* ray_idx_in = dev_alloc<uint32_t>((size_t)n_rays * 2);
		float* sample_t = dev_alloc<float>(cap);
		float* sample_dt = dev_alloc<float>(cap);
		uint32_t* sample_cell = dev_alloc<uint32_t>(cap);
		uint32_t* counters = dev_alloc<uint32_t>(4);   // rays kept, samples, compacted samples
		__half* net = dev_alloc<__half>((size_t)cap * 4);
		float* targets = dev_alloc<float>((size_t)n_rays * 4);
		float* dloss = dev_alloc<float>((size_t)cap * 4);
		float* loss = dev_alloc<float>(n_rays);
		float* rgb_out = dev_alloc<float>((size_t)n_rays * 3);
		float* d_table = dev_alloc<float>(w.table.size());
		HIP_OK(hipMemcpy(d_table, w.table.data(), w.table.size() * 4, hipMemcpyHostToDevice));
		hipLaunchKernelGGL(k_fill_network_output, dim3((cap + 255) / 256), dim3(256), 0, st, d_table, (uint32_t)(w.table.size() / 4 - 1), 47u, cap, net);
		hipLaunchKernelGGL(k_fill_targets, dim3((n_rays + 255) / 256), dim3(256), 0, st, 48u, n_rays, targets);
		HIP_OK(hipStreamSynchronize(st));

		srf_pcg32 rng{0x853c49e6748fea9bULL, 0xda3e39cb94b95bdbULL};
		srf_loss_args la{};
		la.n_rays = n_rays; la.n_max_compacted_coords = cap; la.padded_output_width = 4;
		la.rgb_activation = SRF_ACT_NONE; la.density_activation = SRF_ACT_NONE; la.loss_type = SRF_LOSS_L2; la.loss_scale = 128.0f;
		la.min_optical_thickness = info.min_optical_thickness; la.use_grid = 1;
		la.color_space = SRF_COLOR_LINEAR; la.rng = rng;
		la.network_output_dtype = SRF_DTYPE_F16; la.dloss_dtype = SRF_DTYPE_F32; la.dt_stride = 1;

		uint32_t shift = 0;
		auto march = [&]() {
			HIP_OK(hipMemsetAsync(counters, 0, 16, st));
			sampler.sample_coords_from_dataset(n_rays, shift, cap, ds, rays, rays_rgba, counters + 0, ray_idx, nullptr, counters + 1, rng, st,
			                                   sample_t, sample_dt, sample_cell);
		};
		auto composite = [&]() {
			// the compositing call rewrites (count, offset) per ray in place: keep the march's records to start every call from them
			HIP_OK(hipMemcpyAsync(ray_idx, ray_idx_in, (size_t)n_rays * 8, hipMemcpyDeviceToDevice, st));
			HIP_OK(hipMemsetAsync(counters + 2, 0, 4, st));
		};
		auto composite_call = [&]() {
			marcher.volume_rendering_with_loss_and_gradient(la, targets, counters + 0, ray_idx, sample_dt, nullptr, nullptr, counters + 2, net, dloss, loss,
			                                                sampler.density_grid_mean(), st, rgb_out);
		};

		march();
		HIP_OK(hipStreamSynchronize(st));
		HIP_OK(hipMemcpy(ray_idx_in, ray_idx, (size_t)n_rays * 8, hipMemcpyDeviceToDevice));
		uint32_t h_counters[4];
		HIP_OK(hipMemcpy(h_counters, counters, 16, hipMemcpyDeviceToHost));
		const uint32_t n_kept = h_counters[0], n_samples = h_counters[1];

		Timer tm;
		double march_ms = 0, comp_ms = 0;
		const bool do_march = only.empty() || only == "march", do_comp = only.empty() || only == "composite";
		for (uint32_t k = 0; k < warmup + steps; ++k) {
			if (do_march) {
				tm.start(st);
				march();
				const float ms = tm.stop(st);
				if (k >= warmup) march_ms += ms;
			}
			if (do_comp) {
				composite();
				tm.start(st);
				composite_call();
				const float ms = tm.stop(st);
				if (k >= warmup) comp_ms += ms;
			}
		}
		marcher.sync_check(st);
		HIP_OK(hipMemcpy(h_counters, counters, 16, hipMemcpyDeviceToHost));
		const uint32_t n_compacted = h_counters[2];

		int verify_rc = -1;
		if (verify) {
			const size_t n_out = (size_t)n_compacted * 4;
			std::vector<float> a(n_out), b(n_out), la_(n_rays), lb_(n_rays), ca((size_t)n_rays * 3), cb((size_t)n_rays * 3);
			std::vector<uint32_t> ia((size_t)n_rays * 2), ib((size_t)n_rays * 2);
			auto grab = [&](srf::RayMarcher& mm, std::vector<float>& g, std::vector<float>& l, std::vector<float>& c, std::vector<uint32_t>& idx) {
				HIP_OK(hipMemset(dloss, 0, (size_t)cap * 16)); HIP_OK(hipMemset(loss, 0, (size_t)n_rays * 4)); HIP_OK(hipMemset(rgb_out, 0, (size_t)n_rays * 12));
				composite();
				mm.volume_rendering_with_loss_and_gradient(la, targets, counters + 0, ray_idx, sample_dt, nullptr, nullptr, counters + 2, net, dloss, loss,
				                                           sampler.density_grid_mean(), st, rgb_out);
				mm.sync_check(st);
				HIP_OK(hipMemcpy(g.data(), dloss, n_out * 4, hipMemcpyDeviceToHost));
				HIP_OK(hipMemcpy(l.data(), loss, (size_t)n_rays * 4, hipMemcpyDeviceToHost));
				HIP_OK(hipMemcpy(c.data(), rgb_out, (size_t)n_rays * 12, hipMemcpyDeviceToHost));
				HIP_OK(hipMemcpy(idx.data(), ray_idx, (size_t)n_rays * 8, hipMemcpyDeviceToHost));
			};
			grab(marcher, a, la_, ca, ia);
			setenv("SRF_COMPOSITE_IMPL", "unfused", 1);     // read when a marcher is created
			srf::RayMarcher per_ray(mc);
			unsetenv("SRF_COMPOSITE_IMPL");
			grab(per_ray, b, lb_, cb, ib);
			uint32_t after = 0;
			HIP_OK(hipMemcpy(&after, counters + 2, 4, hipMemcpyDeviceToHost));
			const bool same = after == n_compacted && std::memcmp(a.data(), b.data(), n_out * 4) == 0 && std::memcmp(la_.data(), lb_.data(), (size_t)n_rays * 4) == 0 &&
			                  std::memcmp(ca.data(), cb.data(), (size_t)n_rays * 12) == 0 && std::memcmp(ia.data(), ib.data(), (size_t)n_rays * 8) == 0;
			verify_rc = same ? 0 : 1;
		}

		if (copy_check) {
			const size_t n_words = (size_t)1 << 24;     // 2^24 x 16 B = 256 MiB each way
			uint4* src = dev_alloc<uint4>(n_words);
			uint4* dst = dev_alloc<uint4>(n_words);
			HIP_OK(hipMemset(src, 1, n_words * 16));
			for (int k = 0; k < 3; ++k) hipLaunchKernelGGL(k_plain_copy, dim3(4096), dim3(256), 0, st, (const uint4*)src, dst, n_words);
			HIP_OK(hipStreamSynchronize(st));
			HIP_OK(hipFree(src)); HIP_OK(hipFree(dst));
		}

		const double comp_bytes = 28.0 * n_samples + 36.0 * n_kept;
		std::printf("{\"rays\": %u, \"rays_kept\": %u, \"samples\": %u, \"compacted_samples\": %u, \"steps\": %u, \"march_ms\": %.4f, \"composite_ms\": %.4f, "
		            "\"composite_algorithmic_bytes\": %.0f, \"composite_gbs\": %.1f, \"verify\": %s}\n",
		            n_rays, n_kept, n_samples, n_compacted, steps, do_march ? march_ms / steps : 0.0, do_comp ? comp_ms / steps : 0.0, comp_bytes,
		            do_comp && comp_ms > 0 ? comp_bytes / (comp_ms / steps * 1e-3) / 1e9 : 0.0, verify_rc < 0 ? "null" : (verify_rc == 0 ? "\"ok\"" : "\"MISMATCH\""));
		return verify_rc > 0 ? 1 : 0;
	} catch (const std::runtime_error& e) {
		std::fprintf(stderr, "error: %s\n", e.what());
		return 3;
	}
}
