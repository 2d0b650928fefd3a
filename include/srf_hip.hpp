// C++ face of libsrf_hip.so: two header-only classes with the names, methods and error behaviour of the
// reference's OccupancySampler (internal/sampler/occupancy_sampler.h:11-135) and RayMarcher
// (internal/render/ray_marcher.h:10-82), over the C ABI of srf_hip.h.  Where the reference takes
// tcnn::GPUMemory<T>& these take the raw device pointer (GPUMemory::data()); where it takes a
// nlohmann::json block these take the plain config struct that the JSON keys map onto one to one
// (config_from_strings() does the reference's string -> enum step, occupancy_sampler.cu:865-907,
// ray_marcher.cu:284-292, and throws std::runtime_error on unknown names exactly like it).
// Errors of the C ABI become std::runtime_error(srf_last_error()), the role CUDA_CHECK_THROW plays
// in the reference.  Nothing here touches the device itself; streams are passed through as void*.
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "srf_hip.h"

namespace srf {

inline void check(int rc) {
	if (rc != SRF_OK) throw std::runtime_error(srf_last_error());
}

namespace detail {
inline std::string lower(std::string s) {
	for (char& c : s) if (c >= 'A' && c <= 'Z') c = (char)(c - 'A' + 'a');
	return s;
}
}

// occupancy_sampler.cu:865-880
inline int32_t string_to_warping_type(const std::string& name) {
	const std::string s = detail::lower(name);
	if (s == "ngp") return SRF_WARP_NGP;
	if (s == "mipnerf360") return SRF_WARP_MIPNERF360;
	if (s == "donerf") return SRF_WARP_DONERF;
	if (s == "sigmoid") return SRF_WARP_SIGMOID;
	if (s == "erp") return SRF_WARP_ERP;
	if (s == "sinusoidalprojection") return SRF_WARP_SINUSOIDAL;
	throw std::runtime_error("Unknown warping type: " + name);
}
// occupancy_sampler.cu:882-893
inline int32_t string_to_sampling_type(const std::string& name) {
	const std::string s = detail::lower(name);
	if (s == "original") return SRF_SAMPLING_ORIGINAL;
	if (s == "disparity") return SRF_SAMPLING_DISPARITY;
	if (s == "log") return SRF_SAMPLING_LOG;
	throw std::runtime_error("Unknown sampling type: " + name);
}
// occupancy_sampler.cu:895-907 ("Exp", the constructor's own default, is not among the accepted names there either)
inline int32_t string_to_griddist_type(const std::string& name) {
	const std::string s = detail::lower(name);
	if (s == "warpedspace_exp") return SRF_GRID_WARPED_EXP;
	if (s == "warpedspace_reciprocal") return SRF_GRID_WARPED_RECIPROCAL;
	if (s == "metricspace_exp") return SRF_GRID_METRIC_EXP;
	if (s == "metricspace_reciprocal") return SRF_GRID_METRIC_RECIPROCAL;
	throw std::runtime_error("Unknown grid distribution type: " + name);
}
// ray_marcher.cu:284-292
inline int32_t string_to_regularization_type(const std::string& name) {
	const std::string s = detail::lower(name);
	if (s == "none") return SRF_REG_NONE;
	if (s == "distortion") return SRF_REG_DISTORTION;
	throw std::runtime_error("Unknown regularization type: " + name);
}

class OccupancySampler {
public:
	explicit OccupancySampler(const srf_sampler_config& config) {          // occupancy_sampler.cu:909-944
		check(srf_sampler_create(&config, &m_impl));
		refresh();
	}
	~OccupancySampler() { srf_sampler_destroy(m_impl); }
	OccupancySampler(const OccupancySampler&) = delete;
	OccupancySampler& operator=(const OccupancySampler&) = delete;

	static srf_sampler_config default_config() { srf_sampler_config c; srf_sampler_config_default(&c); return c; }

	// occupancy_sampler.cu:946-978; one uint is drawn from the caller's generator, as there
	void init(uint32_t n_images, const int32_t image_resolution[2], const float focal_length[2], const float principal_point[2],
	          const float* camera_matrices, srf_pcg32& rng, void* stream) {
		check(srf_sampler_init(m_impl, n_images, image_resolution, focal_length, principal_point, camera_matrices, &rng, stream));
		refresh();
	}
	// occupancy_sampler.cu:980-1029
	void sample_positions_from_grid(uint32_t n_uniform_positions, uint32_t n_nonuniform_positions, float* grid_positions, uint32_t* grid_indices, void* stream) {
		check(srf_sampler_sample_positions_from_grid(m_impl, n_uniform_positions, n_nonuniform_positions, grid_positions, grid_indices, stream));
		refresh();
	}
	// occupancy_sampler.cu:1031-1061
	void update_grid(uint32_t n_total_positions, uint32_t padded_output_width, const void* grid_densities, int32_t densities_dtype,
	                 const uint32_t* grid_indices, int32_t density_activation, void* stream) {
		check(srf_sampler_update_grid(m_impl, n_total_positions, padded_output_width, grid_densities, densities_dtype, grid_indices, density_activation, stream));
	}
	// occupancy_sampler.cu:1063-1088
	void update_grid_bitfield(void* stream) { check(srf_sampler_update_grid_bitfield(m_impl, stream)); }
	// snapshot load (testbed.cu:158-168): the caller's grid replaces density_grid
	void set_ray_sphere_bound(const float center[3], float radius) { check(srf_sampler_set_ray_sphere_bound(m_impl, center, radius)); }
	void set_grid_sample_order(bool cell_order) { check(srf_sampler_set_grid_sample_order(m_impl, cell_order ? 1 : 0)); }
	void set_density_grid(const float* density_grid_device, void* stream) { check(srf_sampler_set_density_grid(m_impl, density_grid_device, stream)); }
	// testbed.cu:166-167: the snapshot's grid (host memory) becomes density_grid and the bitfield is rebuilt
	void load_density_grid(const std::vector<float>& density_grid, void* stream) {
		check(srf_sampler_load_density_grid(m_impl, density_grid.data(), (uint32_t)density_grid.size(), stream));
	}

	// occupancy_sampler.cu:1090-1143; sample_t / sample_dt / sample_cell are optional extras (NULL to skip)
	void sample_coords_from_dataset(uint32_t n_rays, uint32_t n_rays_shift, uint32_t n_coords, const srf_dataset& dataset,
	                                float* rays, float* rays_rgba, uint32_t* n_rays_counter, uint32_t* ray_coord_indices, float* coords,
	                                uint32_t* n_coords_counter, srf_pcg32 rng, void* stream,
	                                float* sample_t = nullptr, float* sample_dt = nullptr, uint32_t* sample_cell = nullptr) {
		check(srf_sampler_sample_coords_from_dataset(m_impl, n_rays, n_rays_shift, n_coords, &dataset, rays, rays_rgba, n_rays_counter,
		                                             ray_coord_indices, coords, n_coords_counter, rng, sample_t, sample_dt, sample_cell, stream));
	}
	// occupancy_sampler.cu:1145-1188
	void generate_rays_from_camera_matrix(const int32_t resolution[2], const float focal_length[2], const float principal_point[2],
	                                      const float camera_matrix[12], srf_ray_payload* payload, uint32_t spp, void* stream) {
		check(srf_sampler_generate_rays_from_camera_matrix(m_impl, resolution, focal_length, principal_point, camera_matrix, payload, spp, stream));
	}
	// occupancy_sampler.cu:1190-1216
	void generate_coords_from_rays(uint32_t n_rays, uint32_t n_steps, srf_ray_payload* payloads, float* coords, void* stream) {
		check(srf_sampler_generate_coords_from_rays(m_impl, n_rays, n_steps, payloads, coords, stream));
	}
	// Testbed's setters of the snapping flags and clip distances (testbed.cu:185-199)
	void set_runtime(bool snap_train, bool snap_render, float near_distance, float far_distance) {
		check(srf_sampler_set_runtime(m_impl, snap_train ? 1 : 0, snap_render ? 1 : 0, near_distance, far_distance));
		refresh();
	}

	// the public members of the reference class (occupancy_sampler.h:88-134), refreshed after every call that changes them
	const srf_sampler_info& members() const { return m_info; }
	float* density_grid() const { return m_info.density_grid; }
	float* density_grid_mean() const { return m_info.density_grid_mean; }
	const uint8_t* density_grid_bitfield() const { return m_info.density_grid_bitfield; }   // change it only through update_grid_bitfield
	srf_sampler_t* handle() const { return m_impl; }

private:
	void refresh() { check(srf_sampler_get_info(m_impl, &m_info)); }
	srf_sampler_t* m_impl = nullptr;
	srf_sampler_info m_info{};
};

// ---- snapshots -------------------------------------------------------------------------------------------------------
// The part of a snapshot the sampler needs (Testbed::save_snapshot / load_snapshot, internal/testbed.cu:135-171): the model
// configuration as msgpack (nlohmann's json::to_msgpack) with a "snapshot" object holding, besides the trainer's network (skipped
// here), density_grid (one binary of float32 values), scene_scale and scene_offset.  A missing "snapshot" object throws the
// reference's message; so does a missing scene_scale or scene_offset, which the reference reads unconditionally.
struct Snapshot {
	srf_sampler_config sampler;            // the "samlper" block, defaults of occupancy_sampler.cu:909-944 for absent keys
	std::vector<float> density_grid;
	float scene_scale = 1.f;
	float scene_offset[3] = {0.f, 0.f, 0.f};
};

namespace detail {
// a reader for the subset of msgpack that nlohmann::json writes: values are visited in place, nothing is built
class Msgpack {
public:
	Msgpack(const uint8_t* p, size_t n) : m_p(p), m_end(p + n) {}
	enum Kind { NIL, BOOL, INT, FLOAT, STR, BIN, ARRAY, MAP };
	struct Head { Kind kind; uint64_t n; int64_t i; double f; const uint8_t* data; };      // n: length (str, bin) or element count (array, map)
	// reads the head of the next value; for str and bin the payload is consumed as well
	Head next() {
		const uint8_t b = byte();
		Head h{NIL, 0, 0, 0.0, nullptr};
		if (b <= 0x7f) { h.kind = INT; h.i = b; }
		else if (b >= 0xe0) { h.kind = INT; h.i = (int8_t)b; }
		else if (b >= 0x80 && b <= 0x8f) { h.kind = MAP; h.n = b & 0x0f; }
		else if (b >= 0x90 && b <= 0x9f) { h.kind = ARRAY; h.n = b & 0x0f; }
		else if (b >= 0xa0 && b <= 0xbf) { h.kind = STR; h.n = b & 0x1f; h.data = take(h.n); }
		else switch (b) {
			case 0xc0: break;
			case 0xc2: h.kind = BOOL; h.i = 0; break;
			case 0xc3: h.kind = BOOL; h.i = 1; break;
			case 0xc4: h.kind = BIN; h.n = be(1); h.data = take(h.n); break;
			case 0xc5: h.kind = BIN; h.n = be(2); h.data = take(h.n); break;
			case 0xc6: h.kind = BIN; h.n = be(4); h.data = take(h.n); break;
			case 0xc7: { const uint64_t n = be(1); take(1 + n); h.kind = BIN; break; }     // ext: skipped, reported as an empty binary
			case 0xc8: { const uint64_t n = be(2); take(1 + n); h.kind = BIN; break; }
			case 0xc9: { const uint64_t n = be(4); take(1 + n); h.kind = BIN; break; }
			case 0xca: { const uint32_t u = (uint32_t)be(4); float f; std::memcpy(&f, &u, 4); h.kind = FLOAT; h.f = f; break; }
			case 0xcb: { const uint64_t u = be(8); double d; std::memcpy(&d, &u, 8); h.kind = FLOAT; h.f = d; break; }
			case 0xcc: h.kind = INT; h.i = (int64_t)be(1); break;
			case 0xcd: h.kind = INT; h.i = (int64_t)be(2); break;
			case 0xce: h.kind = INT; h.i = (int64_t)be(4); break;
			case 0xcf: h.kind = INT; h.i = (int64_t)be(8); break;
			case 0xd0: h.kind = INT; h.i = (int8_t)be(1); break;
			case 0xd1: h.kind = INT; h.i = (int16_t)be(2); break;
			case 0xd2: h.kind = INT; h.i = (int32_t)be(4); break;
			case 0xd3: h.kind = INT; h.i = (int64_t)be(8); break;
			case 0xd4: take(2); h.kind = BIN; break;                                        // fixext 1..16
			case 0xd5: take(3); h.kind = BIN; break;
			case 0xd6: take(5); h.kind = BIN; break;
			case 0xd7: take(9); h.kind = BIN; break;
			case 0xd8: take(17); h.kind = BIN; break;
			case 0xd9: h.kind = STR; h.n = be(1); h.data = take(h.n); break;
			case 0xda: h.kind = STR; h.n = be(2); h.data = take(h.n); break;
			case 0xdb: h.kind = STR; h.n = be(4); h.data = take(h.n); break;
			case 0xdc: h.kind = ARRAY; h.n = be(2); break;
			case 0xdd: h.kind = ARRAY; h.n = be(4); break;
			case 0xde: h.kind = MAP; h.n = be(2); break;
			case 0xdf: h.kind = MAP; h.n = be(4); break;
			default: throw std::runtime_error("snapshot: byte 0xc1 is not msgpack");
		}
		return h;
	}
	// skips what is left of a value whose head has been read
	void skip_rest(const Head& h) {
		if (h.kind == ARRAY) for (uint64_t k = 0; k < h.n; ++k) skip();
		if (h.kind == MAP) for (uint64_t k = 0; k < 2 * h.n; ++k) skip();
	}
	void skip() { skip_rest(next()); }
	std::string key() {
		const Head h = next();
		if (h.kind != STR) throw std::runtime_error("snapshot: an object key that is not a string");
		return std::string((const char*)h.data, (size_t)h.n);
	}
	static double number(const Head& h, const char* what) {
		if (h.kind == INT || h.kind == BOOL) return (double)h.i;
		if (h.kind == FLOAT) return h.f;
		throw std::runtime_error(std::string("snapshot: ") + what + " is not a number");
	}
private:
	uint8_t byte() { return *take(1); }
	const uint8_t* take(uint64_t n) {
		if (n > (uint64_t)(m_end - m_p)) throw std::runtime_error("snapshot: the file ends inside a value");
		const uint8_t* p = m_p;
		m_p += n;
		return p;
	}
	uint64_t be(int bytes) {
		const uint8_t* p = take((uint64_t)bytes);
		uint64_t v = 0;
		for (int k = 0; k < bytes; ++k) v = (v << 8) | p[k];
		return v;
	}
	const uint8_t* m_p;
	const uint8_t* m_end;
};

// one entry of the "samlper" block (occupancy_sampler.cu:909-944); grid_size is one number there, three equal entries here, and a
// file written by this library's tools may hold the three
inline void sampler_entry(Msgpack& r, const std::string& key, srf_sampler_config& c) {
	const Msgpack::Head h = r.next();
	auto text = [&]() {
		if (h.kind != Msgpack::STR) throw std::runtime_error("snapshot: samlper." + key + " is not a string");
		return std::string((const char*)h.data, (size_t)h.n);
	};
	auto num = [&]() { return Msgpack::number(h, key.c_str()); };
	if (key == "warping_type") c.warping_type = string_to_warping_type(text());
	else if (key == "grid_distribution_type") c.grid_distribution_type = string_to_griddist_type(text());
	else if (key == "sampling_type") c.sampling_type = string_to_sampling_type(text());
	else if (key == "aabb_scale") c.aabb_scale = (float)num();
	else if (key == "use_grid") c.use_grid = num() != 0.0;
	else if (key == "init_grid_with_mask") c.init_grid_with_mask = num() != 0.0;
	else if (key == "grid_size") {
		if (h.kind == Msgpack::ARRAY) {
			if (h.n != 3) throw std::runtime_error("snapshot: samlper.grid_size must be one number or three");
			for (int k = 0; k < 3; ++k) c.grid_size[k] = (uint32_t)Msgpack::number(r.next(), "grid_size");
		} else c.grid_size[0] = c.grid_size[1] = c.grid_size[2] = (uint32_t)num();
	}
	else if (key == "num_cascades") c.num_cascades = (uint32_t)num();
	else if (key == "ema_decay") c.ema_decay = (float)num();
	else if (key == "maximum_marching_steps") c.maximum_marching_steps = (uint32_t)num();
	else if (key == "cone_angle_constant") c.cone_angle_constant = (float)num();
	else if (key == "min_cone_stepsize") c.min_cone_stepsize = (float)num();
	else if (key == "max_cone_stepsize") c.max_cone_stepsize = (float)num();
	else if (key == "near_distance") c.near_distance = (float)num();
	else if (key == "far_distance") c.far_distance = (float)num();
	else if (key == "snap_to_pixel_centers_in_training") c.snap_to_pixel_centers_in_training = num() != 0.0;
	else if (key == "snap_to_pixel_centers_in_rendering") c.snap_to_pixel_centers_in_rendering = num() != 0.0;
	else if (key == "min_optical_thickness") c.min_optical_thickness = (float)num();
	else r.skip_rest(h);
}
} // namespace detail

// parses a snapshot held in memory
inline Snapshot parse_snapshot(const uint8_t* bytes, size_t n_bytes) {
	using detail::Msgpack;
	Snapshot out;
	srf_sampler_config_default(&out.sampler);
	Msgpack r(bytes, n_bytes);
	const Msgpack::Head top = r.next();
	bool has_snapshot = false, has_sampler = false, has_grid = false, has_scale = false, has_offset = false;
	if (top.kind == Msgpack::MAP) for (uint64_t k = 0; k < top.n; ++k) {
		const std::string key = r.key();
		if (key == "samlper") {
			const Msgpack::Head b = r.next();
			if (b.kind != Msgpack::MAP) throw std::runtime_error("snapshot: \"samlper\" is not an object");
			for (uint64_t j = 0; j < b.n; ++j) { const std::string name = r.key(); detail::sampler_entry(r, name, out.sampler); }
			has_sampler = true;
		} else if (key == "snapshot") {
			const Msgpack::Head b = r.next();
			if (b.kind != Msgpack::MAP) throw std::runtime_error("snapshot: \"snapshot\" is not an object");
			has_snapshot = true;
			for (uint64_t j = 0; j < b.n; ++j) {
				const std::string name = r.key();
				const Msgpack::Head h = r.next();
				if (name == "density_grid") {
					if (h.kind != Msgpack::BIN || h.n % 4) throw std::runtime_error("snapshot.density_grid: a binary of float32 values expected");
					out.density_grid.resize((size_t)(h.n / 4));
					if (h.n) std::memcpy(out.density_grid.data(), h.data, (size_t)h.n);       // little-endian floats, as the host is
					has_grid = true;
				} else if (name == "scene_scale") {
					out.scene_scale = (float)Msgpack::number(h, "snapshot.scene_scale");
					has_scale = true;
				} else if (name == "scene_offset") {
					if (h.kind != Msgpack::ARRAY || h.n != 3) throw std::runtime_error("snapshot.scene_offset: an array of three numbers expected");
					for (int c = 0; c < 3; ++c) out.scene_offset[c] = (float)Msgpack::number(r.next(), "snapshot.scene_offset");
					has_offset = true;
				} else r.skip_rest(h);
			}
		} else r.skip();
	}
	if (!has_snapshot) throw std::runtime_error("ERROR in loading snapshot.");                  // testbed.cu:157-160
	if (!has_scale || !has_offset) throw std::runtime_error("snapshot: scene_scale and scene_offset are required (testbed.cu:163-164)");
	if (!has_grid) throw std::runtime_error("snapshot.density_grid: a binary of float32 values expected");
	if (!has_sampler) throw std::runtime_error("the snapshot holds no \"samlper\" block");
	return out;
}

inline Snapshot read_snapshot(const std::string& path) {
	std::FILE* f = std::fopen(path.c_str(), "rb");
	if (!f) throw std::runtime_error("cannot open snapshot " + path);
	std::vector<uint8_t> raw;
	uint8_t buf[1 << 16];
	for (size_t n; (n = std::fread(buf, 1, sizeof(buf), f)) > 0;) raw.insert(raw.end(), buf, buf + n);
	std::fclose(f);
	return parse_snapshot(raw.data(), raw.size());
}

// An OccupancySampler configured by the snapshot's "samlper" block, holding its density grid, bitfield rebuilt (testbed.cu:152-168)
inline std::unique_ptr<OccupancySampler> sampler_from_snapshot(const Snapshot& snapshot, void* stream) {
	std::unique_ptr<OccupancySampler> s(new OccupancySampler(snapshot.sampler));
	s->load_density_grid(snapshot.density_grid, stream);
	return s;
}

class RayMarcher {
public:
	explicit RayMarcher(const srf_marcher_config& config) { check(srf_marcher_create(&config, &m_impl)); }   // ray_marcher.cu:294-301
	~RayMarcher() { srf_marcher_destroy(m_impl); }
	RayMarcher(const RayMarcher&) = delete;
	RayMarcher& operator=(const RayMarcher&) = delete;

	static srf_marcher_config default_config() { srf_marcher_config c; srf_marcher_config_default(&c); return c; }
	srf_marcher_config config() const { srf_marcher_config c; check(srf_marcher_get_config(m_impl, &c)); return c; }
	void set_config(const srf_marcher_config& c) { check(srf_marcher_set_config(m_impl, &c)); }

	// ray_marcher.cu:303-374
	void volume_rendering_with_loss_and_gradient(const srf_loss_args& args, const float* rays_rgba, const uint32_t* n_rays_counter,
	                                             uint32_t* ray_coord_indices, const float* dt, const float* coords, float* compacted_coords,
	                                             uint32_t* n_compacted_coords_counter, const void* network_output, void* dloss_doutput,
	                                             float* loss_output, const float* density_grid_mean, void* stream, float* rgb_ray_out = nullptr) {
		check(srf_marcher_volume_rendering_with_loss_and_gradient(m_impl, &args, rays_rgba, n_rays_counter, ray_coord_indices, dt, coords, compacted_coords,
		                                                          n_compacted_coords_counter, network_output, dloss_doutput, loss_output, density_grid_mean,
		                                                          rgb_ray_out, stream));
	}
	// waits for the stream; throws if the ordered offsets of the last training call could not be chained (no counterpart in the reference)
	void sync_check(void* stream) { check(srf_marcher_sync_check(m_impl, stream)); }
	// ray_marcher.cu:376-415
	void volume_rendering(const OccupancySampler& sampler, const srf_render_args& args, srf_ray_payload* payloads, float* rgba,
	                      const float* coords, const void* rgbsigma, void* stream) {
		check(srf_marcher_volume_rendering(m_impl, sampler.handle(), &args, payloads, rgba, coords, rgbsigma, stream));
	}
	srf_marcher_t* handle() const { return m_impl; }

private:
	srf_marcher_t* m_impl = nullptr;
};

// Testbed's helper launches (testbed.cu:398-404, 423-477)
inline void compact_rays(const RayMarcher& marcher, uint32_t n, const srf_ray_payload* src_payloads, const float* src_rgba, srf_ray_payload* dst_payloads, float* dst_rgba,
                         srf_ray_payload* final_payloads, float* final_rgba, uint32_t* n_alive_counter, uint32_t* n_final_counter, void* stream) {
	check(srf_compact_rays(marcher.handle(), n, src_payloads, src_rgba, dst_payloads, dst_rgba, final_payloads, final_rgba, n_alive_counter, n_final_counter, stream));
}
inline void shade(uint32_t n_rays, const float* rgba, const srf_ray_payload* payloads, float* frame_buffer, int32_t render_mode, bool train_in_linear_colors, void* stream) {
	check(srf_shade(n_rays, rgba, payloads, frame_buffer, render_mode, train_in_linear_colors ? 1 : 0, stream));
}

// Testbed::render_frame up to shade (internal/testbed.cu:479-611); returns the number of rounds
inline uint32_t render_frame(const OccupancySampler& sampler, const RayMarcher& marcher, const srf_frame_args& args, srf_inference_fn inference, void* user,
                             float* frame_buffer, void* stream) {
	uint32_t rounds = 0;
	check(srf_render_frame(sampler.handle(), marcher.handle(), &args, inference, user, frame_buffer, &rounds, stream));
	return rounds;
}
// CudaRenderBuffer::accumulate / ::tonemap (internal/utils/render_buffer.cu:46-235)
inline void frame_accumulate(const int32_t resolution[2], const float* frame_buffer, float* accumulate_buffer, uint32_t spp, int32_t color_space, void* stream) {
	check(srf_frame_accumulate(resolution, frame_buffer, accumulate_buffer, spp, color_space, stream));
}
inline void frame_tonemap(const int32_t resolution[2], float exposure, const float background_color[4], const float* accumulate_buffer, int32_t color_space,
                          int32_t output_color_space, int32_t tonemap_curve, float* out_rgba, void* stream) {
	check(srf_frame_tonemap(resolution, exposure, background_color, accumulate_buffer, color_space, output_color_space, tonemap_curve, out_rgba, stream));
}

} // namespace srf
