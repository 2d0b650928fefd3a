// Exercises include/srf_hip.hpp the way the reference's Testbed uses its two classes: construct from a config,
// read the public members, run one bitfield update.  Prints one line per check; exit code 0 on success.
// Without a GPU the constructor's device allocation fails and must surface as std::runtime_error (exit code 3).
// With a snapshot file as its argument it does what Testbed::load_snapshot does for the sampler instead: the file is parsed
// (reported on one line, exit code 4 with the message if it is refused), and on a device the sampler is built from it and the
// number of set bits of its bitfield is printed.
#include <cstdio>
#include <cstring>
#include <hip/hip_runtime_api.h>
#include "srf_hip.hpp"

static int snapshot_check(const char* path) {
	srf::Snapshot snap;
	try { snap = srf::read_snapshot(path); }
	catch (const std::runtime_error& e) { std::printf("refused: %s\n", e.what()); return 4; }
	double sum = 0.0;
	for (float v : snap.density_grid) sum += v;
	const srf_sampler_config& c = snap.sampler;
	std::printf("snapshot ok: cells %zu sum %.9g scale %.9g offset %.9g %.9g %.9g warp %d grid %u %u %u cascades %u griddist %d steps %u sampling %d near %.9g mask %d\n",
	            snap.density_grid.size(), sum, snap.scene_scale, snap.scene_offset[0], snap.scene_offset[1], snap.scene_offset[2], c.warping_type,
	            c.grid_size[0], c.grid_size[1], c.grid_size[2], c.num_cascades, c.grid_distribution_type, c.maximum_marching_steps, c.sampling_type,
	            c.near_distance, c.init_grid_with_mask);
	try {
		std::unique_ptr<srf::OccupancySampler> sampler = srf::sampler_from_snapshot(snap, nullptr);
		const size_t n_bytes = sampler->members().n_total_elements / 8;
		std::vector<uint8_t> bits(n_bytes);
		if (hipMemcpy(bits.data(), sampler->density_grid_bitfield(), n_bytes, hipMemcpyDeviceToHost) != hipSuccess) return 1;
		size_t set = 0;
		for (uint8_t b : bits) set += (size_t)__builtin_popcount(b);
		std::printf("device ok: bits set %zu of %zu\n", set, n_bytes * 8);
	} catch (const std::runtime_error& e) {
		std::printf("no device: %s\n", e.what());
		return 3;
	}
	return 0;
}

int main(int argc, char** argv) {
	if (argc > 1) return snapshot_check(argv[1]);
	// the reference's string -> enum step, including its refusal of the constructor's own default "Exp"
	if (srf::string_to_warping_type("ERP") != SRF_WARP_ERP || srf::string_to_sampling_type("Disparity") != SRF_SAMPLING_DISPARITY) return 1;
	bool threw = false;
	try { srf::string_to_griddist_type("Exp"); } catch (const std::runtime_error& e) { threw = std::strstr(e.what(), "Unknown grid distribution type") != nullptr; }
	if (!threw) return 1;
	std::printf("strings ok\n");

	srf_sampler_config c = srf::OccupancySampler::default_config();
	c.warping_type = srf::string_to_warping_type("ERP");
	c.grid_distribution_type = srf::string_to_griddist_type("WarpedSpace_Exp");
	c.sampling_type = srf::string_to_sampling_type("Disparity");
	c.aabb_scale = 16;
	c.grid_size[0] = 32; c.grid_size[1] = 16; c.grid_size[2] = 16;
	c.num_cascades = 3;
	c.maximum_marching_steps = 256;
	c.init_grid_with_mask = 0;
	try {
		srf::OccupancySampler sampler(c);
		const srf_sampler_info& m = sampler.members();
		if (m.n_grid_elements != 32u * 16u * 16u || m.n_cascades != 3 || m.n_total_elements != 3u * 32u * 16u * 16u) return 1;
		if (!(m.min_cone_stepsize > 0.f) || m.aabb_min[0] != 0.5f - 8.f || m.aabb_max[2] != 0.5f + 8.f) return 1;
		sampler.update_grid_bitfield(nullptr);
		sampler.set_grid_sample_order(true);
		sampler.set_grid_sample_order(false);
		srf::RayMarcher marcher(srf::RayMarcher::default_config());
		marcher.sync_check(nullptr);
		if (marcher.config().transmittance_threshold <= 0.f) return 1;
		// a bad argument comes back as an exception carrying the library's message
		threw = false;
		try { sampler.sample_positions_from_grid(8, 0, nullptr, nullptr, nullptr); } catch (const std::runtime_error& e) { threw = std::strlen(e.what()) > 0; }
		if (!threw) return 1;
		std::printf("device ok\n");
	} catch (const std::runtime_error& e) {
		std::printf("no device: %s\n", e.what());
		return 3;
	}
	return 0;
}
