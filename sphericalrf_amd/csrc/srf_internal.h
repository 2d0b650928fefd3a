// Host-side internals of libsrf_hip.so shared by its translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/srf_hip.h"
#include "srf_device.h"
#include "srf_skip.h"

namespace srf {

void set_error(const char* fmt, ...);

#define SRF_FAIL(code, ...) do { ::srf::set_error(__VA_ARGS__); return (code); } while (0)
#define SRF_REQUIRE(cond, ...) do { if (!(cond)) SRF_FAIL(SRF_ERR_INVALID, __VA_ARGS__); } while (0)
#define SRF_HIP(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) SRF_FAIL(SRF_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); } while (0)
#define SRF_LAUNCH_CHECK() SRF_HIP(hipGetLastError())

// A device buffer that only ever grows.  Growing frees the old allocation, which
// waits for the device, so work already enqueued on it stays valid.
struct Workspace {
	void*  ptr = nullptr;
	size_t bytes = 0;
	int reserve(size_t need);
	void release();
};

constexpr uint32_t COUNT_PROBE_BUDGET = 192;   // lookups after which the counting march parks a ray for the wide march
constexpr uint32_t COUNT_PARK_LANES = 32;      // ... once its wavefront has no more rays than this under way

SRF_HD uint32_t div_up(uint32_t a, uint32_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t a, size_t b) { return (a + b - 1) / b * b; }

// exclusive prefix sum of n uint32 values on the device, starting from *initial
// (a device uint32, may be NULL for 0); *initial_plus_total (may alias initial or be
// NULL) receives initial + sum.  scratch must hold scan_scratch_bytes(n).
size_t scan_scratch_bytes(uint32_t n);
int fill_u32(void* p, size_t n_words, uint32_t v, hipStream_t stream);
int scan_exclusive_u32(const uint32_t* in, uint32_t* out, uint32_t n, const uint32_t* initial, uint32_t* initial_plus_total,
                       void* scratch, hipStream_t stream);

} // namespace srf

struct srf_sampler {
	srf::Params P;
	int32_t  init_grid_with_mask;
	uint32_t n_total;
	uint32_t i_step;
	srf::Pcg32 rng;
	float*   density_grid_current;
	float*   density_grid;
	float*   density_grid_mean;
	uint8_t* density_grid_bitfield;
	uint16_t* skip_dist;     // empty-space radii per block (srf_skip.h); rebuilt with the bitfield
	bool     skip_valid;    // skip_dist matches the bitfield
	bool     skip_enabled;  // SRF_MARCH_SKIP=0 in the environment at creation switches the table off
	// Switches the tests use to run both sides of a size-dependent choice on small inputs; read from the environment once, when the
	// sampler is created (-1: the library chooses): SRF_SPLAT_SORT, SRF_GRID_SAMPLE_BITS, SRF_GRID_SAMPLE_BY_CELL = 0|1
	// (SRF_SPLAT_SORT=2: the large-batch splat through the library's radix sort instead of the partition made for it);
	// SRF_COUNT_PROBE_BUDGET = lookups after which the counting march parks a ray (0: never), SRF_COUNT_PARK_LANES = rays a
	// wavefront may have under way when it does
	int      force_splat_sort, force_sample_bits, force_sample_by_cell;
	uint32_t count_probe_budget, count_park_lanes;
	bool     grid_sample_cell_order = false;   // srf_sampler_set_grid_sample_order
	uint32_t dealt_entries = 0;                // leading entries the last sample_positions_from_grid left in cell order
	srf::Workspace ws;
	srf::Workspace park_ws;          // queue of the rays the render marches hand to their one-ray-per-wavefront march
	uint32_t* park_counts = nullptr; // two counters of that queue, used in turn: a march clears the one the next march will use
	uint32_t park_turn = 0;
	bool march_park_all = false;     // SRF_MARCH_PARK_ALL at creation
};

struct srf_marcher {
	srf_marcher_config cfg;
	srf::Workspace ws;          // ordered-offset chain of the streaming compositing kernel
	srf::Workspace wave_ws;     // ordered-offset chain and item table of the wave-per-item compositing kernel
	srf::Workspace ws2;         // per-ray forward results of the three-launch compositing
	srf::Workspace reg;         // reg_distortion_buffer (ray_marcher.h:79-80)
	srf::Workspace compact_ws;  // per-block counts of srf_compact_rays
	srf::Workspace frame_ws;    // ray buffers, coordinates and network output of srf_render_frame
	uint32_t* frame_counter_host = nullptr;  // pinned words through which srf_render_frame reads the ray counters
	unsigned long long* frame_word_dev = nullptr;   // device address of the second of them (8 bytes in), which the compaction kernel writes itself
	uint32_t frame_stamp = 0;                // number of the last compaction srf_render_frame waited for
	bool force_unfused = false;             // SRF_COMPOSITE_IMPL=unfused at creation
	bool force_waves = false;               // SRF_COMPOSITE_IMPL=waves at creation
	int degraded = 0;                       // how often a chain of ordered offsets has given up: after the first time the wave-per-item kernel (whose items never wait
	                                        // for a workgroup that is not running) takes the calls, after the second the three-launch implementation
	volatile uint32_t* host_error = nullptr; // host word the streaming kernel raises when its chain gives up (pinned, device-writable)
	uint32_t* host_error_dev = nullptr;      // the same word as the device addresses it
	uint32_t* chain_error_dev = nullptr;     // device word of the last streaming launch (NULL before the first)
	uint32_t lookback_spin_limit = 1u << 22; // polls before a group gives up waiting for its predecessors
};

namespace srf {
struct LossConst;
// the wave-per-item training compositing (srf_composite_waves.hip): device scratch it needs for a call of n_rays rays (the first 512
// bytes zero before the first call, and left zero by every call), where its error word lies, and the two launches
size_t waves_scratch_bytes(uint32_t n_rays);
uint32_t* waves_error_word(void* scratch);
int launch_waves(const srf_loss_args* a, const LossConst& K, void* scratch, uint32_t* host_error, uint32_t spin_limit, const float* rays_rgba, const uint32_t* n_rays_counter,
                 uint32_t* ray_coord_indices, const float* dt, const float* coords, float* compacted_coords, uint32_t* n_compacted_coords_counter,
                 const void* network_output, void* dloss_doutput, float* loss_output, const float* density_grid_mean, float* rgb_ray_out, hipStream_t st);
// ---- the frame loop paced by the device (srf_render_frame_paced) ----
// What a round of the loop needs to know, kept on the device: the compaction of round r reads the words of round r - 1 and writes
// those of round r (two sets that take turns), every other kernel of round r reads the latter.
struct RoundWords {
	uint32_t n_alive;       // rays alive after this round's compaction (0: the frame is finished, every later kernel returns at once)
	uint32_t n_steps;       // clamp(n_pixels / n_alive, 1, 8), testbed.cu:544-547
	uint32_t offset;        // i_steps_offset of this round's volume_rendering
	uint32_t n_elements;    // n_alive * n_steps: what the network evaluates
	uint32_t next_offset;   // offset + n_steps; the loop ends once it reaches MARCH_ITER (testbed.cu:526)
	uint32_t rounds;        // rounds with live rays so far
	uint32_t pad[2];
};
constexpr uint32_t FRAME_MARCH_ITER = 10000, FRAME_MIN_STEPS = 1, FRAME_MAX_STEPS = 8;      // testbed.h: MARCH_ITER, MIN/MAX_STEPS_INBETWEEN_COMPACTION
// bound: an upper limit of the rays the call has to look at, known to the host; the kernels take the true numbers from the words
int compact_rays_paced(srf_marcher* m, uint32_t bound, uint32_t n_pixels, const RoundWords* in, RoundWords* out, const srf_ray_payload* src_payloads, const float* src_rgba,
                       srf_ray_payload* dst_payloads, float* dst_rgba, srf_ray_payload* final_payloads, float* final_rgba, uint32_t* n_final_counter,
                       hipStream_t stream, unsigned long long* host_word, uint32_t stamp);
int generate_coords_paced(srf_sampler* s, uint32_t bound, const RoundWords* round, srf_ray_payload* payloads, float* coords, hipStream_t stream);
int volume_rendering_paced(srf_marcher* m, const srf_sampler* s, const srf_render_args* a, uint32_t bound, const RoundWords* round,
                           srf_ray_payload* payloads, float* rgba, const float* coords, const void* rgbsigma, hipStream_t stream);
int shade_counted(uint32_t bound, const uint32_t* n_rays, const float* rgba, const srf_ray_payload* payloads, float* frame_buffer,
                  int32_t render_mode, int32_t train_in_linear_colors, hipStream_t stream);

// srf_compact_rays with two more choices: alive_from_zero numbers the live rays from 0 whatever *n_alive_counter holds; host_word
// (device address of a word of host memory, or NULL) receives stamp << 32 | the live-ray counter's new value when the call is done
int compact_rays(srf_marcher* m, uint32_t n, const srf_ray_payload* src_payloads, const float* src_rgba,
                 srf_ray_payload* dst_payloads, float* dst_rgba, srf_ray_payload* final_payloads, float* final_rgba,
                 uint32_t* n_alive_counter, uint32_t* n_final_counter, bool alive_from_zero, hipStream_t stream,
                 unsigned long long* host_word, uint32_t stamp);
}
