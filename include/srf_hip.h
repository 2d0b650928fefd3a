/*
 * libsrf_hip.so — C ABI of the MI355X (gfx950) implementation of SphericalRF's
 * occupancy-grid sampling, ray-marching and compositing path.
 *
 * Every entry point replaces one method (or kernel launch) of the reference's
 * OccupancySampler / RayMarcher classes or of the orchestrator around them; the
 * reference interface is cited as file:line under the reference tree.  All data
 * pointers are DEVICE pointers unless the name ends in _host; every call only
 * enqueues work on `stream` (a hipStream_t passed as void*; NULL = default
 * stream) and returns without synchronising.  Functions return SRF_OK or a
 * negative error code; srf_last_error() gives the message for the calling thread.
 * Nothing throws across this boundary.
 *
 * Record layouts (identical to the reference):
 *   Ray         6 floats  {o.xyz, d.xyz}                    internal/utils/common.h:135-138
 *   Coordinate  7 floats  {pos.xyz, dt, dir.xyz}            internal/utils/common.h:150-155
 *   RayPayload  40 bytes  srf_ray_payload                   internal/utils/common.h:158-165
 *   RGBA        4 floats
 *   camera      12 floats, column-major 3x4 {right, down, forward, origin}
 */
#ifndef SRF_HIP_H
#define SRF_HIP_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SRF_OK               0
#define SRF_ERR_INVALID     -1   /* bad argument (NULL pointer, size mismatch, unknown enum value) */
#define SRF_ERR_HIP         -2   /* a HIP runtime call failed */
#define SRF_ERR_UNSUPPORTED -3   /* valid in the reference but not implemented here */

/* enum values as in internal/utils/common.h:61-115 and internal/utils/loss.h:10-18 */
enum { SRF_ACT_NONE = 0, SRF_ACT_RELU = 1, SRF_ACT_LOGISTIC = 2, SRF_ACT_EXPONENTIAL = 3 };
enum { SRF_RENDER_AO = 0, SRF_RENDER_SHADE = 1, SRF_RENDER_NORMALS = 2, SRF_RENDER_DEPTH = 3, SRF_RENDER_DISTANCE = 4, SRF_RENDER_COST = 5 };
enum { SRF_COLOR_LINEAR = 0, SRF_COLOR_SRGB = 1, SRF_COLOR_VISPOSNEG = 2 };
enum { SRF_WARP_NGP = 0, SRF_WARP_MIPNERF360 = 1, SRF_WARP_DONERF = 2, SRF_WARP_SIGMOID = 3, SRF_WARP_ERP = 4, SRF_WARP_SINUSOIDAL = 5 };
enum { SRF_SAMPLING_ORIGINAL = 0, SRF_SAMPLING_DISPARITY = 1, SRF_SAMPLING_LOG = 2 };
enum { SRF_GRID_WARPED_EXP = 0, SRF_GRID_WARPED_RECIPROCAL = 1, SRF_GRID_METRIC_EXP = 2, SRF_GRID_METRIC_RECIPROCAL = 3 };
enum { SRF_REG_NONE = 0, SRF_REG_DISTORTION = 1 };
enum { SRF_LOSS_L2 = 0, SRF_LOSS_L1 = 1, SRF_LOSS_MAPE = 2, SRF_LOSS_SMAPE = 3, SRF_LOSS_SMOOTHL1 = 4, SRF_LOSS_LOGL1 = 5, SRF_LOSS_RELATIVEL2 = 6 };
enum { SRF_DTYPE_F16 = 0, SRF_DTYPE_F32 = 1 };

typedef struct srf_sampler srf_sampler_t;   /* OccupancySampler, internal/sampler/occupancy_sampler.h:13-135 */
typedef struct srf_marcher srf_marcher_t;   /* RayMarcher,       internal/render/ray_marcher.h:13-81 */
/* Threads and streams: a handle owns workspaces that its calls reuse without locking, as the reference's objects own their
 * GPUMemory members.  Use one handle from one thread at a time, and keep its calls on one stream (or order the streams yourself
 * with events): two calls on one handle that overlap on the device share those workspaces and race.  Different handles are
 * independent, except for srf_marcher_volume_rendering_with_loss_and_gradient_noalloc (see there). */

/* tcnn::pcg32 state; callers keep it on the host exactly as Testbed::m_rng does (internal/testbed.h:92-93) */
typedef struct srf_pcg32 { uint64_t state, inc; } srf_pcg32;

/* RayPayload, internal/utils/common.h:158-165 */
typedef struct srf_ray_payload {
	uint8_t  alive;
	uint8_t  pad_[3];
	float    o[3];
	float    d[3];
	uint32_t idx;
	float    t;
	uint32_t n_steps;
} srf_ray_payload;

/*
 * The "samlper" [sic] config block, internal/sampler/occupancy_sampler.cu:909-944.
 * A negative min_cone_stepsize / max_cone_stepsize asks for the reference's
 * derived default.  grid_size has one entry per warped axis (x azimuth, y polar,
 * z radial); the reference has a single "grid_size", i.e. three equal entries.
 */
typedef struct srf_sampler_config {
	int32_t  warping_type;
	float    aabb_scale;
	int32_t  use_grid;
	int32_t  init_grid_with_mask;
	uint32_t grid_size[3];
	uint32_t num_cascades;
	float    ema_decay;
	int32_t  grid_distribution_type;
	uint32_t maximum_marching_steps;
	float    cone_angle_constant;
	float    min_cone_stepsize;
	float    max_cone_stepsize;
	float    near_distance;
	float    far_distance;
	int32_t  sampling_type;
	int32_t  snap_to_pixel_centers_in_training;
	int32_t  snap_to_pixel_centers_in_rendering;
	float    min_optical_thickness;
} srf_sampler_config;

/* read-out of OccupancySampler's public members (internal/sampler/occupancy_sampler.h:88-134) */
typedef struct srf_sampler_info {
	int32_t  warping_type;
	uint32_t aabb_scale;
	float    aabb_min[3], aabb_max[3];
	int32_t  use_grid, init_grid_with_mask;
	uint32_t grid_size[3];
	uint32_t n_grid_elements, n_cascades, n_total_elements;
	uint32_t i_step;
	float    ema_decay;
	uint32_t n_max_steps;
	float    cone_angle_constant, min_cone_stepsize, max_cone_stepsize, near_distance, far_distance;
	int32_t  sampling_type;
	int32_t  snap_to_pixel_centers_in_training, snap_to_pixel_centers_in_rendering;
	float    min_optical_thickness;
	int32_t  griddist_type;
	float*   density_grid_current;       /* device, n_total_elements floats */
	float*   density_grid;               /* device, n_total_elements floats */
	float*   density_grid_mean;          /* device, 1 float */
	uint8_t* density_grid_bitfield;      /* device, n_total_elements / 8 bytes */
	srf_pcg32 rng;
} srf_sampler_info;

/* Dataset fields the sampler reads (internal/dataset/dataset.h:19-39) */
typedef struct srf_dataset {
	uint32_t n_images;
	int32_t  image_resolution[2];
	float    focal_length[2];
	float    principal_point[2];
	const float*    xforms;                /* n_images x 12 floats */
	const uint16_t* images;                /* half RGBA per pixel; NULL: ray targets are written as zeros */
	const uint16_t* sampling_probability;  /* half per pixel; NULL: every pixel is eligible */
} srf_dataset;

/* the "render" config block, internal/render/ray_marcher.cu:294-301 */
typedef struct srf_marcher_config {
	int32_t train_with_random_bg_color;
	int32_t train_in_linear_color;
	float   transmittance_threshold;
	int32_t regularization_type;
} srf_marcher_config;

const char* srf_last_error(void);
/* number of HIP devices visible; negative on error.  Does not create a context. */
int srf_device_count(void);

/* ---------------- OccupancySampler ---------------- */
void srf_sampler_config_default(srf_sampler_config* cfg);                       /* occupancy_sampler.cu:911-943 defaults */
int  srf_sampler_create(const srf_sampler_config* cfg, srf_sampler_t** out);    /* OccupancySampler::OccupancySampler, occupancy_sampler.cu:909 */
void srf_sampler_destroy(srf_sampler_t* s);
int  srf_sampler_get_info(const srf_sampler_t* s, srf_sampler_info* out);
/* the public members Python pokes at run time (internal/python_api.cu:97-108) */
int  srf_sampler_set_runtime(srf_sampler_t* s, int32_t snap_train, int32_t snap_render, float near_distance, float far_distance);

/* OccupancySampler::init, occupancy_sampler.cu:946-978.  rng_host is advanced by one next_uint() as the reference does. */
int  srf_sampler_init(srf_sampler_t* s, uint32_t n_images, const int32_t image_resolution[2], const float focal_length[2],
                      const float principal_point[2], const float* camera_matrices, srf_pcg32* rng_host, void* stream);

/* No counterpart in the reference, which bounds rays by the box alone (bounding_box.h:145-180); off unless set.  With a
 * sphere set, the training and render marches keep exactly those samples of the unbounded march whose t lies within the
 * ray's stretch inside the sphere (the chain of t is not moved); radius <= 0 removes the bound.  Takes effect from the next call. */
int  srf_sampler_set_ray_sphere_bound(srf_sampler_t* s, const float center[3], float radius);

/* The same stretch for n_rays rays laid out as (origin, direction) x 6 floats: t_near[i] <= t <= t_far[i] is inside the
 * sphere; a ray whose line misses it gets t_near = +inf, t_far = -inf.  All pointers device memory. */
int  srf_ray_sphere_bounds(uint32_t n_rays, const float* rays, const float center[3], float radius, float* t_near, float* t_far, void* stream);

/* Testbed::load_snapshot, internal/testbed.cu:167: overwrite density_grid (n_total_elements floats, device) */
int  srf_sampler_set_density_grid(srf_sampler_t* s, const float* density_grid, void* stream);
/* The two sampler lines of Testbed::load_snapshot, internal/testbed.cu:166-167: density_grid is assigned from the snapshot's values
 * in host memory (n_values must be n_total_elements) and the bitfield is rebuilt.  Returns when the copy has finished. */
int  srf_sampler_load_density_grid(srf_sampler_t* s, const float* density_grid_host, uint32_t n_values, void* stream);

/* No counterpart in the reference: the order in which srf_sampler_sample_positions_from_grid hands the uniform points over.
 * 0 (default): the reference's, point i in entry i.  1, cell order: with a power-of-two cell count n_cells (at least 2048) the
 * first n_cells * floor(n_uniform / n_cells) entries hold the same points sorted by the cell they fall in, entry
 * t = m * n_cells + v holding point i = ((v * A' - step * n_uniform) mod n_cells) + m * n_cells (A' the inverse of 56924617
 * modulo 2^32, step the number of srf_sampler_update_grid calls so far); every later entry is as in order 0.  The non-uniform
 * draw, whose entries follow those of the uniform one, is laid out the same way with n_nonuniform in place of n_uniform.
 * srf_sampler_update_grid, given densities and indices in that same order, then combines the uniform draw's sorted entries per
 * cell without sorting them (it checks each entry's index, so arrays in any other order still give the right grid, only slower).
 * The set of points, their positions and indices and the grid that results are those of order 0. */
int  srf_sampler_set_grid_sample_order(srf_sampler_t* s, int32_t cell_order);

/* OccupancySampler::sample_positions_from_grid, occupancy_sampler.cu:980-1029.
 * grid_positions: (n_uniform + n_nonuniform) x 3 floats; grid_indices: as many uint32. */
int  srf_sampler_sample_positions_from_grid(srf_sampler_t* s, uint32_t n_uniform_positions, uint32_t n_nonuniform_positions,
                                            float* grid_positions, uint32_t* grid_indices, void* stream);

/* OccupancySampler::update_grid, occupancy_sampler.cu:1031-1061.  grid_densities: element i*padded_output_width is sample i's density. */
int  srf_sampler_update_grid(srf_sampler_t* s, uint32_t n_total_positions, uint32_t padded_output_width,
                             const void* grid_densities, int32_t densities_dtype, const uint32_t* grid_indices,
                             int32_t density_activation, void* stream);

/* OccupancySampler::update_grid_bitfield, occupancy_sampler.cu:1063-1088 */
int  srf_sampler_update_grid_bitfield(srf_sampler_t* s, void* stream);

/*
 * OccupancySampler::sample_coords_from_dataset, occupancy_sampler.cu:1090-1143 (generate_training_samples_nerf, :513-689).
 * Offsets are the ones a one-thread-at-a-time execution of the reference kernel produces:
 * ray i's samples start at (*n_coords_counter before the call) + sum of the counts of rays < i.
 * coords (Coordinate records) may be NULL when only the side arrays are wanted; the side arrays
 * (sample_t, sample_dt: one float per sample; sample_cell: cell index + level * n_grid_elements) may be NULL too.
 */
int  srf_sampler_sample_coords_from_dataset(srf_sampler_t* s, uint32_t n_rays, uint32_t n_rays_shift, uint32_t n_coords,
                                            const srf_dataset* dataset, float* rays, float* rays_rgba,
                                            uint32_t* n_rays_counter, uint32_t* ray_coord_indices, float* coords,
                                            uint32_t* n_coords_counter, srf_pcg32 rng,
                                            float* sample_t, float* sample_dt, uint32_t* sample_cell, void* stream);

/* OccupancySampler::generate_rays_from_camera_matrix, occupancy_sampler.cu:1145-1188.
 * spp replaces CudaRenderBuffer::spp(). */
int  srf_sampler_generate_rays_from_camera_matrix(srf_sampler_t* s, const int32_t resolution[2], const float focal_length[2],
                                                  const float principal_point[2], const float camera_matrix_host[12],
                                                  srf_ray_payload* payload, uint32_t spp, void* stream);

/* OccupancySampler::generate_coords_from_rays, occupancy_sampler.cu:1190-1216 */
int  srf_sampler_generate_coords_from_rays(srf_sampler_t* s, uint32_t n_rays, uint32_t n_steps,
                                           srf_ray_payload* payloads, float* coords, void* stream);

/* ---------------- RayMarcher ---------------- */
void srf_marcher_config_default(srf_marcher_config* cfg);                       /* ray_marcher.cu:296-300 defaults */
int  srf_marcher_create(const srf_marcher_config* cfg, srf_marcher_t** out);    /* RayMarcher::RayMarcher, ray_marcher.cu:294 */
void srf_marcher_destroy(srf_marcher_t* m);
int  srf_marcher_get_config(const srf_marcher_t* m, srf_marcher_config* out);
int  srf_marcher_set_config(srf_marcher_t* m, const srf_marcher_config* cfg);

/* arguments of RayMarcher::volume_rendering_with_loss_and_gradient that are plain values (ray_marcher.h:19-52) */
typedef struct srf_loss_args {
	uint32_t n_rays;
	uint32_t n_max_compacted_coords;
	int32_t  padded_output_width;       /* stride (elements) of dloss_doutput records; network_output records are 4 wide as in the reference */
	int32_t  rgb_activation, density_activation;
	int32_t  loss_type;
	float    loss_scale;
	float    min_optical_thickness;
	int32_t  use_grid;
	float    background_color[3];
	int32_t  color_space;
	srf_pcg32 rng;
	int32_t  network_output_dtype;      /* SRF_DTYPE_*; the reference is F16 */
	int32_t  dloss_dtype;               /* SRF_DTYPE_*; the reference is F16 */
	uint32_t dt_stride;                 /* floats between consecutive samples' dt: 7 when `dt` points at coords[0].dt, 1 for a packed array */
} srf_loss_args;

/*
 * RayMarcher::volume_rendering_with_loss_and_gradient, ray_marcher.cu:303-374 (kernel :9-202).
 * dt points at the first sample's step size (see dt_stride).  coords / compacted_coords may both be NULL
 * to skip the Coordinate copy (ray_marcher.cu:174).  Compacted offsets are those of a one-thread-at-a-time
 * execution (exclusive prefix sum of the per-ray counts after early termination, starting at the counter's
 * value before the call).  density_grid_mean is the sampler's device float.  rgb_ray_out (3 floats per ray)
 * and loss_output may be NULL.
 */
int  srf_marcher_volume_rendering_with_loss_and_gradient(srf_marcher_t* m, const srf_loss_args* args,
        const float* rays_rgba, const uint32_t* n_rays_counter, uint32_t* ray_coord_indices,
        const float* dt, const float* coords, float* compacted_coords, uint32_t* n_compacted_coords_counter,
        const void* network_output, void* dloss_doutput, float* loss_output,
        const float* density_grid_mean, float* rgb_ray_out, void* stream);

/*
 * The same call for callers that must not allocate device memory while they run (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  It runs the single-launch implementation with its
 * scratch (the per-item status words, item lists and per-ray side array of the ordered-offset chain) in an array that is part of
 * the library's device image, about 1.8 MB on every GPU the library runs on, and calls no hipMalloc / hipFree.
 * Limits: n_rays <= SRF_NOALLOC_MAX_RAYS; no distortion regulariser; 64 consecutive rays whose samples need more than eight of the
 * kernel's windows of 1920 are composited on a slower path (same results); refused on a marcher that has left the streaming kernel
 * (after a failed chain, or created under SRF_COMPOSITE_IMPL).  All calls on one GPU, of whatever marcher, share the array and
 * the chain's error word in it: at most one such call may be in flight per GPU, and calls that overlap on one GPU (different
 * streams or threads) race.  Because the next call's preparation clears the shared error word, a marcher without a host-visible
 * error word of its own must call srf_marcher_sync_check before another marcher uses this entry point on the same GPU.
 * The first call on a device, and the first for each combination of data types and activations, does host-side look-ups (the
 * array's address, the kernel's occupancy): make those calls before a graph capture begins, not inside one.
 * Arguments, results and error reporting are those of srf_marcher_volume_rendering_with_loss_and_gradient.
 */
#define SRF_NOALLOC_MAX_RAYS 262144u
int  srf_marcher_volume_rendering_with_loss_and_gradient_noalloc(srf_marcher_t* m, const srf_loss_args* args,
        const float* rays_rgba, const uint32_t* n_rays_counter, uint32_t* ray_coord_indices,
        const float* dt, const float* coords, float* compacted_coords, uint32_t* n_compacted_coords_counter,
        const void* network_output, void* dloss_doutput, float* loss_output,
        const float* density_grid_mean, float* rgb_ray_out, void* stream);

typedef struct srf_render_args {
	uint32_t n_rays, n_steps, i_steps_offset;
	uint32_t padded_output_width;
	int32_t  density_activation, rgb_activation, render_mode;
	float    camera_matrix[12];
	float    depth_scale;
	int32_t  network_output_dtype;
} srf_render_args;

/* Waits for `stream` and reports whether the ordered-offset chain of the training compositing calls so far completed.
 * No counterpart in the reference (its offsets come from one atomicAdd per ray and cannot fail this way).
 * The streaming kernel's workgroups wait, with a bound, for the sample counts of the groups before theirs.  If a wait runs
 * out, that call's compacted counter reads 0xffffffff, every ray of the affected groups gets a zero count and no gradients, and
 * the failure is returned by this function or by the next srf_marcher_volume_rendering_with_loss_and_gradient on the marcher,
 * whichever comes first; from then on the marcher uses the wave-per-item kernel, whose items are handed out by a counter and so
 * never wait for a workgroup that is not running (and, should that kernel's waits run out as well, the three-launch
 * implementation, which has none). */
int  srf_marcher_sync_check(srf_marcher_t* m, void* stream);

/* RayMarcher::volume_rendering, ray_marcher.cu:376-415 (kernel :204-282) */
int  srf_marcher_volume_rendering(srf_marcher_t* m, const srf_sampler_t* s, const srf_render_args* args,
                                  srf_ray_payload* payloads, float* rgba, const float* coords, const void* rgbsigma, void* stream);

/* ---------------- orchestrator kernels ---------------- */
/* compact_rays_kernel, internal/testbed.cu:423-446; survivors keep their relative order. Counters are device uint32, caller-zeroed.
 * The marcher owns the scratch the ordered compaction needs (flags and positions, 16 bytes per ray). */
int  srf_compact_rays(srf_marcher_t* m, uint32_t n_elements, const srf_ray_payload* src_payloads, const float* src_rgba,
                      srf_ray_payload* dst_payloads, float* dst_rgba, srf_ray_payload* final_payloads, float* final_rgba,
                      uint32_t* n_alive_counter, uint32_t* n_final_counter, void* stream);
/* shade_kernel, internal/testbed.cu:448-477 */
int  srf_shade(uint32_t n_rays, const float* rgba, const srf_ray_payload* payloads, float* frame_buffer,
               int32_t render_mode, int32_t train_in_linear_colors, void* stream);
/* tcnn::fill_rollover / fill_rollover_and_rescale as launched at internal/testbed.cu:398-404 */
int  srf_fill_rollover(uint32_t n_elements, uint32_t stride_bytes, const uint32_t* n_input_elements, void* inout, void* stream);
int  srf_fill_rollover_and_rescale(uint32_t n_elements, uint32_t stride, const uint32_t* n_input_elements, void* inout, int32_t dtype, void* stream);

/*
 * Whole-frame render with a table-lookup stand-in for the network: Testbed::render_frame,
 * internal/testbed.cu:479-598, with NGPNetwork::inference_mixed_precision replaced by
 * rgbsigma = table[hash(cascade cell of the sample) & (table_size-1)].  One kernel marches and
 * composites each pixel's ray to completion, which yields the frame the reference's
 * compact / generate_coords / volume_rendering loop yields.  frame_buffer: resolution.x*resolution.y RGBA
 * floats (overwritten); n_samples (uint32 per pixel) may be NULL.
 */
typedef struct srf_field { const float* table; uint32_t table_size; uint32_t seed; } srf_field;
int  srf_render_frame_fused(srf_sampler_t* s, const srf_marcher_t* m, const srf_field* field,
                            const int32_t resolution[2], const float focal_length[2], const float principal_point[2],
                            const float camera_matrix_host[12], uint32_t spp, float* frame_buffer, uint32_t* n_samples, void* stream);
/* the stand-in evaluated over an array of Coordinate records (what the harness calls in place of the network) */
int  srf_field_eval(const srf_sampler_t* s, const srf_field* field, uint32_t n_coords, const float* coords,
                    void* rgbsigma, int32_t dtype, uint32_t padded_output_width, void* stream);
/* the same with the number of records read from device memory when the kernel starts (*n_coords_dev <= max_coords; NULL: max_coords) */
int  srf_field_eval_counted(const srf_sampler_t* s, const srf_field* field, const uint32_t* n_coords_dev, uint32_t max_coords, const float* coords,
                            void* rgbsigma, int32_t dtype, uint32_t padded_output_width, void* stream);

/* ---------------- a whole frame, library side ---------------- */
/* What a caller's network does between srf_sampler_generate_coords_from_rays and srf_marcher_volume_rendering
 * (m_network->inference_mixed_precision, internal/testbed.cu:552-556): n_elements coordinates of 7 floats in, one row of
 * padded_output_width values of `dtype` per coordinate out, enqueued on `stream`.  Returns 0, or a negative SRF_ERR_* code
 * (any other value is reported as SRF_ERR_INVALID). */
typedef int (*srf_inference_fn)(void* user, uint32_t n_elements, const float* coords, void* rgbsigma, int32_t dtype, uint32_t padded_output_width, void* stream);

/* What the caller's network does in Normals mode between inference and srf_marcher_volume_rendering
 * (m_network->input_gradient(stream, 3, coords, coords), internal/testbed.cu:558-560): the first three floats of each of the
 * n_elements coordinate records are overwritten with the density's gradient with respect to them, enqueued on `stream`.
 * Returns like srf_inference_fn. */
typedef int (*srf_input_gradient_fn)(void* user, uint32_t n_elements, float* coords, void* stream);

typedef struct srf_frame_args {
	int32_t  resolution[2];
	float    focal_length[2], principal_point[2];
	float    camera_matrix[12];          /* column-major 3x4, host memory */
	uint32_t spp;
	int32_t  render_mode, density_activation, rgb_activation;
	float    depth_scale;                /* 1 / scene_scale (testbed.cu:577) */
	int32_t  network_output_dtype;
	uint32_t padded_output_width;
	srf_input_gradient_fn input_gradient; /* called after inference when render_mode is SRF_RENDER_NORMALS (which is refused with */
	void*    input_gradient_user;         /* SRF_ERR_UNSUPPORTED when this is NULL); ignored in every other mode */
} srf_frame_args;

/* Testbed::render_frame up to and including shade_kernel, internal/testbed.cu:479-611: rays from the camera, then rounds of
 * compact_rays / generate_coords_from_rays / inference / volume_rendering with n_steps = clamp(n_pixels / n_alive, 1, 8) until no ray
 * is alive, then shade into frame_buffer (4 floats a pixel, cleared first).  The marcher owns the ray, coordinate and network-output
 * buffers.  Like the reference the host learns the number of rays left once a round: the compaction's last workgroup stores it into
 * mapped host memory and the calling thread polls that word (a busy wait on one host core, with hipStreamQuery every 4096 polls and a
 * copy plus hipStreamSynchronize should the word not arrive).  *n_iterations (may be NULL) receives the number of rounds. */
int  srf_render_frame(srf_sampler_t* s, srf_marcher_t* m, const srf_frame_args* args, srf_inference_fn inference, void* user,
                      float* frame_buffer, uint32_t* n_iterations, void* stream);

/* an srf_inference_fn that evaluates the stand-in field (srf_field_eval); user points at an srf_field_inference_ctx */
typedef struct srf_field_inference_ctx { const srf_sampler_t* sampler; const srf_field* field; } srf_field_inference_ctx;
int  srf_field_inference(void* user, uint32_t n_elements, const float* coords, void* rgbsigma, int32_t dtype, uint32_t padded_output_width, void* stream);
/* an srf_input_gradient_fn for the stand-in field (user as above): the position of each record becomes the first three values,
 * minus one half, of the table row that the field with seed ^ 0x9e3779b9 selects for it */
int  srf_field_input_gradient(void* user, uint32_t n_elements, float* coords, void* stream);

/*
 * srf_render_frame with the loop paced by the device.  The reference's loop (internal/testbed.cu:526-597) learns on the host, once a
 * round, how many rays are left, and sizes the round's launches by it; the GPU idles while the host finds out.  Here the numbers
 * of a round (rays left, n_steps, i_steps_offset) stay in device memory: the compaction writes them, the kernels of the round read
 * them, launched over an upper limit that the host knows (the last count it has seen arrive, which can only have fallen since).
 * The host runs a few rounds ahead of the device and stops launching once it sees a count of zero; rounds launched past the end
 * return at once.  The network therefore gets its element count as a device pointer plus an upper limit (at most resolution.x *
 * resolution.y): a network that needs the count on the host cannot be used here and goes through srf_render_frame.
 * input_gradient may be NULL except in Normals mode.  Frame and *n_iterations are those of srf_render_frame; the host waits for
 * the stream once, at the end, and only when n_iterations is not NULL.
 */
typedef int (*srf_inference_counted_fn)(void* user, const uint32_t* n_elements, uint32_t max_elements, const float* coords, void* rgbsigma,
                                        int32_t dtype, uint32_t padded_output_width, void* stream);
typedef int (*srf_input_gradient_counted_fn)(void* user, const uint32_t* n_elements, uint32_t max_elements, float* coords, void* stream);
int  srf_render_frame_paced(srf_sampler_t* s, srf_marcher_t* m, const srf_frame_args* args, srf_inference_counted_fn inference, void* user,
                            srf_input_gradient_counted_fn input_gradient, void* input_gradient_user,
                            float* frame_buffer, uint32_t* n_iterations, void* stream);
/* the stand-in field as such callbacks (user points at an srf_field_inference_ctx) */
int  srf_field_inference_counted(void* user, const uint32_t* n_elements, uint32_t max_elements, const float* coords, void* rgbsigma,
                                 int32_t dtype, uint32_t padded_output_width, void* stream);
int  srf_field_input_gradient_counted(void* user, const uint32_t* n_elements, uint32_t max_elements, float* coords, void* stream);

/* CudaRenderBuffer::accumulate, internal/utils/render_buffer.cu:46-85, :211-227: running mean of the frames of one view.  spp is the
 * number of frames already accumulated (0: the buffer is cleared first); the caller counts. */
enum { SRF_TONEMAP_IDENTITY = 0, SRF_TONEMAP_ACES = 1, SRF_TONEMAP_HABLE = 2, SRF_TONEMAP_REINHARD = 3 };
int  srf_frame_accumulate(const int32_t resolution[2], const float* frame_buffer, float* accumulate_buffer, uint32_t spp, int32_t color_space, void* stream);
/* CudaRenderBuffer::tonemap, internal/utils/render_buffer.cu:87-178, :229-235: exposure, background (sRGB, premultiplied by its alpha
 * through the remaining transparency), tone curve, output encoding.  out_rgba takes the place of the reference's CUDA surface. */
int  srf_frame_tonemap(const int32_t resolution[2], float exposure, const float background_color[4], const float* accumulate_buffer,
                       int32_t color_space, int32_t output_color_space, int32_t tonemap_curve, float* out_rgba, void* stream);

/* ---------------- test hooks ---------------- */
/* number of polls a workgroup of the streaming compositing kernel makes before it gives up waiting for its predecessors
 * (default 2^22).  0 lets a test exercise the give-up path without any kernel waiting for long. */
int  srf_marcher_debug_set_lookback_spin_limit(srf_marcher_t* m, uint32_t polls);
/* evaluates one of the shared elementary functions on the device over n inputs:
 * which = 0 exp, 1 log, 2 sin, 3 cos, 4 asin, 5 atan2(a,b), 6 pow(a,b), 7 sqrt, 8 a/b, 9 float->half->float,
 * 10 1/a (the reciprocal of the disparity stepping) */
int  srf_debug_eval_elem(int32_t which, uint32_t n, const float* a, const float* b, float* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif
