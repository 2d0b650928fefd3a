/*
 * CPU oracle for the occupancy-grid sampling / ray-marching / compositing path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C++ restatement of the reference's
 * CUDA kernels, executed sequentially (atomics become running counters in ray
 * order).  It exists to check the HIP kernels and to be timed as the CPU
 * baseline; nothing in the shipped library may call it.
 *
 * All pointers are host pointers.  Layouts follow the reference:
 *   Ray         6 floats  {o.xyz, d.xyz}                internal/utils/common.h:135-138
 *   Coordinate  7 floats  {pos.xyz, dt, dir.xyz}        internal/utils/common.h:150-155
 *   RayPayload  40 bytes  (orc_payload below)           internal/utils/common.h:158-165
 *   camera      12 floats, column major 3x4 {right, down, forward, origin}
 */
#ifndef SRF_ORACLE_H
#define SRF_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* enum values: internal/utils/common.h:61-115, internal/utils/loss.h:10-18 */
enum { ORC_ACT_NONE = 0, ORC_ACT_RELU = 1, ORC_ACT_LOGISTIC = 2, ORC_ACT_EXPONENTIAL = 3 };
enum { ORC_RENDER_AO = 0, ORC_RENDER_SHADE = 1, ORC_RENDER_NORMALS = 2, ORC_RENDER_DEPTH = 3, ORC_RENDER_DISTANCE = 4, ORC_RENDER_COST = 5 };
enum { ORC_COLOR_LINEAR = 0, ORC_COLOR_SRGB = 1, ORC_COLOR_VISPOSNEG = 2 };
enum { ORC_WARP_NGP = 0, ORC_WARP_MIPNERF360 = 1, ORC_WARP_DONERF = 2, ORC_WARP_SIGMOID = 3, ORC_WARP_ERP = 4, ORC_WARP_SINUSOIDAL = 5 };
enum { ORC_SAMPLING_ORIGINAL = 0, ORC_SAMPLING_DISPARITY = 1, ORC_SAMPLING_LOG = 2 };
enum { ORC_GRID_WARPED_EXP = 0, ORC_GRID_WARPED_RECIPROCAL = 1, ORC_GRID_METRIC_EXP = 2, ORC_GRID_METRIC_RECIPROCAL = 3 };
enum { ORC_REG_NONE = 0, ORC_REG_DISTORTION = 1 };
enum { ORC_LOSS_L2 = 0, ORC_LOSS_L1 = 1, ORC_LOSS_MAPE = 2, ORC_LOSS_SMAPE = 3, ORC_LOSS_SMOOTHL1 = 4, ORC_LOSS_LOGL1 = 5, ORC_LOSS_RELATIVEL2 = 6 };
enum { ORC_DTYPE_F16 = 0, ORC_DTYPE_F32 = 1 };

/* The sampler's public members (internal/sampler/occupancy_sampler.h:88-134). */
typedef struct orc_params {
	int32_t  warping_type;
	int32_t  griddist_type;
	int32_t  sampling_type;
	int32_t  use_grid;
	float    aabb_min[3];
	float    aabb_max[3];
	uint32_t aabb_scale;
	uint32_t grid_size[3];      /* cells along warped x (azimuth), y (polar), z (radial); the reference has one n_grid_size */
	uint32_t n_cascades;
	uint32_t n_max_steps;
	float    cone_angle_constant;
	float    min_cone_stepsize;
	float    max_cone_stepsize;
	float    near_distance;
	float    far_distance;
	int32_t  snap_to_pixel_centers_in_training;
	int32_t  snap_to_pixel_centers_in_rendering;
	float    min_optical_thickness;
	float    ema_decay;
} orc_params;

typedef struct orc_payload {
	uint8_t  alive;
	uint8_t  pad_[3];
	float    o[3];
	float    d[3];
	uint32_t idx;
	float    t;
	uint32_t n_steps;
} orc_payload;

typedef struct orc_pcg32 { uint64_t state, inc; } orc_pcg32;

typedef struct orc_dataset {
	uint32_t n_images;
	int32_t  resolution[2];
	float    focal_length[2];
	float    principal_point[2];
	const float*    xforms;                /* n_images x 12, column major */
	const uint16_t* images;                /* half RGBA per pixel, may be NULL (targets written as zeros) */
	const uint16_t* sampling_probability;  /* half per pixel, may be NULL (every pixel eligible) */
} orc_dataset;

int  orc_max_threads(void);
void orc_set_threads(int n);
/* 1 when transcendental calls go to glibc (-DSRF_ORACLE_LIBM build), 0 for the shared definitions */
int  orc_uses_libm(void);

/* ---- primitives (tiny-cuda-nn definitions, see the .cpp for provenance) ---- */
uint32_t orc_morton3d(uint32_t x, uint32_t y, uint32_t z);
uint32_t orc_morton3d_invert(uint32_t x);
void     orc_pcg32_seed(orc_pcg32* r, uint64_t initstate, uint64_t initseq);
void     orc_pcg32_default(orc_pcg32* r);
uint32_t orc_pcg32_next_uint(orc_pcg32* r);
float    orc_pcg32_next_float(orc_pcg32* r);
void     orc_pcg32_advance(orc_pcg32* r, int64_t delta);
uint32_t orc_sobol(uint32_t index, uint32_t dim);
float    orc_ld_random_val(uint32_t index, uint32_t seed, uint32_t dim);
void     orc_ld_random_pixel_offset(uint32_t spp, float out[2]);
float    orc_half_to_float(uint16_t h);
uint16_t orc_float_to_half(float f);

/* ---- scalar device helpers ---- */
float orc_elem(int which, float a, float b);   /* 0 exp 1 log 2 sin 3 cos 4 asin 5 atan2(a,b) 6 pow(a,b) 7 sqrt 8 a/b */
void  orc_params_default(orc_params* p);        /* occupancy_sampler.cu:909-944 defaults */
void  orc_params_finalize(orc_params* p, float aabb_scale, int min_step_given, int max_step_given);
void  orc_aabb_ray_intersect(const float mn[3], const float mx[3], const float o[3], const float d[3], float out[2]);
int   orc_aabb_contains(const float mn[3], const float mx[3], const float p[3]);
float orc_calc_dt(const orc_params* p, float t, float cone_angle);
void  orc_warp_position(const orc_params* p, const float pos[3], float out[3]);
void  orc_unwarp_position(const orc_params* p, const float wpos[3], float out[3]);
int   orc_level_from_pos(const orc_params* p, const float pos[3], const float wpos[3]);
uint32_t orc_cascaded_grid_idx_at(const orc_params* p, const float pos[3], const float wpos[3], uint32_t level);
int   orc_occupied_at(const orc_params* p, const uint8_t* bitfield, const float pos[3], const float wpos[3], uint32_t level);
void  orc_pixel_to_ray(const int32_t pixel[2], const int32_t res[2], const float focal[2], const float pp[2],
                       const float cam[12], uint32_t spp, int snap, float ray_out[6]);
float orc_network_to_rgb(float v, int act);
float orc_network_to_rgb_derivative(float v, int act);
float orc_network_to_density(float v, int act);
float orc_network_to_density_derivative(float v, int act);
float orc_srgb_to_linear(float v);
float orc_linear_to_srgb(float v);
void  orc_loss_and_gradient(int loss_type, const float target[3], const float pred[3], float loss[3], float grad[3]);

/* ---- grid maintenance ---- */
void  orc_generate_grid_samples(const orc_params* p, uint32_t n_elements, orc_pcg32 rng, uint32_t step,
                                const float* grid_in, float thresh, float* positions_out, uint32_t* indices_out);
void  orc_accumulate(uint32_t n_pixels, const float* frame_buffer, float* accumulate_buffer, float sample_count, int color_space);
void  orc_tonemap(uint32_t n_pixels, float exposure, const float background_color[4], const float* accumulate_buffer, int color_space,
                  int output_color_space, int tonemap_curve, float* out);
void  orc_mark_untrained_density_grid(const orc_params* p, uint32_t n_images, const int32_t resolution[2], const float focal_length[2],
                                      const float* xforms, float* grid_out);
void  orc_splat_grid_samples(const orc_params* p, uint32_t n_elements, const uint32_t* indices, uint32_t padded_output_width,
                             const void* network_output, int dtype, int density_activation, float* grid_current);
void  orc_ema_grid(uint32_t n_elements, const float* grid_current, float decay, float* grid);
float orc_grid_mean(const float* grid, uint32_t n_elements);
void  orc_grid_to_bitfield(uint32_t n_bytes, const float* grid, uint8_t* bitfield, float mean, float min_optical_thickness);
void  orc_bitfield_max_pool(const orc_params* p, const uint8_t* prev_level, uint8_t* next_level);
/* update_grid_bitfield as a whole (occupancy_sampler.cu:1063-1088); returns the mean */
float orc_update_grid_bitfield(const orc_params* p, const float* grid, uint8_t* bitfield);

/* ---- training sampler ---- */
void  orc_generate_training_samples(const orc_params* p, uint32_t n_rays, uint32_t n_rays_shift, uint32_t n_coords,
                                    const orc_dataset* ds, const uint8_t* bitfield, orc_pcg32 rng,
                                    uint32_t* ray_counter, uint32_t* numsteps_counter,
                                    float* rays_out, float* rays_rgba, uint32_t* numsteps_out, float* coords_out,
                                    float* sample_t_out, uint32_t* sample_cell_out, uint32_t* ray_src_index_out);

/* ---- rendering sampler ---- */
void  orc_init_rays_with_payload(const orc_params* p, const int32_t res[2], const float focal[2], const float pp[2],
                                 const float cam[12], uint32_t spp, orc_payload* payloads);
void  orc_advance_pos(const orc_params* p, uint32_t n_rays, uint32_t spp, orc_payload* payloads, const uint8_t* bitfield);
void  orc_generate_coords_from_rays(const orc_params* p, uint32_t n_rays, uint32_t n_steps, const uint8_t* bitfield,
                                    orc_payload* payloads, float* coords);

/* ---- compositing ---- */
typedef struct orc_loss_args {
	uint32_t n_rays;
	uint32_t n_max_compacted_coords;
	int32_t  padded_output_width;
	int32_t  rgb_activation, density_activation;
	int32_t  loss_type;
	float    loss_scale;
	int32_t  regularization_type;
	float    mean_density;
	float    min_optical_thickness;
	int32_t  use_grid;
	float    background_color[3];
	int32_t  color_space;
	int32_t  train_with_random_bg_color;
	int32_t  train_in_linear_color;
	float    transmittance_threshold;
	orc_pcg32 rng;
	int32_t  network_output_dtype;   /* ORC_DTYPE_* */
	int32_t  dloss_dtype;
	uint32_t dt_stride;              /* floats between consecutive samples' dt (7 for Coordinate records, 1 for a plain array) */
} orc_loss_args;

void  orc_volume_rendering_with_loss_and_gradient(const orc_loss_args* a,
        const float* rays_rgba, const uint32_t* n_rays_counter, uint32_t* ray_coord_indices,
        const float* dt, const float* coords /* may be NULL */, float* compacted_coords /* may be NULL */,
        uint32_t* n_compacted_coords_counter, const void* network_output, void* dloss_doutput,
        float* loss_output, float* reg_distortion_buffer, float* rgb_ray_out /* may be NULL, 3 per ray */);

typedef struct orc_render_args {
	uint32_t n_rays, n_steps, n_steps_offset;
	uint32_t padded_output_width;
	int32_t  density_activation, rgb_activation, render_mode;
	float    camera[12];
	float    depth_scale;
	float    transmittance_threshold;
	int32_t  network_output_dtype;
} orc_render_args;

void  orc_volume_rendering(const orc_params* p, const orc_render_args* a, orc_payload* payloads, float* rgba,
                           const float* coords, const void* network_output);

/* ---- orchestrator kernels (internal/testbed.cu:423-477) and tiny-cuda-nn fill_rollover ---- */
void  orc_compact_rays(uint32_t n, const orc_payload* src_payloads, const float* src_rgba,
                       orc_payload* dst_payloads, float* dst_rgba, orc_payload* final_payloads, float* final_rgba,
                       uint32_t* n_alive, uint32_t* n_final);
void  orc_shade(uint32_t n, const float* rgba, const orc_payload* payloads, float* frame_buffer, int render_mode, int train_in_linear_colors);
void  orc_fill_rollover(uint32_t n_out, uint32_t width_bytes, uint32_t n_in, uint8_t* buf);
void  orc_fill_rollover_and_rescale(uint32_t n_out, uint32_t width, uint32_t n_in, void* buf, int dtype);

/* ---- whole-frame render in the reference's loop order with a table-lookup stand-in for the network ---- */
typedef struct orc_field {
	const float* table;     /* table_size x 4 floats (r, g, b, sigma) */
	uint32_t     table_size; /* power of two */
	uint32_t     seed;
} orc_field;
void  orc_field_eval(const orc_params* p, const orc_field* f, const float wpos[3], float out[4]);
/* returns the number of loop iterations taken; frame is res.x*res.y*4 floats, zero-initialised by the callee */
uint32_t orc_render_frame(const orc_params* p, const orc_field* f, const uint8_t* bitfield,
                          const int32_t res[2], const float focal[2], const float pp[2], const float cam[12],
                          uint32_t spp, float transmittance_threshold, int train_in_linear_colors,
                          float* frame, uint32_t* n_samples_per_pixel /* may be NULL */);
/* stand-in for the network's input gradient: overwrites the position of one coordinate record (not in the reference) */
void  orc_field_input_gradient(const orc_params* p, const orc_field* f, float* coord);
/* the same loop in a given render mode (internal/testbed.cu:558-560: Normals mode replaces the coordinates by the input gradient) */
uint32_t orc_render_frame_mode(const orc_params* p, const orc_field* f, const uint8_t* bitfield,
                               const int32_t res[2], const float focal[2], const float pp[2], const float cam[12],
                               uint32_t spp, float transmittance_threshold, int train_in_linear_colors, int render_mode,
                               float* frame, uint32_t* n_samples_per_pixel /* may be NULL */);

#ifdef __cplusplus
}
#endif
#endif
