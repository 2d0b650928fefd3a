"""Do the pins bite?  Each entry below is a plausible one-line slip in oracle/srf_oracle.cpp (a wrong stride, swapped operands, a
dropped term).  The altered source is compiled into a scratch directory, loaded beside the real oracle, and the pin named with
the entry must FAIL on it.  The real oracle source is never touched."""
import os
import subprocess

import pytest

from oracle import oracle as O
from tests import test_oracle_pins as pins

ORACLE_DIR = os.path.dirname(os.path.abspath(O.__file__))
SOURCE = os.path.join(ORACLE_DIR, "srf_oracle.cpp")

# (name, text in the source (must occur exactly once), replacement, pin that has to fail, reference lines the text restates)
MUTATIONS = [
    ("training_rng_stride", "pcg_advance(rng, (int64_t)(uint32_t)(i * 8u));", "pcg_advance(rng, (int64_t)(uint32_t)(i * 4u));",
     pins.pin_training_rays, "occupancy_sampler.cu:563"),
    ("pixel_draws_swapped", "xy[0] = pcg_next_float(rng);\n\t\txy[1] = pcg_next_float(rng);", "xy[1] = pcg_next_float(rng);\n\t\txy[0] = pcg_next_float(rng);",
     pins.pin_training_rays, "occupancy_sampler.cu:564"),
    ("start_jitter_constant", "startt += calc_dt(P, startt, cone_angle) * pcg_next_float(rng);", "startt += calc_dt(P, startt, cone_angle) * 0.5f;",
     pins.pin_training_rays, "occupancy_sampler.cu:590"),
    ("near_plane_dropped", "tmm[0] = fmaxf(tmm[0], P.near_distance);", "",
     pins.pin_training_rays, "occupancy_sampler.cu:587"),
    ("principal_point_ignored_x", "(xy[0] - ds->principal_point[0])", "(xy[0] - 0.5f)",
     pins.pin_training_rays, "occupancy_sampler.cu:577-581"),
    ("principal_point_ignored_y", "(xy[1] - ds->principal_point[1])", "(xy[1] - 0.5f)",
     pins.pin_training_rays, "occupancy_sampler.cu:577-581"),
    ("focal_axes_swapped", "(float)res[0] / ds->focal_length[0]", "(float)res[0] / ds->focal_length[1]",
     pins.pin_training_rays, "occupancy_sampler.cu:577-581"),
    ("target_pixel_index_transposed",
     "uint64_t pidx = (uint64_t)px + (uint64_t)py * (uint64_t)res[0] + (uint64_t)s.img * (uint64_t)res[0] * (uint64_t)res[1];",
     "uint64_t pidx = (uint64_t)py + (uint64_t)px * (uint64_t)res[1] + (uint64_t)s.img * (uint64_t)res[0] * (uint64_t)res[1];",
     pins.pin_training_rays, "common_device.h:191-213"),
    ("probability_pixel_index_transposed",
     "uint64_t pidx = (uint64_t)px + (uint64_t)py * (uint64_t)res[0] + (uint64_t)img * (uint64_t)res[0] * (uint64_t)res[1];",
     "uint64_t pidx = (uint64_t)py + (uint64_t)px * (uint64_t)res[1] + (uint64_t)img * (uint64_t)res[0] * (uint64_t)res[1];",
     pins.pin_sampling_probability_pixel, "occupancy_sampler.cu:569"),
    ("probability_test_sign", "if (half_to_float(ds->sampling_probability[pidx]) <= 0.f) continue;", "if (half_to_float(ds->sampling_probability[pidx]) > 0.f) continue;",
     pins.pin_sampling_probability_pixel, "occupancy_sampler.cu:570"),
    ("nan_probability_skipped", "if (half_to_float(ds->sampling_probability[pidx]) <= 0.f) continue;", "if (!(half_to_float(ds->sampling_probability[pidx]) > 0.f)) continue;",
     pins.pin_sampling_probability_pixel, "occupancy_sampler.cu:571"),
    ("snap_without_half_pixel", "xy[a] = ((float)px + 0.5f) / (float)res[a];", "xy[a] = ((float)px) / (float)res[a];",
     pins.pin_training_rays, "occupancy_sampler.cu:566"),
    ("snap_always", "if (P.snap_to_pixel_centers_in_training) {", "if (true) {",
     pins.pin_training_rays_without_snapping, "occupancy_sampler.cu:565"),
    ("entry_point_ignored", "float startt = tmm[0];", "float startt = P.near_distance;",
     pins.pin_training_rays_entering_the_box, "occupancy_sampler.cu:585-589"),
    ("grid_sample_rng_stride", "pcg_advance(rng, (int64_t)(uint32_t)(i * 4u));", "pcg_advance(rng, (int64_t)(uint32_t)(i * 3u));",
     pins.pin_grid_sample_draws, "occupancy_sampler.cu:125"),
    ("grid_sample_level_not_drawn", "uint32_t level = (uint32_t)(pcg_next_float(rng) * (float)P.n_cascades) % P.n_cascades;",
     "uint32_t level = i % P.n_cascades; (void)pcg_next_float(rng);",
     pins.pin_grid_sample_draws, "occupancy_sampler.cu:126"),
    ("grid_sample_jitter_order", "float rx = pcg_next_float(rng), ry = pcg_next_float(rng), rz = pcg_next_float(rng);",
     "float rz = pcg_next_float(rng), ry = pcg_next_float(rng), rx = pcg_next_float(rng);",
     pins.pin_grid_sample_draws, "occupancy_sampler.cu:147"),
    ("grid_sample_cascade_scale", "pos = pos * srf_exp2i(-(int)(P.n_cascades - level - 1));\n\t\t\tpos = pos + V3{0.5f, 0.5f, 0.5f};\n\t\t\tbreak;\n\t\tcase ORC_GRID_WARPED_RECIPROCAL:",
     "pos = pos * srf_exp2i(-(int)(P.n_cascades - level));\n\t\t\tpos = pos + V3{0.5f, 0.5f, 0.5f};\n\t\t\tbreak;\n\t\tcase ORC_GRID_WARPED_RECIPROCAL:",
     pins.pin_grid_sample_draws, "occupancy_sampler.cu:153"),
    ("grid_sample_retry_ignores_cascade", "idx += level * n_grid_elements;\n\t\t\tif (grid_in[idx] > thresh) break;", "if (grid_in[idx] > thresh) { idx += level * n_grid_elements; break; }\n\t\t\tidx += level * n_grid_elements;",
     pins.pin_grid_sample_retries, "occupancy_sampler.cu:131-135"),
    ("background_behind_terminated_rays", "if (n == f.numsteps) rgb_ray = rgb_ray + T * bg;", "rgb_ray = rgb_ray + T * bg;",
     pins.pin_background_only_behind_unterminated_rays, "ray_marcher.cu:106-109"),
    ("background_not_linearised", "V3 bg{srgb_to_linear(bg_in.x), srgb_to_linear(bg_in.y), srgb_to_linear(bg_in.z)};", "V3 bg{bg_in.x, bg_in.y, bg_in.z};",
     pins.pin_background_only_behind_unterminated_rays, "ray_marcher.cu:86"),
    ("srgb_target_not_unpremultiplied", "V3 q{linear_to_srgb(tex[0] / tex[3]), linear_to_srgb(tex[1] / tex[3]), linear_to_srgb(tex[2] / tex[3])};",
     "V3 q{linear_to_srgb(tex[0]), linear_to_srgb(tex[1]), linear_to_srgb(tex[2])};",
     pins.pin_srgb_target_unpremultiplies, "ray_marcher.cu:99"),
    ("srgb_target_zero_alpha", "} else target = bg;", "} else target = v3(tex);",
     pins.pin_srgb_target_unpremultiplies, "ray_marcher.cu:101"),
    ("linear_target_not_converted", "if (!a.train_in_linear_color) {\n\t\t\t\ttarget = V3{linear_to_srgb(target.x), linear_to_srgb(target.y), linear_to_srgb(target.z)};",
     "if (!a.train_in_linear_color) {",
     pins.pin_srgb_target_unpremultiplies, "ray_marcher.cu:93-95"),
    ("loss_output_not_normalised", "if (loss_output) loss_output[i] = mean_loss / (float)a.n_rays;", "if (loss_output) loss_output[i] = mean_loss;",
     pins.pin_loss_output_is_divided_by_n_rays, "ray_marcher.cu:131"),
    ("loss_scale_not_normalised", "const float loss_scale = a.loss_scale / (float)a.n_rays;", "const float loss_scale = a.loss_scale;",
     pins.pin_loss_output_is_divided_by_n_rays, "ray_marcher.cu:133"),
    ("exponential_rgb_regulariser_off", "const float output_l2_reg = a.rgb_activation == ORC_ACT_EXPONENTIAL ? 1e-4f : 0.0f;", "const float output_l2_reg = 0.0f;",
     pins.pin_exponential_rgb_regulariser, "ray_marcher.cu:135"),
    ("regulariser_for_every_activation", "const float output_l2_reg = a.rgb_activation == ORC_ACT_EXPONENTIAL ? 1e-4f : 0.0f;", "const float output_l2_reg = 1e-4f;",
     pins.pin_exponential_rgb_regulariser, "ray_marcher.cu:135"),
    ("mean_over_every_cascade", "const float mean = orc_grid_mean(grid, nc);", "const float mean = orc_grid_mean(grid, nc * P.n_cascades);",
     pins.pin_bitfield_mean_is_cascade_zero_only, "occupancy_sampler.cu:1066-1070"),
    ("mean_counts_masked_cells", "t4[k] = e < n_elements ? fmaxf(grid[e], 0.f) / denom : 0.f;", "t4[k] = e < n_elements ? grid[e] / denom : 0.f;",
     pins.pin_bitfield_mean_is_cascade_zero_only, "occupancy_sampler.cu:1069"),
]


def _flags():
    """oracle/Makefile's flags, without optimisation: the pins are small and the build is what takes time"""
    return ["-O0", "-std=c++17", "-fPIC", "-fopenmp", "-ffp-contract=off", "-fno-fast-math", "-mfma", "-msse4.1", "-shared"]


@pytest.fixture(scope="module")
def source():
    with open(SOURCE) as f:
        return f.read()


@pytest.mark.parametrize("name,old,new,pin,where", MUTATIONS, ids=[m[0] for m in MUTATIONS])
def test_a_wrong_oracle_fails_its_pin(name, old, new, pin, where, source, tmp_path, orc):
    assert source.count(old) == 1, "the text of mutation %s must occur exactly once in srf_oracle.cpp (found %d)" % (name, source.count(old))
    mutant_src = tmp_path / "srf_oracle.cpp"
    mutant_src.write_text(source.replace(old, new))
    lib = tmp_path / ("liboracle_%s.so" % name)
    cmd = [os.environ.get("CXX", "g++")] + _flags() + ["-I", ORACLE_DIR, "-I", os.path.join(ORACLE_DIR, "..", "sphericalrf_amd", "csrc"),
                                                         "-o", str(lib), str(mutant_src)]
    subprocess.run(cmd, check=True)
    mutant = O.Oracle(path=str(lib))
    pin(orc)                                   # the real oracle passes ...
    with pytest.raises(AssertionError):        # ... and the wrong one (restating %s wrongly) does not
        pin(mutant)
