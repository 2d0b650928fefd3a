"""The disparity chain of the marching kernels in its short form (sphericalrf_amd/csrc/srf_bodies.h: ShortForm, ShortChain).

The reference steps t by calc_dt (internal/sampler/occupancy_sampler.cu:287-331): dt = 1/(c + 1/t) - t with two correctly
rounded divisions.  The kernels walk long stretches of that chain and carry the reciprocal of t from step to step, which
rests on two facts checked here on the host with IEEE arithmetic:
  * one fused Newton step from g gives the correctly rounded 1/RN(1/g), for every mantissa of g;
  * inside the short form's range the chain of t is, bit for bit, the chain of calc_dt.
"""
import ctypes as C

import numpy as np
import pytest

from tests.helpers import ptr
from oracle import oracle as O


def test_carried_reciprocal_is_correctly_rounded_for_every_mantissa(hostsim):
    hostsim.lib.hs_carried_reciprocal_failures.restype = C.c_uint32
    assert hostsim.lib.hs_carried_reciprocal_failures() == 0


@pytest.mark.parametrize("near,far,n_steps", [(0.05, 100.0, 2048), (0.2, 100.0, 2048), (0.1, 16.0, 256), (0.05, 1000.0, 1024), (0.5, 3.0, 64), (0.01, 1e4, 4096)])
def test_short_chain_is_the_chain_of_calc_dt(orc, hostsim, near, far, n_steps):
    p = orc.params(aabb_scale=64, grid_size=(16, 16, 16), n_cascades=1, warping_type=O.WARP_ERP, griddist_type=O.GRID_WARPED_EXP,
                   sampling_type=O.SAMPLING_DISPARITY, near_distance=near, far_distance=far, n_max_steps=n_steps)
    hostsim.lib.hs_disparity_chains.restype = C.c_uint32
    rng = np.random.default_rng(n_steps)
    c = (1.0 / far - 1.0 / near) / n_steps
    t_hi = 0.49 / -c
    covered = 0
    for _ in range(40):
        # starts spread in reciprocal space like the rays' own, from the near plane up to the end of the short form's range
        t0 = np.float32(1.0 / rng.uniform(1.0 / min(far, t_hi), 1.0 / near))
        n = n_steps + 8
        t_calc, t_short = np.zeros(n, np.float32), np.zeros(n, np.float32)
        taken = hostsim.lib.hs_disparity_chains(C.byref(p), C.c_float(t0), n, ptr(t_calc), ptr(t_short))
        assert taken >= 1
        assert np.array_equal(t_short[:taken].view(np.uint32), t_calc[:taken].view(np.uint32))
        assert np.all(np.diff(t_short[:taken]) > 0)
        # the short form covers the chain up to 0.49/|c| (or to its end)
        assert taken == n or t_short[taken - 2] <= t_hi < t_short[taken - 1] * 2
        covered += taken
    assert covered > 40 * min(n_steps, 64) // 4


def test_many_additions_at_once_equal_the_loop(hostsim):
    """short_chain_jump (srf_bodies.h): the k additions r <- c + r that end at or below S, in closed form on the mantissas, against the
    loop itself; operands over every binade and step size, including steps exactly halfway between two floats, which it must decline"""
    hostsim.lib.hs_chain_jump_mismatches.restype = C.c_uint32
    out = (C.c_uint32 * 2)()
    assert hostsim.lib.hs_chain_jump_mismatches(3, 400000, out) == 0
    assert out[0] > 100000 and 1000 < out[1] < out[0]


def test_wide_march_bookkeeping_matches_the_step_by_step_loop(hostsim):
    """wide_apply (64 steps of one ray at once, srf_bodies.h) against the loop of occupancy_sampler.cu:595-632 taken a step
    at a time, on random batches that include the exits the marches of the other tests rarely reach: the sample cap in
    the middle of a batch, a zero step, leaving the box, logs that are too short."""
    hostsim.lib.hs_wide_apply_mismatches.restype = C.c_uint32
    assert hostsim.lib.hs_wide_apply_mismatches(11, 200000) == 0


def test_table_driven_generator_skip_ahead_equals_the_plain_one(hostsim):
    """pcg_advance_u32 (one multiply-add per set bit of the distance) and pcg_advance_skip16 (one per hexadecimal digit,
    srf_device.h) against pcg_advance, the reference generator's own skip-ahead (pcg32.h advance), over random streams,
    states and distances."""
    hostsim.lib.hs_pcg_skip_mismatches.restype = C.c_uint32
    assert hostsim.lib.hs_pcg_skip_mismatches(5, 20000) == 0


def test_reciprocal_of_the_reciprocal_is_the_number_itself_below_sqrt_two():
    """what lets the render marches replace chained steps by additions: for every float g with a mantissa below sqrt 2,
    RN(1/RN(1/g)) == g; above it the identity fails for about three mantissas in ten, by one ulp either way"""
    m = np.arange(1 << 23, dtype=np.uint32)
    one = np.float32(1.0)
    for exponent in (0x3f800000, 0x41000000, 0x3c000000):          # [1, 2), [8, 16), [2^-7, 2^-6)
        g = (np.uint32(exponent) | m).view(np.float32)
        back = one / (one / g)
        same = back == g
        below = g < np.float32(1.4142134) * (np.uint32(exponent)).view(np.float32)
        assert same[below].all() and below.sum() > 3_400_000
        assert 0.25 < (~same[~below]).mean() < 0.35
