"""Pins of the oracle's display post-process (internal/utils/render_buffer.cu:46-178) against float64 statements of what the
kernels are for: a running mean, and exposure / background / published tone curves / sRGB encoding."""
import numpy as np
import pytest

from oracle import oracle as O

ID, ACES, HABLE, REINHARD = 0, 1, 2, 3


def _srgb_encode(x):
    """the reference's linear_to_srgb, exponent literal 0.41666 included (common_device.h)"""
    x = np.asarray(x, np.float64)
    return np.where(x < 0.0031308, 12.92 * x, 1.055 * np.power(np.maximum(x, 1e-300), 0.41666) - 0.055)


def _srgb_decode(s):
    s = np.asarray(s, np.float64)
    return np.where(s <= 0.04045, s / 12.92, np.power((s + 0.055) / 1.055, 2.4))


def test_accumulate_is_a_running_mean(orc):
    rng = np.random.default_rng(0)
    frames = rng.random((6, 50, 4)).astype(np.float32)
    for space, enc in ((O.COLOR_LINEAR, lambda x: x), (O.COLOR_SRGB, _srgb_encode)):
        acc = np.full((50, 4), 7.0, np.float32)        # whatever it held: the first frame (sample count 0) replaces it
        for k, f in enumerate(frames):
            orc.accumulate(f, acc, float(k), space)
            want = frames[:k + 1].astype(np.float64).copy()
            want[..., :3] = enc(want[..., :3])
            assert np.allclose(acc, want.mean(axis=0), rtol=2e-6, atol=1e-7)
    # VisPosNeg: red minus green is the signed value that is averaged; the mean goes back to red (positive) or green (negative)
    acc = np.zeros((50, 4), np.float32)
    signed = []
    for k, f in enumerate(frames):
        orc.accumulate(f, acc, float(k), O.COLOR_VISPOSNEG)
        signed.append(f[:, 0].astype(np.float64) - f[:, 1])
        m = np.mean(signed, axis=0)
        assert np.allclose(acc[:, 0], np.maximum(m, 0), atol=1e-6) and np.allclose(acc[:, 1], np.maximum(-m, 0), atol=1e-6)
        assert np.allclose(acc[:, 3], frames[:k + 1, :, 3].astype(np.float64).mean(axis=0), rtol=2e-6)


def test_tonemap_identity_exposure_and_background(orc):
    rng = np.random.default_rng(1)
    acc = rng.random((64, 4)).astype(np.float32)
    # nothing to do: opaque-or-not, a background with alpha 0 adds nothing; identity curve; linear in, linear out
    out = orc.tonemap(acc, 0.0, (0.3, 0.6, 0.9, 0.0), O.COLOR_LINEAR, O.COLOR_LINEAR, ID)
    assert np.array_equal(out, acc)
    # exposure is a power of two on the colour, not on alpha
    out = orc.tonemap(acc, 3.0, (0, 0, 0, 0.0), O.COLOR_LINEAR, O.COLOR_LINEAR, ID)
    assert np.array_equal(out[:, :3], acc[:, :3] * np.float32(8)) and np.array_equal(out[:, 3], acc[:, 3])
    # the background (given in sRGB) shows through what the pixel leaves transparent
    bg = np.array([0.2, 0.5, 0.8, 0.75])
    out = orc.tonemap(acc, 0.0, tuple(bg), O.COLOR_LINEAR, O.COLOR_LINEAR, ID).astype(np.float64)
    weight = (1 - acc[:, 3].astype(np.float64)) * bg[3]
    assert np.allclose(out[:, :3], acc[:, :3] + _srgb_decode(bg[:3])[None] * weight[:, None], rtol=1e-5, atol=1e-6)
    assert np.allclose(out[:, 3], acc[:, 3] + weight, rtol=1e-6)
    # output encoding, and an sRGB buffer that is decoded before the curve (background taken as it is)
    out = orc.tonemap(acc, 0.0, (0, 0, 0, 0.0), O.COLOR_LINEAR, O.COLOR_SRGB, ID)
    assert np.allclose(out[:, :3], _srgb_encode(acc[:, :3]), rtol=1e-5, atol=1e-6)
    out = orc.tonemap(acc, 0.0, (0.2, 0.5, 0.8, 1.0), O.COLOR_SRGB, O.COLOR_LINEAR, ID)
    blended = acc[:, :3].astype(np.float64) + np.array([0.2, 0.5, 0.8])[None] * (1 - acc[:, 3:4].astype(np.float64))
    assert np.allclose(out[:, :3], _srgb_decode(blended), rtol=2e-5, atol=1e-6)


def test_tone_curves_against_their_published_forms(orc):
    x = np.concatenate([np.linspace(0, 4, 97), [5.6, 11.2, -0.5]]).astype(np.float32)
    acc = np.stack([x, x[::-1], np.full_like(x, 0.25), np.ones_like(x)], axis=1).astype(np.float32)
    xs = np.maximum(acc[:, :3].astype(np.float64), 0)

    def run(curve):
        return orc.tonemap(acc, 0.0, (0, 0, 0, 0.0), O.COLOR_LINEAR, O.COLOR_LINEAR, curve)[:, :3].astype(np.float64)

    # Narkowicz's ACES fit x(2.51x + 0.03) / (x(2.43x + 0.59) + 0.14), on 0.6 x
    y = 0.6 * xs
    assert np.allclose(run(ACES), y * (2.51 * y + 0.03) / (y * (2.43 * y + 0.59) + 0.14), rtol=2e-5, atol=1e-6)
    # Hable's Uncharted 2 curve with exposure bias 2 and white point 11.2: h(2x) / h(11.2), h(v) = (v(Av + CB) + DE) / (v(Av + B) + DF) - E/F
    A, B, C, D, E, F = 0.15, 0.50, 0.10, 0.20, 0.02, 0.30
    h = lambda v: (v * (A * v + C * B) + D * E) / (v * (A * v + B) + D * F) - E / F
    assert np.allclose(run(HABLE), h(2 * xs) / h(11.2), rtol=5e-5, atol=2e-6)
    assert abs(orc.tonemap(np.array([[5.6, 0, 0, 1]], np.float32), 0.0, (0, 0, 0, 0.0), O.COLOR_LINEAR, O.COLOR_LINEAR, HABLE)[0, 0] - 1.0) < 1e-5
    # Reinhard on the Rec. 709 luminance
    Y = xs @ np.array([0.2126, 0.7152, 0.0722])
    assert np.allclose(run(REINHARD), xs / (1 + Y)[:, None], rtol=2e-6, atol=1e-7)
    # the identity curve does not even clamp
    assert np.array_equal(orc.tonemap(acc, 0.0, (0, 0, 0, 0.0), O.COLOR_LINEAR, O.COLOR_LINEAR, ID), acc)
