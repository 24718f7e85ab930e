"""Pins the numpy restatement of the reference's RMS-norm operators (oracle/norm.py)."""
import numpy as np
import pytest

from oracle.norm import fused_add_rms_norm, rms_norm


def module_form(x, w, eps):
    """weight * (x * rsqrt(mean(x^2) + eps)), the reference's module (layernorm.py:17-22), float64."""
    xf = x.astype(np.float64)
    return w.astype(np.float64) * (xf / np.sqrt((xf * xf).mean(-1, keepdims=True) + eps))


@pytest.mark.parametrize("hidden", [8, 100, 4096])
def test_matches_module_form(hidden):
    rng = np.random.default_rng(hidden)
    x = (rng.standard_normal((5, hidden)) * 3).astype(np.float16)
    w = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    got = rms_norm(x, w, 1e-6).astype(np.float64)
    np.testing.assert_allclose(got, module_form(x, w, 1e-6), rtol=2.5e-3, atol=1e-6)   # two fp16 roundings


def test_closed_forms():
    w = np.full(64, 0.5, np.float16)
    x = np.full((2, 64), -3.0, np.float16)
    assert np.array_equal(rms_norm(x, w, 0.0), np.full((2, 64), -0.5, np.float16))    # constant row -> sign * weight
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 256)).astype(np.float16)
    ones = np.ones(256, np.float16)
    y = rms_norm(x, ones, 0.0).astype(np.float64)
    np.testing.assert_allclose(np.sqrt((y * y).mean(-1)), 1.0, rtol=1e-3)            # unit RMS
    np.testing.assert_allclose(rms_norm((x * np.float16(4)).astype(np.float16), ones, 0.0).astype(np.float64), y,
                               rtol=2e-3, atol=1e-6)                                  # scale invariance
    big_eps = rms_norm(x, ones, 1e6).astype(np.float64)
    assert np.abs(big_eps).max() < 1e-2                                               # epsilon sits inside the root


def test_fused_equals_add_then_norm():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((4, 128)).astype(np.float16)
    r = rng.standard_normal((4, 128)).astype(np.float16)
    w = (1 + 0.1 * rng.standard_normal(128)).astype(np.float16)
    out, new_r = fused_add_rms_norm(x, r, w, 1e-5)
    s = x.astype(np.float32) + r.astype(np.float32)
    assert np.array_equal(new_r, s.astype(np.float16))
    np.testing.assert_allclose(out.astype(np.float64), module_form(s, w, 1e-5), rtol=3e-3, atol=1e-6)
