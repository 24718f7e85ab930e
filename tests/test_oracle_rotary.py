"""Pins the numpy restatement of the reference's rotary embedding (oracle/rotary.py).

The reference states the operator twice, independently: the kernel pairs elements
(pos_encoding_kernels.cu:24-50) and the module's `_forward` computes x*cos + rotate(x)*sin on
whole rows (rotary_embedding_vllm.py:29-40,95-135).  The second form is written out here in
float64 as the checker; a swapped pair, a wrong sign or the sine half of the cache read as
cosines fails it.  The rest is what a rotation fixes."""
import numpy as np
import pytest

from oracle.rotary import cos_sin_cache, rotary_embedding


def rotate_neox(x):
    h = x.shape[-1] // 2
    return np.concatenate([-x[..., h:], x[..., :h]], axis=-1)


def rotate_gptj(x):
    x1, x2 = x[..., ::2], x[..., 1::2]
    return np.stack([-x2, x1], axis=-1).reshape(x.shape)


def whole_row_form(positions, rows, head_size, cache, is_neox):
    """x*cos + rotate(x)*sin on the first rot_dim elements of each head, float64."""
    rot_dim = cache.shape[1]
    x = rows.astype(np.float64).reshape(rows.shape[0], -1, head_size)
    cs = cache[np.asarray(positions)].astype(np.float64)
    cos, sin = cs[:, :rot_dim // 2], cs[:, rot_dim // 2:]
    if is_neox:
        cos, sin = np.tile(cos, (1, 2)), np.tile(sin, (1, 2))
    else:
        cos, sin = np.repeat(cos, 2, axis=-1), np.repeat(sin, 2, axis=-1)
    rot = x[..., :rot_dim]
    fn = rotate_neox if is_neox else rotate_gptj
    out = x.copy()
    out[..., :rot_dim] = rot * cos[:, None, :] + fn(rot) * sin[:, None, :]
    return out.reshape(rows.shape)


def test_cache_layout_and_values():
    cache = cos_sin_cache(8, 50, base=10000.0)
    assert cache.shape == (50, 8) and cache.dtype == np.float16
    p, r = 7, 2
    f = 10000.0 ** (-2 * r / 8)
    assert abs(float(cache[p, r]) - np.cos(p * f)) < 1e-3
    assert abs(float(cache[p, 4 + r]) - np.sin(p * f)) < 1e-3
    assert np.all(cache[0, :4] == 1) and np.all(cache[0, 4:] == 0)


@pytest.mark.parametrize("is_neox", [True, False])
@pytest.mark.parametrize("head_size,rot_dim,n_heads,n_kv", [(128, 128, 4, 4), (64, 32, 3, 1), (16, 16, 2, 2)])
def test_matches_whole_row_form(is_neox, head_size, rot_dim, n_heads, n_kv):
    rng = np.random.default_rng(3)
    cache = cos_sin_cache(rot_dim, 300)
    n = 9
    pos = rng.integers(0, 300, n)
    q = rng.standard_normal((n, n_heads * head_size)).astype(np.float16)
    k = rng.standard_normal((n, n_kv * head_size)).astype(np.float16)
    gq, gk = rotary_embedding(pos, q, k, head_size, cache, is_neox)
    for got, src in ((gq, q), (gk, k)):
        want = whole_row_form(pos, src, head_size, cache, is_neox)
        # three fp16 roundings of values up to ~5: a few fp16 ulps
        np.testing.assert_allclose(got.astype(np.float64), want, atol=6e-3, rtol=2e-3)
        # fp32 steps instead of fp16 steps agree with float64 to fp16 output rounding
    gq32, _ = rotary_embedding(pos, q, None, head_size, cache, is_neox, step_dtype=np.float32)
    want = whole_row_form(pos, q, head_size, cache, is_neox)
    np.testing.assert_allclose(gq32.astype(np.float64), want, atol=2.5e-3, rtol=6e-4)


@pytest.mark.parametrize("is_neox", [True, False])
def test_position_zero_is_identity_and_passthrough(is_neox):
    rng = np.random.default_rng(4)
    cache = cos_sin_cache(16, 10)
    q = rng.standard_normal((3, 2 * 32)).astype(np.float16)
    got, _ = rotary_embedding([0, 0, 0], q, None, 32, cache, is_neox)
    assert np.array_equal(got, q)
    got, _ = rotary_embedding([5, 1, 9], q, None, 32, cache, is_neox)
    g3, q3 = got.reshape(3, 2, 32), q.reshape(3, 2, 32)
    assert np.array_equal(g3[..., 16:], q3[..., 16:])       # past rot_dim: untouched
    assert not np.array_equal(g3[..., :16], q3[..., :16])


@pytest.mark.parametrize("is_neox", [True, False])
def test_rotation_properties(is_neox):
    """Pair norms are kept; q_m . k_n depends on m - n only."""
    rng = np.random.default_rng(5)
    d = 64
    # exact cosines and sines in the cache's layout (the fp16 cache is only unitary to 1e-3)
    ang = np.arange(200, dtype=np.float64)[:, None] * 10000.0 ** (-np.arange(0, d, 2, dtype=np.float64) / d)
    cache = np.concatenate([np.cos(ang), np.sin(ang)], axis=-1)
    q = rng.standard_normal((1, d))
    k = rng.standard_normal((1, d))
    dots = []
    for m, n in ((10, 3), (57, 50), (107, 100)):
        gq, _ = rotary_embedding([m], q, None, d, cache, is_neox, step_dtype=np.float64)
        gk, _ = rotary_embedding([n], k, None, d, cache, is_neox, step_dtype=np.float64)
        dots.append(float((gq[0] * gk[0]).sum()))
        if is_neox:
            pair = lambda a: a[0, :d // 2] ** 2 + a[0, d // 2:] ** 2
        else:
            pair = lambda a: a[0, ::2] ** 2 + a[0, 1::2] ** 2
        np.testing.assert_allclose(pair(gq.astype(np.float64)), pair(q.astype(np.float64)), rtol=1e-9)
    assert abs(dots[0] - dots[1]) < 1e-9 and abs(dots[0] - dots[2]) < 1e-9
