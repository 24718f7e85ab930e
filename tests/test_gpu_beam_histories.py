"""Random histories that mix the beam-search operations (duplicate, append_completion) with
insertion, decode appends and removal on the GPU cache: after every few operations each
sequence's attention output must equal textbook attention over that sequence's own K/V history,
kept beside the cache as plain arrays, and the native tree must equal the oracle's."""
import random

import numpy as np
import pytest

from chunk_attn import capi
from gpu_helpers import ATOL, RTOL, make_attention, to_dev
from oracle.prefix_tree import PrefixTree

pytestmark = pytest.mark.gpu

H = 2


def textbook(q, k, v):
    sc = np.einsum("hd,thd->ht", q.astype(np.float64), k.astype(np.float64)) / np.sqrt(128.0)
    p = np.exp(sc - sc.max(axis=1, keepdims=True))
    return np.einsum("ht,thd->hd", p / p.sum(axis=1, keepdims=True), v.astype(np.float64))


def run_history(seed, c, n_ops=50):
    rng = random.Random(seed)
    nrng = np.random.default_rng(seed)

    def rows(n):
        return (nrng.standard_normal((n, H, 128)).astype(np.float16), nrng.standard_normal((n, H, 128)).astype(np.float16))

    attn = make_attention(H, c, 900)
    ora = PrefixTree(c, attn.max_chunks)
    family = [rng.randint(0, 50) for _ in range(4 * c)]
    fk, fv = rows(len(family))
    hist = []                                                  # per sequence (k, v)
    for op_i in range(n_ops):
        r = rng.random()
        n = len(hist)
        if r < 0.25 or n == 0:
            cut, extra = rng.randint(1, len(family)), rng.randint(0, c + 3)
            toks = family[:cut] + [1000 + rng.randint(0, 10 ** 6) for _ in range(extra)]
            ek, ev = rows(extra)
            k, v = np.concatenate([fk[:cut], ek]), np.concatenate([fv[:cut], ev])
            idx = attn.add_seq(toks, to_dev(k), to_dev(v))
            assert idx == ora.add_seq(toks)[0]
            hist.insert(idx, (k, v))
        elif r < 0.45:
            toks = [2 * 10 ** 6 + rng.randint(0, 10 ** 6) for _ in range(n)]
            k, v = rows(n)
            attn.append_token(toks, to_dev(k), to_dev(v))
            ora.append_token(toks)
            hist = [(np.concatenate([hk, k[i:i + 1]]), np.concatenate([hv, v[i:i + 1]])) for i, (hk, hv) in enumerate(hist)]
        elif r < 0.6 and n < 40:
            i, copies = rng.randrange(n), rng.randint(1, 3)
            attn.duplicate(i, copies)
            ora.duplicate(i, copies)
            hist[i + 1:i + 1] = [hist[i]] * copies
        elif r < 0.85 and n < 40:
            i, cand = rng.randrange(n), rng.randint(1, 4)
            toks = [3 * 10 ** 6 + rng.randint(0, 10 ** 6) for _ in range(cand)]
            k, v = rows(cand)
            attn.append_completion(i, toks, to_dev(k), to_dev(v))
            ora.append_completion(i, toks)
            base = hist[i]
            hist[i:i + 1] = [(np.concatenate([base[0], k[j:j + 1]]), np.concatenate([base[1], v[j:j + 1]])) for j in range(cand)]
        else:
            i = rng.randrange(n)
            attn.remove_seq(i)
            ora.remove_seq(i)
            del hist[i]
        if op_i % 5 == 4 and hist:
            orows = np.array([x.as_tuple() for x in ora.get_chunks()], np.int32).reshape(-1, 4)
            np.testing.assert_array_equal(attn.get_chunks(), orows)
            q = nrng.standard_normal((len(hist), H, 128)).astype(np.float16)
            for partition in (0, 2):
                out = attn.forward(to_dev(q), partition).float().cpu().numpy()
                for s, (k, v) in enumerate(hist):
                    np.testing.assert_allclose(out[s], textbook(q[s], k, v), atol=ATOL, rtol=RTOL)
    attn.clear()
    assert attn.tree.used_chunks == 0


@pytest.mark.parametrize("seed,c", [(0, 32), (1, 64), (2, 128), (3, 32)])
def test_beam_history(seed, c):
    run_history(seed, c)
