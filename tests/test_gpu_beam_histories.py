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


def test_chunk_copies_and_row_writes_in_one_launch():
    """ca_copy_chunks / ca_copy_chunks_put_rows against the same steps done one after the other
    with tensor assignments (reference Chunk::deep_copy, chunk.cpp:93-107, and the row appends of
    Attention::append_completion, attention.cpp:243,253): the beam-search shape (every candidate's
    row at the same index of its own copy: one launch), shapes that take two launches (a row
    written in a source chunk only), and what is rejected."""
    import torch
    c, n_slots = 32, 12
    attn = make_attention(H, c, n_slots)
    rng = torch.Generator(device="cuda").manual_seed(11)
    kp, vp = attn.pool_views()
    st = torch.cuda.current_stream().cuda_stream
    k = torch.randn((4, H, 128), device="cuda", generator=rng).half()
    v = torch.randn((4, H, 128), device="cuda", generator=rng).half()
    cases = [
        ([(0, 5), (0, 6), (0, 7)], [(0, 9), (5, 9), (6, 9), (7, 9)]),    # a beam step with four candidates
        ([(1, 8)], [(1, 31), (8, 31), (8, 0)]),                          # two written rows in one destination
        ([(2, 9), (3, 10)], [(2, 4), (10, 4)]),                          # row of a source only: copies first, then rows
        ([(2, 9)], [(9, 1), (9, 2), (9, 3)]),                            # three rows in one chunk: two launches
        ([(4, 11)], []),
        ([], [(4, 0), (11, 31)]),
    ]
    for pairs, targets in cases:
        kp.copy_(torch.randn(kp.shape, device="cuda", generator=rng).half())
        vp.copy_(torch.randn(vp.shape, device="cuda", generator=rng).half())
        want_k, want_v = kp.clone(), vp.clone()
        for src, dst in pairs:
            want_k[dst] = want_k[src]
            want_v[dst] = want_v[src]
        for i, (slot, row) in enumerate(targets):
            want_k[slot, :, row] = k[i]
            want_v[slot, :, row] = v[i]
        attn.ctx.copy_chunks_put_rows(pairs, k.data_ptr(), v.data_ptr(), targets, st)
        torch.cuda.synchronize()
        assert torch.equal(kp, want_k) and torch.equal(vp, want_v), (pairs, targets)
    # the plain copy entry points
    before_k, before_v = kp.clone(), vp.clone()
    attn.ctx.copy_chunks([(0, 3), (1, 4), (2, 5)], st)
    attn.ctx.copy_chunk(6, 7, st)
    torch.cuda.synchronize()
    for src, dst in ((0, 3), (1, 4), (2, 5), (6, 7)):
        assert torch.equal(kp[dst], before_k[src]) and torch.equal(vp[dst], before_v[src])
    for untouched in (0, 1, 2, 6, 8, 9, 10, 11):
        assert torch.equal(kp[untouched], before_k[untouched])
    for bad in ([(0, 1), (1, 2)], [(0, 2), (1, 2)], [(3, 3)], [(0, attn.max_chunks)]):
        with pytest.raises(capi.ChunkAttnError) as e:
            attn.ctx.copy_chunks(bad, st)
        assert e.value.code == -1
    with pytest.raises(capi.ChunkAttnError):
        attn.ctx.copy_chunks_put_rows([(0, 1)], k.data_ptr(), v.data_ptr(), [(0, c)], st)


def test_more_chunk_copies_and_rows_than_one_launch_takes():
    """70 chunk pairs and 70 rows: more than the 64 of either that one launch's argument block
    holds, so the calls split their work over several launches; same result as tensor assignments."""
    import torch
    c, n = 32, 70
    attn = make_attention(H, c, 2 * n + 4)
    rng = torch.Generator(device="cuda").manual_seed(12)
    kp, vp = attn.pool_views()
    st = torch.cuda.current_stream().cuda_stream
    kp.copy_(torch.randn(kp.shape, device="cuda", generator=rng).half())
    vp.copy_(torch.randn(vp.shape, device="cuda", generator=rng).half())
    k = torch.randn((n, H, 128), device="cuda", generator=rng).half()
    v = torch.randn((n, H, 128), device="cuda", generator=rng).half()
    pairs = [(i, n + i) for i in range(n)]
    targets = [(n + i, (7 * i) % c) for i in range(n)]
    want_k, want_v = kp.clone(), vp.clone()
    for src, dst in pairs:
        want_k[dst], want_v[dst] = want_k[src], want_v[src]
    for i, (slot, row) in enumerate(targets):
        want_k[slot, :, row], want_v[slot, :, row] = k[i], v[i]
    attn.ctx.copy_chunks_put_rows(pairs, k.data_ptr(), v.data_ptr(), targets, st)
    torch.cuda.synchronize()
    assert torch.equal(kp, want_k) and torch.equal(vp, want_v)
    # the copies alone, back again
    attn.ctx.copy_chunks([(n + i, i) for i in range(n)], st)
    torch.cuda.synchronize()
    assert torch.equal(kp[:n], want_k[n:2 * n]) and torch.equal(vp[:n], want_v[n:2 * n])
