"""Pins the C restatement of the reference's fp32 CPU attention (oracle/cpu_attn.c):
float64 textbook softmax attention on whole sequences (the check the reference's own tests
use), closed forms, and a pure-Python brute force on tiny inputs."""
import math

import numpy as np
import pytest

from helpers import build_host_case, rows_of
from oracle.attention_ref import CpuAttention, textbook_attention, textbook_partials


def random_case(seed, n_seqs, shared, unique_max, c, H, d):
    rng = np.random.default_rng(seed)
    shared_ids = list(range(shared))
    sk = rng.standard_normal((shared, H, d)).astype(np.float32)
    sv = rng.standard_normal((shared, H, d)).astype(np.float32)
    toks, kv = [], []
    for s in range(n_seqs):
        u = int(rng.integers(0, unique_max + 1))
        toks.append(shared_ids + [10_000 * (s + 1) + i for i in range(u)] or [7])
        T = len(toks[-1])
        k = rng.standard_normal((T, H, d)).astype(np.float32)
        v = rng.standard_normal((T, H, d)).astype(np.float32)
        k[:min(shared, T)] = sk[:min(shared, T)]
        v[:min(shared, T)] = sv[:min(shared, T)]
        kv.append((k, v))
    return toks, kv


@pytest.mark.parametrize("blas", ["none", "auto"])
@pytest.mark.parametrize("partition", [0, 2])
@pytest.mark.parametrize("c,H,d,threads", [(4, 2, 8, 1), (8, 3, 16, 8), (32, 2, 128, 4)])
def test_matches_textbook(blas, partition, c, H, d, threads):
    toks, kv = random_case(1, 6, 3 * c + 1, 2 * c + 3, c, H, d)
    tree, kpool, vpool, order = build_host_case(toks, kv, c, H, d)
    rng = np.random.default_rng(2)
    q = rng.standard_normal((len(toks), H, d)).astype(np.float32)
    cpu = CpuAttention(blas)
    got = cpu.attention(q, rows_of(tree), kpool, vpool, partition, threads)
    want = textbook_attention(q, rows_of(tree), kpool, vpool)
    np.testing.assert_allclose(got, want, atol=2e-5, rtol=1e-4)
    # and per original sequence: attention over exactly the K/V that were inserted
    for i, sid in enumerate(order):
        k, v = kv[sid]
        for h in range(H):
            s = (k[:, h, :].astype(np.float64) @ q[i, h].astype(np.float64)) / math.sqrt(d)
            p = np.exp(s - s.max())
            p /= p.sum()
            np.testing.assert_allclose(got[i, h], p @ v[:, h, :].astype(np.float64), atol=2e-5, rtol=1e-4)


def test_locked_path_many_threads_few_heads():
    # H < threads takes the (chunk, head)-parallel branch with per-head locks
    toks, kv = random_case(3, 9, 16, 20, 8, 2, 16)
    tree, kpool, vpool, _ = build_host_case(toks, kv, 8, 2, 16)
    q = np.random.default_rng(4).standard_normal((9, 2, 16)).astype(np.float32)
    cpu = CpuAttention("none")
    a = cpu.attention(q, rows_of(tree), kpool, vpool, 0, 8)
    b = cpu.attention(q, rows_of(tree), kpool, vpool, 0, 1)
    np.testing.assert_allclose(a, b, atol=1e-5, rtol=1e-5)
    np.testing.assert_allclose(a, textbook_attention(q, rows_of(tree), kpool, vpool), atol=2e-5, rtol=1e-4)


@pytest.mark.parametrize("partition", [0, 2])
def test_closed_forms(partition):
    c, H, d = 4, 2, 8
    rng = np.random.default_rng(5)
    # (a) all keys equal -> uniform weights -> output is the mean of V
    T = 11
    k = np.tile(rng.standard_normal((1, H, d)).astype(np.float32), (T, 1, 1))
    v = rng.standard_normal((T, H, d)).astype(np.float32)
    # (b) a single token -> output is its value row
    k1 = rng.standard_normal((1, H, d)).astype(np.float32)
    v1 = rng.standard_normal((1, H, d)).astype(np.float32)
    tree, kpool, vpool, order = build_host_case([list(range(T)), [99]], [(k, v), (k1, v1)], c, H, d)
    q = rng.standard_normal((2, H, d)).astype(np.float32)
    got = CpuAttention("none").attention(q, rows_of(tree), kpool, vpool, partition, 2)
    np.testing.assert_allclose(got[order.index(0)], v.mean(axis=0), atol=1e-5)
    np.testing.assert_allclose(got[order.index(1)], v1[0], atol=1e-6)


def test_tiny_brute_force():
    c, H, d = 2, 1, 2
    k = np.array([[[1.0, 0.0]], [[0.0, 1.0]], [[1.0, 1.0]]], np.float32)
    v = np.array([[[1.0, 2.0]], [[3.0, 4.0]], [[5.0, 6.0]]], np.float32)
    q = np.array([[[2.0, 0.0]]], np.float32)
    tree, kpool, vpool, _ = build_host_case([[1, 2, 3]], [(k, v)], c, H, d)
    sc = [2.0 / math.sqrt(2), 0.0, 2.0 / math.sqrt(2)]
    w = [math.exp(x) for x in sc]
    want = [sum(w[i] * v[i, 0, e] for i in range(3)) / sum(w) for e in range(2)]
    for partition in (0, 1, 2):
        got = CpuAttention("none").attention(q, rows_of(tree), kpool, vpool, partition, 1)
        np.testing.assert_allclose(got[0, 0], want, atol=1e-6)


def test_bad_partition():
    tree, kpool, vpool, _ = build_host_case([[1]], [(np.ones((1, 1, 2), np.float32),) * 2], 2, 1, 2)
    with pytest.raises(RuntimeError):
        CpuAttention("none").attention(np.ones((1, 1, 2), np.float32), rows_of(tree), kpool, vpool, 3, 1)


def test_partials_consistent_with_whole_attention():
    # merging textbook per-chunk partials reproduces textbook attention (pins the partial helper)
    toks, kv = random_case(7, 4, 8, 5, 4, 2, 8)
    tree, kpool, vpool, _ = build_host_case(toks, kv, 4, 2, 8)
    q = np.random.default_rng(8).standard_normal((4, 2, 8)).astype(np.float32)
    rows = rows_of(tree)
    B, H, d = q.shape
    m = np.full((B, H), -np.inf)
    l = np.zeros((B, H))
    o = np.zeros((B, H, d))
    for (slot, nt, b, e) in rows:
        if nt == 0:
            continue
        pm, pl, po = textbook_partials(q, slot, nt, b, e, kpool, vpool)
        for i, s in enumerate(range(b, e)):
            for h in range(H):
                mn = max(m[s, h], pm[h, i])
                a, bb = math.exp(m[s, h] - mn), math.exp(pm[h, i] - mn)
                o[s, h] = a * o[s, h] + bb * po[h, i]
                l[s, h] = a * l[s, h] + bb * pl[h, i]
                m[s, h] = mn
    np.testing.assert_allclose(o / l[:, :, None], textbook_attention(q, rows, kpool, vpool), atol=1e-10)
