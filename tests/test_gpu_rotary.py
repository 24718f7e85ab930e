"""GPU parity of the rotary operator and of the fused rotate-and-append decode step, called
through the C-ABI, against the numpy oracle (oracle/rotary.py) and float64 arithmetic.

Tolerances: against the oracle, whose every product and sum rounds to fp16 as the reference's
kernel does, atol 2e-3 / rtol 1e-2 (the decode path's tolerance); against float64 arithmetic on
the same fp16 inputs, one fp16 rounding (rtol 1e-3), since the HIP kernels form the products in
fp32 and round once."""
import math

import numpy as np
import pytest
import torch

import synth
from chunk_attn import capi
from gpu_helpers import ATOL, RTOL, assert_close, dev, host_state, load_workload, make_attention, to_dev
from oracle.rotary import cos_sin_cache, rotary_embedding

pytestmark = pytest.mark.gpu


def exact_rotation(pos, rows, head_size, cache, is_neox):
    """float64 pairwise rotation of fp16 rows with the fp16 cache values."""
    out, _ = rotary_embedding(pos, rows.astype(np.float64), None, head_size, cache.astype(np.float64), is_neox,
                              step_dtype=np.float64)
    return out


@pytest.mark.parametrize("is_neox", [True, False])
@pytest.mark.parametrize("head_size,rot_dim,n_heads,n_kv", [(128, 128, 32, 32), (64, 32, 5, 1), (16, 16, 2, 2), (6, 2, 3, 2), (64, 24, 3, 3), (20, 12, 2, 1)])
def test_rotary_embedding(is_neox, head_size, rot_dim, n_heads, n_kv):
    rng = np.random.default_rng(11)
    n, max_pos = 37, 500
    cache = cos_sin_cache(rot_dim, max_pos)
    pos = rng.integers(0, max_pos, n)
    q = rng.standard_normal((n, n_heads * head_size)).astype(np.float16)
    k = rng.standard_normal((n, n_kv * head_size)).astype(np.float16)
    tq, tk, tc, tp = to_dev(q), to_dev(k), to_dev(cache), to_dev(pos.astype(np.int64))
    capi.rotary_embedding(tp, tq, tk, head_size, tc, is_neox)
    wq, wk = rotary_embedding(pos, q, k, head_size, cache, is_neox)
    assert_close(tq, wq.astype(np.float64))
    assert_close(tk, wk.astype(np.float64))
    np.testing.assert_allclose(tq.float().cpu().numpy(), exact_rotation(pos, q, head_size, cache, is_neox),
                               rtol=1e-3, atol=1e-6)
    np.testing.assert_allclose(tk.float().cpu().numpy(), exact_rotation(pos, k, head_size, cache, is_neox),
                               rtol=1e-3, atol=1e-6)


def test_rotary_embedding_strided_rows_and_errors():
    rng = np.random.default_rng(12)
    n, H, d = 5, 4, 128
    cache = cos_sin_cache(d, 64)
    qkv = rng.standard_normal((n, 3 * H * d)).astype(np.float16)   # fused projection output
    t = to_dev(qkv)
    tq, tk = t[:, :H * d], t[:, H * d:2 * H * d]
    pos = np.arange(n, dtype=np.int64) + 7
    capi.rotary_embedding(to_dev(pos), tq, tk, d, to_dev(cache), True)
    got = t.cpu().numpy()
    wq, wk = rotary_embedding(pos, qkv[:, :H * d], qkv[:, H * d:2 * H * d], d, cache, True)
    assert_close(torch.from_numpy(got[:, :H * d]), wq.astype(np.float64))
    assert_close(torch.from_numpy(got[:, H * d:2 * H * d]), wk.astype(np.float64))
    assert np.array_equal(got[:, 2 * H * d:], qkv[:, 2 * H * d:])   # the value third is untouched
    with pytest.raises(RuntimeError):
        capi.rotary_embedding(to_dev(pos[:3]), tq, tk, d, to_dev(cache), True)
    lib = capi.load()
    assert lib.ca_rotary_embedding(0, 0, 0, 0, 4, 2, 2, 128, 127, 64, 256, 256, 1, 0) == -1   # odd rot_dim
    assert b"rot_dim" in lib.ca_last_error()


def assert_one_ulp(a, b):
    """The two kernels do the same fp32 arithmetic, but the compiler is free to round the
    result to fp16 in one step (fused multiply-add with fp16 result) or in two: at most one
    fp16 unit in the last place apart."""
    a = a.float().cpu().numpy() if isinstance(a, torch.Tensor) else a.astype(np.float32)
    b = b.float().cpu().numpy() if isinstance(b, torch.Tensor) else b.astype(np.float32)
    assert (np.abs(a - b) <= 2.0 ** -10 * np.maximum(np.abs(a), np.abs(b)) + 2.0 ** -24).all()


def small_cache(H=4, c=32, seed=3):
    w = synth.two_level_workload("rotary-small", groups=2, per_group=3, chunk_size=c, root=2 * c, mid=c,
                                 unique=c // 2 + 3, n_heads=H, append_steps=c + 2)
    attn, order = load_workload(w, seed)
    assert order == list(range(w.n_seqs))
    return w, attn


def seq_lengths(attn):
    n = attn.tree.n_seqs
    return np.array([sum(r[1] for r in attn.get_chunks() if r[2] <= s < r[3]) for s in range(n)])


@pytest.mark.parametrize("is_neox,rot_dim", [(True, 128), (False, 128), (True, 64), (False, 40)])
def test_fused_rotate_and_append(is_neox, rot_dim):
    H, c, d = 4, 32, 128
    rng = np.random.default_rng(13)
    _, fused = small_cache(H, c)
    _, plain = small_cache(H, c)
    n = fused.tree.n_seqs
    cache = cos_sin_cache(rot_dim, 4096)
    tc = to_dev(cache)
    rows0 = fused.get_chunks()
    for step in range(c + 2):          # crosses a chunk boundary: reserve + table rebuild on the way
        lens = seq_lengths(fused)
        q = rng.standard_normal((n, H, d)).astype(np.float16)
        k = rng.standard_normal((n, H, d)).astype(np.float16)
        v = rng.standard_normal((n, H, d)).astype(np.float16)
        toks = [5_000_000 + 100 * step + s for s in range(n)]
        tq, tk = to_dev(q), to_dev(k)
        fused.append_token_rotary(toks, tq, tk, to_dev(v), tc, is_neox)
        assert np.array_equal(tk.cpu().numpy(), k)            # k itself is left as it was
        # the same step as two operators on the twin cache
        pq, pk = to_dev(q), to_dev(k)
        capi.rotary_embedding(to_dev(lens.astype(np.int64)), pq.view(n, H * d), pk.view(n, H * d), d, tc, is_neox)
        plain.append_token(toks, pk, to_dev(v))
        wq, wk = rotary_embedding(lens, q.reshape(n, H * d), k.reshape(n, H * d), d, cache, is_neox)
        assert_close(tq.view(n, H * d), wq.astype(np.float64))
        assert_one_ulp(tq, pq)
        out_f = fused.forward(tq)
        out_p = plain.forward(pq)
        assert_close(out_f, out_p.float().cpu().numpy())
    rf, kf, vf = host_state(fused, as_float=False)
    rp, kp, vp = host_state(plain, as_float=False)
    assert np.array_equal(rf, rp) and len(rf) > len(rows0)
    for slot, n_tok, _, _ in rf:       # every attended row: V identical, rotated K to the last place
        assert_one_ulp(kf[slot][:, :n_tok], kp[slot][:, :n_tok])
        assert np.array_equal(vf[slot][:, :n_tok], vp[slot][:, :n_tok])


def test_fused_explicit_positions_and_errors():
    H, c, d = 4, 32, 128
    rng = np.random.default_rng(14)
    _, a = small_cache(H, c)
    _, b = small_cache(H, c)
    n = a.tree.n_seqs
    cache = to_dev(cos_sin_cache(d, 1024))
    lens = seq_lengths(a)
    q = rng.standard_normal((n, H, d)).astype(np.float16)
    k = rng.standard_normal((n, H, d)).astype(np.float16)
    v = rng.standard_normal((n, H, d)).astype(np.float16)
    qa, qb = to_dev(q), to_dev(q)
    a.append_token_rotary(list(range(n)), qa, to_dev(k), to_dev(v), cache)
    b.append_token_rotary(list(range(n)), qb, to_dev(k), to_dev(v), cache, positions=to_dev(lens.astype(np.int64)))
    assert torch.equal(qa, qb) and torch.equal(a.forward(qa), b.forward(qb))
    short = to_dev(cos_sin_cache(d, 8))      # sequences are longer than this cache
    with pytest.raises(capi.ChunkAttnError, match="longer than the cos/sin cache"):
        a.append_token_rotary(list(range(n)), qa, to_dev(k), to_dev(v), short)
    bad = to_dev(cos_sin_cache(24, 1024))    # NeoX needs whole 8-element pieces per half
    with pytest.raises(capi.ChunkAttnError, match="rot_dim"):
        a.append_token_rotary(list(range(n)), qa, to_dev(k), to_dev(v), bad)


@torch.no_grad()
def test_llama_layer_prefill_then_decode():
    """The reference's attention layer (modeling_llama.py:48-113) with seeded weights: prefill of
    three prompts that share a prefix, then decode steps, against an fp32 recomputation of the
    whole layer over the full history."""
    from chunk_attn.llama_layer import LlamaChunkAttention
    torch.manual_seed(0)
    H, d, c = 4, 128, 32
    hidden = H * d
    layer = LlamaChunkAttention(hidden, H, max_position_embeddings=512)
    for p in (layer.q_proj, layer.k_proj, layer.v_proj, layer.o_proj):
        with torch.no_grad():
            p.weight.copy_((torch.randn(hidden, hidden) / math.sqrt(hidden)).half())
    emb = torch.randn(1000, hidden).half().to(dev())      # token id -> hidden state
    shared = list(range(72))
    seqs = [shared + [100 + 30 * s + i for i in range(25)] for s in range(3)]
    cache = make_attention(H, c, 64)
    T0 = len(seqs[0])

    def reference(history):
        """fp32 layer output for the last token of one sequence over its whole history."""
        x = emb[history].float()
        T = len(history)
        q = (x @ layer.q_proj.weight.float().T).half().float().view(T, H, d)
        k = (x @ layer.k_proj.weight.float().T).half().float().view(T, H, d)
        v = (x @ layer.v_proj.weight.float().T).half().float().view(T, H, d)
        cs = layer.rotary_emb.cos_sin_cache[:T].float()
        cos, sin = cs[:, None, :d // 2], cs[:, None, d // 2:]
        rot = lambda t: torch.cat([t[..., :d // 2] * cos - t[..., d // 2:] * sin,
                                   t[..., d // 2:] * cos + t[..., :d // 2] * sin], dim=-1)
        q, k = rot(q), rot(k)
        s = torch.einsum("hd,thd->ht", q[-1], k) / math.sqrt(d)
        o = torch.einsum("ht,thd->hd", torch.softmax(s, dim=-1), v).reshape(hidden)
        return o @ layer.o_proj.weight.float().T

    hs = torch.stack([emb[s] for s in seqs])                       # [3, 97, hidden]
    pos = torch.arange(T0, device=dev()).repeat(3, 1)
    out = layer(hs, seqs, pos, cache, prefill=True)
    assert layer.last_indices == [0, 1, 2]
    want = torch.stack([reference(s) for s in seqs])
    np.testing.assert_allclose(out[:, -1].float().cpu().numpy(), want.cpu().numpy(), atol=1e-2, rtol=2e-2)
    rows = cache.get_chunks()
    assert sum(1 for r in rows if r[3] - r[2] == 3) == 2           # two full shared chunks of 32

    for step in range(36):                                          # crosses chunk boundaries
        new = [800 + step * 3 + s for s in range(3)]
        seqs = [s + [t] for s, t in zip(seqs, new)]
        hs = emb[new].view(3, 1, hidden)
        pos = torch.tensor([[len(s) - 1] for s in seqs], device=dev())
        out = layer(hs, seqs, pos, cache, prefill=False)
        want = torch.stack([reference(s) for s in seqs])
        np.testing.assert_allclose(out[:, 0].float().cpu().numpy(), want.cpu().numpy(), atol=1e-2, rtol=2e-2)
