"""The fused decode step (ca_decode_step / Attention.decode_step): one call that appends the new
token's K/V rows and attends, the attention launch writing the rows itself.  Checked against the
two-call form (append_token, then forward) on a twin cache -- outputs and pools bit for bit, at
every step of ragged decode histories in which last chunks fill up and roll over at different
steps -- and against the oracle within the path's tolerance.  Reference behaviour:
Attention::append_token + Attention::forward (cpp/chunk_attn/attention.cpp:57-114)."""
import numpy as np
import pytest
import torch

import chunk_attn
from chunk_attn import capi
from gpu_helpers import assert_close, dev, host_state, make_attention, to_dev
from oracle.attention_ref import textbook_attention
from oracle.prefix_tree import PrefixTree

pytestmark = pytest.mark.gpu


def ragged_batch(rng, c, H, n_seqs, shared, spread):
    """n_seqs sequences over one shared prompt with private parts of different lengths (so that
    their last chunks fill at different steps); one sequence ends exactly on a chunk boundary."""
    sk, sv = (rng.standard_normal((shared, H, 128)).astype(np.float16) for _ in range(2))
    seqs = []
    for s in range(n_seqs):
        extra = c if s == 1 else (11 * s + 3) % spread + 1
        toks = list(range(shared)) + [10_000 * (s + 1) + j for j in range(extra)]
        k = np.concatenate([sk, rng.standard_normal((extra, H, 128)).astype(np.float16)])
        v = np.concatenate([sv, rng.standard_normal((extra, H, 128)).astype(np.float16)])
        seqs.append((toks, k, v))
    return seqs


def pools_equal(a, b):
    """Every chunk either cache uses holds the same bits (rows past a chunk's tokens included:
    both caches started from zeroed pools here)."""
    rows_a, ka, va = host_state(a, as_float=False)
    rows_b, kb, vb = host_state(b, as_float=False)
    np.testing.assert_array_equal(rows_a, rows_b)
    for slot in sorted(set(rows_a[:, 0].tolist())):
        assert np.array_equal(ka[slot].view(np.uint16), kb[slot].view(np.uint16)), "K of chunk %d" % slot
        assert np.array_equal(va[slot].view(np.uint16), vb[slot].view(np.uint16)), "V of chunk %d" % slot


def zeroed(attn):
    attn.key_storage.zero_()
    attn.value_storage.zero_()
    return attn


# (chunk size, heads, sequences, shared tokens, spread of the private lengths, steps)
CASES = [
    (32, 4, 9, 96, 64, 70),      # two chunks per streamed tile; every tail rolls at least twice
    (64, 4, 9, 192, 128, 70),    # the benchmark's chunk size
    (128, 2, 5, 256, 200, 140),  # two sub-tiles per chunk
    (64, 4, 400, 1024, 40, 30),  # many short private runs: stream items run one per wave, wide chunk-first items
    (64, 2, 20, 0, 100, 70),     # nothing shared: the stream-only form of the kernel
]


@pytest.mark.parametrize("c,H,B,shared,spread,steps", CASES)
def test_fused_step_equals_append_then_forward(c, H, B, shared, spread, steps):
    rng = np.random.default_rng(1000 + c + B)
    n_chunks = B * (spread // c + steps // c + 4) + shared // c + 8
    two_call = zeroed(make_attention(H, c, n_chunks))
    fused = zeroed(make_attention(H, c, n_chunks))
    ora = PrefixTree(c, two_call.max_chunks)
    for toks, k, v in ragged_batch(rng, c, H, B, shared, spread):
        assert two_call.add_seq(toks, to_dev(k), to_dev(v)) == fused.add_seq(toks, to_dev(k), to_dev(v)) == ora.add_seq(toks)[0]
    per_wave_seen = False
    rolled_steps = 0
    for step in range(steps):
        toks = [900_000 + step * 64 + s for s in range(B)]
        k, v, q = (to_dev(rng.standard_normal((B, H, 128)).astype(np.float16)) for _ in range(3))
        n_new = two_call.append_token(toks, k, v)
        want = two_call.forward(q)
        got = fused.decode_step(toks, q, k, v)
        assert len(ora.append_token(toks)) == n_new
        rolled_steps += n_new > 0
        assert torch.equal(got, want), "step %d" % step
        assert fused.ctx.delta_tokens == two_call.ctx.delta_tokens
        per_wave_seen |= bool(fused.ctx.plan_info().stream_per_wave)
        if n_new or step % 16 == 0 or step == steps - 1:
            pools_equal(two_call, fused)
            rows, kpool, vpool = host_state(fused)
            np.testing.assert_array_equal(rows, np.array([r.as_tuple() for r in ora.get_chunks()], np.int32))
            assert_close(got, textbook_attention(q.cpu().numpy().astype(np.float32), rows.tolist(), kpool, vpool))
    assert rolled_steps >= 2
    if B == 400:
        assert per_wave_seen
    # the two forms can be mixed on one cache
    toks = [7_000_000 + s for s in range(B)]
    k, v, q = (to_dev(rng.standard_normal((B, H, 128)).astype(np.float16)) for _ in range(3))
    fused.append_token(toks, k, v)
    got = fused.forward(q)
    assert torch.equal(got, two_call.decode_step(toks, q, k, v))
    pools_equal(two_call, fused)


def test_fused_step_through_the_pybind_class():
    rng = np.random.default_rng(77)
    c, H, B, shared = 64, 4, 6, 128
    mb = max(1, (B * 6 + 8) * c * H * 512 >> 20) + 1
    a, b = (chunk_attn.Attention(n_heads=H, d_head=128, chunk_size=c, memory_mb=mb, dtype=torch.float16, device=dev())
            for _ in range(2))
    for toks, k, v in ragged_batch(rng, c, H, B, shared, 2 * c):
        assert a.add_seq(toks, to_dev(k), to_dev(v)) == b.add_seq(toks, to_dev(k), to_dev(v))
    for step in range(c + 10):
        toks = [900_000 + step * 64 + s for s in range(B)]
        k, v, q = (to_dev(rng.standard_normal((B, H, 128)).astype(np.float16)) for _ in range(3))
        fresh = a.append_token(toks, k, v)
        want = a.forward(q)
        got = b.decode_step(toks, q, k, v)
        assert torch.equal(got, want), "step %d" % step
        assert [t.n_tokens for t in a.tails] == [t.n_tokens for t in b.tails]
        if fresh:
            for ta, tb in zip(a.tails, b.tails):    # rows past a chunk's tokens were never written
                n = ta.n_tokens
                assert torch.equal(a.key(ta)[:, :n], b.key(tb)[:, :n]) and torch.equal(a.value(ta)[:, :n], b.value(tb)[:, :n])
    for (ca_, ba, ea), (cb, bb, eb) in zip(a.get_chunks(), b.get_chunks()):
        assert (ca_.slot, ca_.n_tokens, ba, ea) == (cb.slot, cb.n_tokens, bb, eb)
        n = ca_.n_tokens
        assert torch.equal(a.key(ca_)[:, :n], b.key(cb)[:, :n]) and torch.equal(a.value(ca_)[:, :n], b.value(cb)[:, :n])
    with pytest.raises(RuntimeError):
        b.decode_step([1], q, k, v)   # one token per sequence


def test_fused_step_when_last_chunks_are_attended_chunk_first():
    """tpp_threshold 0 makes every chunk a chunk-first chunk, last chunks included: the step
    falls back to an append launch in front of the forward, with the same results."""
    rng = np.random.default_rng(5)
    c, H, B = 32, 2, 5
    a = zeroed(make_attention(H, c, 64, tpp_threshold=0))
    b = zeroed(make_attention(H, c, 64, tpp_threshold=0))
    for toks, k, v in ragged_batch(rng, c, H, B, c, c):
        a.add_seq(toks, to_dev(k), to_dev(v))
        b.add_seq(toks, to_dev(k), to_dev(v))
    for step in range(c + 3):
        toks = [900_000 + step * 64 + s for s in range(B)]
        k, v, q = (to_dev(rng.standard_normal((B, H, 128)).astype(np.float16)) for _ in range(3))
        a.append_token(toks, k, v)
        want = a.forward(q)
        assert torch.equal(b.decode_step(toks, q, k, v), want)
    pools_equal(a, b)
    rows, kpool, vpool = host_state(b)
    assert_close(want, textbook_attention(q.cpu().numpy().astype(np.float32), rows.tolist(), kpool, vpool))


def test_fused_step_checks_its_arguments():
    rng = np.random.default_rng(6)
    c, H = 32, 2
    attn = make_attention(H, c, 16)
    k, v = (rng.standard_normal((c - 1, H, 128)).astype(np.float16) for _ in range(2))
    attn.add_seq(list(range(c - 1)), to_dev(k), to_dev(v))
    q = to_dev(rng.standard_normal((1, H, 128)).astype(np.float16))
    attn.append_token([c - 1], q, q)                           # the last chunk is full now
    assert attn.ctx.delta_tokens == 1
    out = torch.empty_like(q)
    st = torch.cuda.current_stream().cuda_stream
    with pytest.raises(capi.ChunkAttnError) as e:             # no free row: reserve first
        attn.ctx.decode_step(q.data_ptr(), q.data_ptr(), q.data_ptr(), out.data_ptr(), 1, st)
    assert e.value.code == -3 and attn.ctx.delta_tokens == 1
    with pytest.raises(capi.ChunkAttnError) as e:
        attn.ctx.decode_step(q.data_ptr(), 0, q.data_ptr(), out.data_ptr(), 1, st)
    assert e.value.code == -1
    with pytest.raises(capi.ChunkAttnError) as e:
        attn.ctx.decode_step(q.data_ptr(), q.data_ptr(), q.data_ptr(), out.data_ptr(), 2, st)
    assert e.value.code == -3
    got = attn.decode_step([5], q, q, q)                       # the class reserves by itself
    rows, kpool, vpool = host_state(attn)
    assert rows[:, 1].tolist() == [c, 1]
    assert_close(got, textbook_attention(q.cpu().numpy().astype(np.float32), rows.tolist(), kpool, vpool))
