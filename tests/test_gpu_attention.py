"""GPU parity: the HIP decode path, called through the C-ABI, against the CPU oracle on the
same seeded inputs.  Tolerance atol 2e-3 / rtol 1e-2 (fp16 output, fp32 accumulation)."""
import math

import numpy as np
import pytest
import torch

import synth
from chunk_attn import capi
from gpu_helpers import (ATOL, RTOL, assert_close, dev, host_state, load_workload, make_attention,
                         oracle_output, to_dev)
from oracle.attention_ref import textbook_attention, textbook_partials

pytestmark = pytest.mark.gpu


def rand16(rng, *shape, sigma=1.0):
    return (rng.standard_normal(shape) * sigma).astype(np.float16)


@pytest.mark.parametrize("c", [32, 64, 128])
def test_two_sequences_shared_prefix(c):
    # the reference's test_forward scenario (tests/test_chunk_attn_cpu.py:234-265) at d_head 128
    rng = np.random.default_rng(0)
    H = 2
    T1, T2, P = 2 * c + 5, 2 * c + 9, 2 * c
    k1, v1 = rand16(rng, T1, H, 128), rand16(rng, T1, H, 128)
    k2, v2 = rand16(rng, T2, H, 128), rand16(rng, T2, H, 128)
    k2[:P], v2[:P] = k1[:P], v1[:P]
    attn = make_attention(H, c, 16)
    assert attn.add_seq(list(range(T1)), to_dev(k1), to_dev(v1)) == 0
    assert attn.add_seq(list(range(P)) + [900 + i for i in range(T2 - P)], to_dev(k2), to_dev(v2)) == 1
    q = rand16(rng, 2, H, 128)
    for partition in (0, 1, 2):
        out = attn.forward(to_dev(q), partition)
        want = np.zeros((2, H, 128))
        for i, (k, v) in enumerate(((k1, v1), (k2, v2))):
            for h in range(H):
                s = k[:, h].astype(np.float64) @ q[i, h].astype(np.float64) / math.sqrt(128)
                p = np.exp(s - s.max())
                want[i, h] = (p / p.sum()) @ v[:, h].astype(np.float64)
        assert_close(out, want)


@pytest.mark.parametrize("c", [32, 64, 128])
def test_check_result_with_textbook(c):
    # reference tests/test_chunk_attn_cuda.py:19-72: 32 requests x 2000 tokens, 1000 shared
    rng = np.random.default_rng(1)
    H, B, T, P = 2, 32, 2000, 1000
    sk, sv = rand16(rng, P, H, 128), rand16(rng, P, H, 128)
    attn = make_attention(H, c, B * (T // c + 2))
    for s in range(B):
        k, v = rand16(rng, T, H, 128), rand16(rng, T, H, 128)
        k[:P], v[:P] = sk, sv
        toks = list(range(P)) + [100_000 * (s + 1) + i for i in range(T - P)]
        assert attn.add_seq(toks, to_dev(k), to_dev(v)) == s
    q = rand16(rng, B, H, 128)
    want = oracle_output(attn, q, exact=True)
    for partition in (0, 1, 2):
        assert_close(attn.forward(to_dev(q), partition), want)
    info = attn.ctx.plan_info()
    assert info.n_seqs == B


def test_partials_match_reference_layout():
    # reference cpp/tests/test_gpu_kernel.cpp:8-64: 15 sequences sharing every chunk, 16 heads
    rng = np.random.default_rng(2)
    H, c, n, n_chunks = 16, 64, 15, 24
    attn = make_attention(H, c, n_chunks + n + 4)
    attn.ctx.set_plan(shared_seg_chunks=1)
    T = n_chunks * c
    k, v = rand16(rng, T, H, 128), rand16(rng, T, H, 128)
    for s in range(n):
        attn.add_seq(list(range(T)), to_dev(k), to_dev(v))
    q = rand16(rng, n, H, 128)
    attn.refresh_kernel_context()
    qd = to_dev(q)
    attn.ctx.attn_chunks_first(qd.data_ptr(), n)
    maxs, sums, attns = attn.ctx.export_partials()
    rows, kpool, vpool = host_state(attn)
    ref = attn.ctx.ref_tables()
    shared = [r for r in rows.tolist() if r[3] - r[2] > 1]
    assert len(shared) == n_chunks == ref["n_shared"]
    for i, (slot, nt, b, e) in enumerate(shared):
        m, l, o = textbook_partials(q.astype(np.float32), slot, nt, b, e, kpool, vpool)
        off, nn = int(ref["offsets"][i]), e - b
        sl = slice(off * H, off * H + H * nn)
        np.testing.assert_allclose(maxs[sl].reshape(H, nn), m, atol=1e-3, rtol=1e-3)
        np.testing.assert_allclose(sums[sl].reshape(H, nn), l, atol=1e-3, rtol=2e-3)
        np.testing.assert_allclose(attns[sl].reshape(H, nn, 128), o, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("n_shared_seqs", [1, 3, 16, 17, 40, 64, 65, 95, 96, 100, 128, 129, 200])
def test_any_number_of_sharing_sequences(n_shared_seqs):
    # M tiling: row counts that are not multiples of 16 and beyond one 64-row tile
    w = synth.prefix_workload("m-tiles", n_shared_seqs, 64, 192, 70, n_heads=4)
    attn, order = load_workload(w)
    assert order == list(range(w.n_seqs))
    q = w.q()
    assert_close(attn.forward(to_dev(q)), oracle_output(attn, q))


@pytest.mark.parametrize("n_seqs,c,schedule", [(64, 64, 0), (70, 64, 0), (95, 64, 0), (64, 64, 1), (70, 64, 1),
                                               (95, 64, 1), (64, 32, 0), (80, 32, 1), (64, 128, 0), (80, 128, 1),
                                               (33, 64, 0), (40, 64, 1), (49, 32, 0), (63, 128, 1)])
def test_long_shared_run_under_33_to_95_sequences(n_seqs, c, schedule):
    # a run of 2048 tokens or more shared by 33..95 sequences is attended in the row-split wide
    # form: one workgroup for all rows, 16 rows per wave up to 64 sequences, 32 beyond
    w = synth.prefix_workload("long-run", n_seqs, c, 3136, 70, n_heads=2)
    attn, order = load_workload(w)
    assert order == list(range(w.n_seqs))
    attn.ctx.set_schedule(schedule)
    attn.refresh_kernel_context()
    info = attn.ctx.plan_info()
    rows = attn.get_chunks()
    plan = capi.build_tables(rows, w.n_seqs, c, 1, 0, n_heads=2)["plan"]
    assert len(plan["shared_items"]) == info.n_shared_items
    assert set(plan["shared_items"][:, 7].tolist()) == {1} and plan["shared_items"][:, 1].max() == n_seqs
    q = w.q()
    want = oracle_output(attn, q)
    for _ in range(2):
        assert_close(attn.forward(to_dev(q)), want)
    k, v = w.append_kv(0)
    attn.append_token(w.append_tokens(0), to_dev(k), to_dev(v))
    assert_close(attn.forward(to_dev(q)), oracle_output(attn, q))


def test_two_level_tree_and_remove():
    w = synth.two_level_workload("two-level", 3, 5, 32, 96, 64, 40, n_heads=4)
    attn, order = load_workload(w)
    q = w.q()
    assert_close(attn.forward(to_dev(q)), oracle_output(attn, q))
    # removing sequences re-indexes the rest; outputs must follow
    attn.remove_seq(7)
    attn.remove_seq(0)
    keep = [i for i in range(w.n_seqs) if i not in (0, 7)]
    q2 = q[keep]
    out = attn.forward(to_dev(q2))
    assert_close(out, oracle_output(attn, q2))
    assert_close(out, oracle_output(attn, q2, exact=True))


@pytest.mark.parametrize("tpp", [0, 2, 100])
def test_tpp_threshold(tpp):
    w = synth.two_level_workload("tpp", 2, 3, 64, 128, 64, 30, n_heads=2)
    attn, _ = load_workload(w, tpp_threshold=tpp)
    q = w.q()
    assert_close(attn.forward(to_dev(q)), oracle_output(attn, q))


def test_append_tokens_across_chunk_boundaries():
    c, H = 32, 4
    w = synth.prefix_workload("append", 6, c, 64, 0, n_heads=H)
    # ragged private parts: tails at different fill levels, one exactly full
    lens = [1, 31, 32, 33, 5, 63]
    for s, n in enumerate(lens):
        w.seqs[s].append(synth.Segment(1_000_000 * (s + 1) + np.arange(n), synth.STREAM_K_UNIQUE + s, synth.STREAM_V_UNIQUE + s))
    attn, _ = load_workload(w)
    kv_host = [list(w.kv(s)) for s in range(w.n_seqs)]
    rng = np.random.default_rng(3)
    for step in range(70):
        k, v = w.append_kv(step)
        attn.append_token(w.append_tokens(step), to_dev(k), to_dev(v))
        for s in range(w.n_seqs):
            kv_host[s][0] = np.concatenate([kv_host[s][0], k[s:s + 1]])
            kv_host[s][1] = np.concatenate([kv_host[s][1], v[s:s + 1]])
        if step % 9 == 0 or step in (30, 31, 32, 33, 69):
            q = rand16(rng, w.n_seqs, H, 128)
            out = attn.forward(to_dev(q))
            want = np.zeros((w.n_seqs, H, 128))
            for s in range(w.n_seqs):
                kk, vv = kv_host[s]
                for h in range(H):
                    sc = kk[:, h].astype(np.float64) @ q[s, h].astype(np.float64) / math.sqrt(128)
                    p = np.exp(sc - sc.max())
                    want[s, h] = (p / p.sum()) @ vv[:, h].astype(np.float64)
            assert_close(out, want)
    # the pool holds exactly the appended rows
    rows, kpool, vpool = host_state(attn)
    for s in range(w.n_seqs):
        mine = [r for r in rows.tolist() if r[2] <= s < r[3]]
        got = np.concatenate([kpool[r[0]][:, :r[1]] for r in mine if r[1]], axis=1)
        np.testing.assert_array_equal(got, np.transpose(kv_host[s][0], (1, 0, 2)).astype(np.float32))


def test_stale_rows_do_not_leak():
    # a freed chunk full of NaN is reused as a partially filled tail
    c, H = 32, 2
    attn = make_attention(H, c, 8)
    bad = np.full((c, H, 128), np.nan, np.float16)
    attn.add_seq(list(range(c)), to_dev(bad), to_dev(bad))
    attn.remove_seq(0)
    rng = np.random.default_rng(4)
    k, v = rand16(rng, 5, H, 128), rand16(rng, 5, H, 128)
    attn.add_seq([7, 8, 9, 10, 11], to_dev(k), to_dev(v))
    q = rand16(rng, 1, H, 128)
    for partition in (0, 1, 2):
        assert_close(attn.forward(to_dev(q), partition), oracle_output(attn, q, exact=True))


def test_errors_through_the_c_abi():
    attn = make_attention(2, 64, 8)
    rng = np.random.default_rng(5)
    k = to_dev(rand16(rng, 3, 2, 128))
    attn.add_seq([1, 2, 3], k, k)
    with pytest.raises(RuntimeError, match="q is not contiguous"):
        attn.forward(to_dev(rand16(rng, 1, 2, 256))[:, :, :128])
    with pytest.raises(capi.ChunkAttnError, match="does not match the tables"):
        attn.forward(to_dev(rand16(rng, 2, 2, 128)))
    with pytest.raises(RuntimeError, match="num of seqs is not equal to num of tokens"):
        attn.append_token([1, 2], k[:2], k[:2])
    with pytest.raises(capi.ChunkAttnError, match="Unsupported partition type"):
        attn.forward(to_dev(rand16(rng, 1, 2, 128)), 3)
    small = make_attention(2, 64, 0)
    with pytest.raises(capi.ChunkAttnError, match="capacity reached"):
        for i in range(100):
            small.add_seq([i] * 64, to_dev(rand16(rng, 64, 2, 128)), to_dev(rand16(rng, 64, 2, 128)))
    odd = capi.Attention(n_heads=2, d_head=128, chunk_size=48, memory_mb=4, dtype=torch.float16, device=dev())
    odd.add_seq([1, 2, 3], k, k)
    with pytest.raises(capi.ChunkAttnError, match="unsupported chunk_size 48"):
        odd.forward(to_dev(rand16(rng, 1, 2, 128)))


@pytest.mark.parametrize("schedule", [0, 1])
@pytest.mark.parametrize("case", ["prefix", "two-level", "wide", "ragged-appends"])
def test_both_launch_schedules(schedule, case):
    # schedule 0: decode launch + merge launch; 1: single launch, the last finisher merges
    if case == "prefix":
        w = synth.prefix_workload("p", 24, 64, 640, 300, n_heads=8)
    elif case == "two-level":
        w = synth.two_level_workload("t", 4, 6, 32, 256, 160, 70, n_heads=8)
    elif case == "wide":
        w = synth.prefix_workload("w", 150, 64, 384, 40, n_heads=4)
    else:
        w = synth.prefix_workload("r", 9, 32, 96, 0, n_heads=4)
        for s, n in enumerate([1, 31, 32, 33, 64, 65, 100, 5, 127]):
            w.seqs[s].append(synth.Segment(1_000_000 * (s + 1) + np.arange(n), synth.STREAM_K_UNIQUE + s, synth.STREAM_V_UNIQUE + s))
    attn, _ = load_workload(w)
    attn.ctx.set_schedule(schedule)
    rng = np.random.default_rng(7)
    for step in range(3):
        q = rand16(rng, w.n_seqs, w.n_heads, 128)
        want = oracle_output(attn, q)
        for partition in (0, 1, 2):
            for _ in range(2):      # twice: completion counters must come back to zero
                assert_close(attn.forward(to_dev(q), partition), want)
        k, v = w.append_kv(step)
        attn.append_token(w.append_tokens(step), to_dev(k), to_dev(v))


def test_forward_under_graph_capture():
    # with valid tables the forward is kernel launches only: capture it once, replay with new q
    w = synth.two_level_workload("g", 3, 4, 64, 256, 128, 90, n_heads=8)
    attn, _ = load_workload(w)
    rng = np.random.default_rng(8)
    q = to_dev(rand16(rng, w.n_seqs, w.n_heads, 128))
    out = torch.empty_like(q)
    attn.refresh_kernel_context()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        attn.ctx.attention(q.data_ptr(), out.data_ptr(), w.n_seqs, 0, side.cuda_stream)   # warm-up
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        attn.ctx.attention(q.data_ptr(), out.data_ptr(), w.n_seqs, 0, torch.cuda.current_stream().cuda_stream)
    for _ in range(4):
        qn = rand16(rng, w.n_seqs, w.n_heads, 128)
        q.copy_(to_dev(qn))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = attn.forward(q)
        assert torch.equal(out, eager)
        assert_close(out, oracle_output(attn, qn))


def test_captured_forward_is_bound_to_its_delta_tokens():
    """delta_tokens travels as a kernel argument, so a captured forward keeps the value it was
    captured with: replayed after an append it attends the cache as it was at capture time (the
    appended token is ignored); the eager forward sees the new token.  Callers that capture
    re-capture after every append_token."""
    w = synth.prefix_workload("gd", 4, 64, 128, 30, n_heads=4)
    attn, _ = load_workload(w)
    rng = np.random.default_rng(9)
    qn = rand16(rng, w.n_seqs, w.n_heads, 128)
    q = to_dev(qn)
    out = torch.empty_like(q)
    before = attn.forward(q).clone()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        attn.ctx.attention(q.data_ptr(), out.data_ptr(), w.n_seqs, 0, side.cuda_stream)   # warm-up
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        attn.ctx.attention(q.data_ptr(), out.data_ptr(), w.n_seqs, 0, torch.cuda.current_stream().cuda_stream)
    k, v = rand16(rng, w.n_seqs, w.n_heads, 128), rand16(rng, w.n_seqs, w.n_heads, 128)
    attn.append_token(w.append_tokens(0), to_dev(3 * k), to_dev(v))
    assert attn.ctx.valid and attn.ctx.delta_tokens == 1      # tables untouched, only delta moved
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, before)
    eager = attn.forward(q)
    assert not torch.equal(eager, before)
    assert_close(eager, oracle_output(attn, qn))


def test_negative_delta_tokens_is_rejected():
    w = synth.prefix_workload("nd", 2, 64, 64, 10, n_heads=2)
    attn, _ = load_workload(w)
    attn.refresh_kernel_context()
    with pytest.raises(capi.ChunkAttnError) as e:
        attn.ctx.delta_tokens = -1
    assert e.value.code == -1 and attn.ctx.delta_tokens == 0
    with pytest.raises(capi.ChunkAttnError):
        attn.ctx.set_timing(7)


def test_marker_ranges_do_not_change_results():
    """roctx ranges around the C-ABI calls are bookkeeping on the host only."""
    w = synth.prefix_workload("mk", 5, 64, 130, 70, n_heads=2)
    attn, _ = load_workload(w)
    q = to_dev(w.q())
    base = attn.forward(q).clone()
    try:
        capi.set_markers(True)
    except capi.ChunkAttnError as e:
        assert "marker library" in str(e)
        return
    try:
        attn.refresh_kernel_context(True)
        k, v = w.append_kv(0)
        assert torch.equal(attn.forward(q), base)
        attn.append_token(w.append_tokens(0), to_dev(k), to_dev(v))
        assert_close(attn.forward(q), oracle_output(attn, w.q()))
    finally:
        capi.set_markers(False)


def test_read_probe_reads_and_checks_its_arguments():
    """The bench's yardstick launch: runs over aligned buffers of any length that holds one
    16-byte unit, leaves the buffer alone, and rejects what it cannot read."""
    w = synth.prefix_workload("rp", 2, 64, 64, 10, n_heads=2)
    attn, _ = load_workload(w)
    buf = torch.arange(1 << 18, dtype=torch.int64, device=dev())
    before = buf.clone()
    st = torch.cuda.current_stream().cuda_stream
    for n_bytes, per_cu in ((16, 1), (4096 + 16, 2), (buf.numel() * 8, 1), (buf.numel() * 8, 4)):
        attn.ctx.bench_read_probe(buf.data_ptr(), n_bytes, per_cu, st)
    torch.cuda.synchronize()
    assert torch.equal(buf, before)
    for ptr, n_bytes, per_cu in ((buf.data_ptr() + 8, 64, 1), (buf.data_ptr(), 8, 1), (0, 64, 1),
                                 (buf.data_ptr(), 64, 0), (buf.data_ptr(), 64, 9)):
        with pytest.raises(capi.ChunkAttnError) as e:
            attn.ctx.bench_read_probe(ptr, n_bytes, per_cu, st)
        assert e.value.code == -1


@pytest.mark.parametrize("c", [32, 64, 128])
def test_repeated_forwards_are_bit_identical(c):
    """The default schedule merges partial rows in a fixed order, so a forward is a pure function
    of the cache and q.  Anything that depends on timing or on what freshly allocated buffers
    held before (a read that races its producer, a register read before a matrix op has
    written it) shows up as a difference between repetitions."""
    rng = np.random.default_rng(40 + c)
    H = 2
    T1, T2, P = 2 * c + 5, 2 * c + 9, 2 * c
    k1, v1 = rand16(rng, T1, H, 128), rand16(rng, T1, H, 128)
    k2, v2 = rand16(rng, T2, H, 128), rand16(rng, T2, H, 128)
    k2[:P], v2[:P] = k1[:P], v1[:P]
    attn = make_attention(H, c, 16)
    attn.add_seq(list(range(T1)), to_dev(k1), to_dev(v1))
    attn.add_seq(list(range(P)) + [900 + i for i in range(T2 - P)], to_dev(k2), to_dev(v2))
    q = rand16(rng, 2, H, 128)
    for partition in (0, 1, 2):
        first = attn.forward(to_dev(q), partition).clone()
        for _ in range(6):
            junk = torch.randn(4096, device=dev())     # moves the allocator's free blocks around
            assert torch.equal(attn.forward(to_dev(q), partition), first)
            del junk


@pytest.mark.parametrize("c", [32, 64])
def test_long_paths_split_into_items_of_at_most_64_chunks(c):
    """Sequences far longer than 64 chunks, with plan sizes asked for beyond what an item may
    hold: the work list is capped and every partition still matches the oracle."""
    rng = np.random.default_rng(50)
    H, B = 2, 3
    P, U = 70 * c, 75 * c + 7          # 70 shared chunks, 76 private chunks per sequence
    sk, sv = rand16(rng, P, H, 128), rand16(rng, P, H, 128)
    attn = make_attention(H, c, 70 + B * 78)
    for s in range(B):
        k, v = rand16(rng, P + U, H, 128), rand16(rng, P + U, H, 128)
        k[:P], v[:P] = sk, sv
        assert attn.add_seq(list(range(P)) + [10_000_000 * (s + 1) + i for i in range(U)], to_dev(k), to_dev(v)) == s
    q = rand16(rng, B, H, 128)
    want = oracle_output(attn, q, exact=True)
    for seg, strm in ((0, 0), (400, 400)):
        attn.ctx.set_plan(seg, strm)
        for partition in (0, 1, 2):
            assert_close(attn.forward(to_dev(q), partition), want)
            tables = capi.build_tables(attn.get_chunks(), B, c, 1, partition, seg, strm, n_heads=H)
            for items in (tables["plan"]["shared_items"], tables["plan"]["stream_items"]):
                assert len(items) == 0 or items[:, 3].max() <= 64


def test_many_short_private_runs_one_item_per_wave():
    """Enough short private runs (sequences x heads) make the plan run stream items one per
    wave.  Ragged runs of one to three chunks, sequences that end exactly on a chunk boundary,
    appends that fill tails and open new chunks: every step must match the oracle, in the
    default schedule (per wave) and in the single-launch schedule (which must not use it)."""
    rng = np.random.default_rng(60)
    H, c, B = 32, 32, 56
    P = 2 * c
    sk, sv = rand16(rng, P, H, 128), rand16(rng, P, H, 128)
    attn = make_attention(H, c, 2 + B * 6)
    for s in range(B):
        U = [5, c, c + 7, 2 * c, 2 * c + 9, 1][s % 6]
        k, v = rand16(rng, P + U, H, 128), rand16(rng, P + U, H, 128)
        k[:P], v[:P] = sk, sv
        assert attn.add_seq(list(range(P)) + [1_000_000 * (s + 1) + i for i in range(U)], to_dev(k), to_dev(v)) == s
    q = rand16(rng, B, H, 128)
    attn.refresh_kernel_context()
    assert attn.ctx.plan_info().stream_per_wave == 1
    for step in range(c + 3):
        if step % 8 == 0 or step > c - 2:
            want = oracle_output(attn, q, exact=True)
            assert_close(attn.forward(to_dev(q)), want)
            assert_close(attn.forward(to_dev(q), 2), want)      # everything streamed
        k1, v1 = rand16(rng, B, H, 128), rand16(rng, B, H, 128)
        attn.append_token([7_000_000 + 64 * step + s for s in range(B)], to_dev(k1), to_dev(v1))
    want = oracle_output(attn, q, exact=True)
    assert_close(attn.forward(to_dev(q)), want)
    attn.ctx.set_schedule(1)
    assert_close(attn.forward(to_dev(q)), want)
    assert attn.ctx.plan_info().stream_per_wave == 0
    attn.ctx.set_schedule(0)
    assert_close(attn.forward(to_dev(q)), want)
    assert attn.ctx.plan_info().stream_per_wave == 1


def test_beam_search_operations_through_the_c_abi():
    """duplicate and append_completion (reference attention.cpp:227-261, 287-313) on the GPU cache:
    every sequence's attention equals textbook attention over its own K/V history."""
    rng = np.random.default_rng(21)
    H, c = 4, 32
    attn = make_attention(H, c, 64)
    hist = []                                   # per sequence: (k rows, v rows) as numpy

    def rows(n):
        return (rng.standard_normal((n, H, 128)).astype(np.float16), rng.standard_normal((n, H, 128)).astype(np.float16))

    k0, v0 = rows(70)                            # two full chunks and a tail of 6
    attn.add_seq(list(range(70)), to_dev(k0), to_dev(v0))
    k1, v1 = rows(31)
    attn.add_seq(list(range(64)) + list(range(1000, 1031)), to_dev(np.concatenate([k0[:64], k1])),
                 to_dev(np.concatenate([v0[:64], v1])))
    hist = [(k0, v0), (np.concatenate([k0[:64], k1]), np.concatenate([v0[:64], v1]))]

    def check():
        n = len(hist)
        q = rng.standard_normal((n, H, 128)).astype(np.float16)
        out = attn.forward(to_dev(q)).float().cpu().numpy()
        for s, (k, v) in enumerate(hist):
            sc = np.einsum("hd,thd->ht", q[s].astype(np.float64), k.astype(np.float64)) / np.sqrt(128.0)
            p = np.exp(sc - sc.max(axis=1, keepdims=True))
            want = np.einsum("ht,thd->hd", p / p.sum(axis=1, keepdims=True), v.astype(np.float64))
            np.testing.assert_allclose(out[s], want, atol=ATOL, rtol=RTOL)

    check()
    attn.duplicate(1, 2)                         # sequences 1, 2, 3 are the same now
    hist[2:2] = [hist[1], hist[1]]
    assert attn.tree.n_seqs == 4
    check()
    # beam step on sequence 2: three candidates; its tail holds 31 of 32 rows, so all three fill up
    nk, nv = rows(3)
    assert attn.append_completion(2, [7, 8, 9], to_dev(nk), to_dev(nv)) == 2
    base = hist[2]
    hist[2:3] = [(np.concatenate([base[0], nk[i:i + 1]]), np.concatenate([base[1], nv[i:i + 1]])) for i in range(3)]
    assert attn.tree.n_seqs == 6
    check()
    # and the decode loop goes on from there
    ak, av = rows(6)
    attn.append_token(list(range(500, 506)), to_dev(ak), to_dev(av))
    hist = [(np.concatenate([k, ak[i:i + 1]]), np.concatenate([v, av[i:i + 1]])) for i, (k, v) in enumerate(hist)]
    check()
    attn.remove_seq(3)
    del hist[3]
    check()


def test_stream_hint_does_not_change_results():
    """ca_ctx_set_stream_hint only picks the load instruction for private chunks."""
    w = synth.two_level_workload("hint", groups=2, per_group=3, chunk_size=64, root=128, mid=64, unique=150, n_heads=4)
    attn, _ = load_workload(w, 5)
    q = to_dev(w.q(5))
    outs = []
    for mode in (0, 1, 2):
        attn.ctx.set_stream_hint(mode)
        outs.append(attn.forward(q))
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    assert_close(outs[0], oracle_output(attn, w.q(5), exact=True))
    with pytest.raises(capi.ChunkAttnError, match="stream hint"):
        attn.ctx.set_stream_hint(3)


def test_timing_modes_leave_results_alone():
    # HIP-event timing inside the library (modes 1, 2): every mode writes the complete output.  The
    # launch-only measurement aids are entry points of their own and leave the context as it was.
    w = synth.prefix_workload("timing", 6, 64, 256, 200, n_heads=4)
    attn, _ = load_workload(w)
    q = to_dev(w.q())
    want = attn.forward(q).clone()
    out = torch.empty_like(q)
    stream = torch.cuda.current_stream().cuda_stream
    for mode in (1, 2):
        attn.ctx.set_timing(mode)
        attn.ctx.read_timing(reset=True)
        for _ in range(3):
            attn.ctx.attention(q.data_ptr(), out.data_ptr(), w.n_seqs, 0, stream)
        t = attn.ctx.read_timing(reset=True)
        assert t["calls"] == 3 and t["shared_ms"] > 0 and t["merge_ms"] > 0
        if mode == 2:
            assert t["stream_ms"] > 0
        assert torch.equal(out, want)
    attn.ctx.set_timing(0)
    scratch_out = torch.empty_like(q)
    for what in (0, 1, 2):   # partial work only: outputs are not complete, nothing is recorded
        attn.ctx.bench_decode_launch(q.data_ptr(), scratch_out.data_ptr(), w.n_seqs, what, stream)
        assert attn.ctx.read_timing(reset=True)["calls"] == 0
    with pytest.raises(capi.ChunkAttnError):
        attn.ctx.bench_decode_launch(q.data_ptr(), scratch_out.data_ptr(), w.n_seqs, 3, stream)
    assert torch.equal(attn.forward(q), want)
    for mode in (3, 4, 5):   # ca_attention has no mode that leaves outputs incomplete
        with pytest.raises(capi.ChunkAttnError):
            attn.ctx.set_timing(mode)
