"""The entry point that allocates nothing (ca_attention_noalloc: partial rows in the library's
static device scratch) against ca_attention, through the C-ABI: same kernels, so the outputs must
be identical, and within the decode path's tolerance of the CPU oracle.  Two calls in a row on
one GPU, the second over a smaller cache: the scratch keeps the first call's rows."""
import numpy as np
import pytest
import torch

import synth
from chunk_attn import capi
from gpu_helpers import assert_close, load_workload, oracle_output, to_dev

pytestmark = pytest.mark.gpu


def _both(attn, w):
    q = w.q()
    qd = to_dev(q)
    stream = torch.cuda.current_stream().cuda_stream
    want = attn.forward(qd)                     # ca_attention: builds tables, context-owned buffer
    got = torch.full_like(want, float("nan"))
    attn.ctx.attention_noalloc(qd.data_ptr(), got.data_ptr(), w.n_seqs, stream)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got.cpu().numpy().view(np.uint16), want.cpu().numpy().view(np.uint16))
    assert_close(got, oracle_output(attn, q))
    return attn.ctx.plan_info()


def test_noalloc_matches_attention_twice_second_call_smaller():
    big = synth.two_level_workload("noalloc-big", 4, 6, 64, 512, 256, 200, n_heads=8)
    small = synth.prefix_workload("noalloc-small", 5, 64, 192, 70, n_heads=8)
    a_big, _ = load_workload(big)
    a_small, _ = load_workload(small)
    info_big = _both(a_big, big)
    info_small = _both(a_small, small)
    assert info_big.n_part_rows > info_small.n_part_rows > 0
    # and again the other way round: the big call after the small one
    _both(a_big, big)


def test_noalloc_rejects_what_it_cannot_run():
    w = synth.prefix_workload("noalloc-reject", 3, 64, 128, 40, n_heads=4)
    attn, _ = load_workload(w)
    qd = to_dev(w.q())
    out = torch.empty_like(qd)
    stream = torch.cuda.current_stream().cuda_stream
    with pytest.raises(capi.ChunkAttnError) as e:       # tables not valid yet: it never builds them
        attn.ctx.attention_noalloc(qd.data_ptr(), out.data_ptr(), w.n_seqs, stream)
    assert e.value.code == -3
    attn.forward(qd, 2)                                  # tables now those of partition 2
    with pytest.raises(capi.ChunkAttnError) as e:
        attn.ctx.attention_noalloc(qd.data_ptr(), out.data_ptr(), w.n_seqs, stream)
    assert e.value.code == -3 and "partition" in str(e.value)
    attn.forward(qd)
    attn.ctx.attention_noalloc(qd.data_ptr(), out.data_ptr(), w.n_seqs, stream)
    # more partial rows than the static scratch holds: one shared chunk per segment, many sequences
    many = synth.prefix_workload("noalloc-many", 200, 32, 32 * 12, 8, n_heads=32)
    a_many, _ = load_workload(many)
    a_many.ctx.set_plan(1, 0)
    qm = to_dev(many.q())
    om = a_many.forward(qm)
    rows = a_many.ctx.plan_info().n_part_rows
    assert rows * 32 * 640 > (32 << 20)
    with pytest.raises(capi.ChunkAttnError) as e:
        a_many.ctx.attention_noalloc(qm.data_ptr(), om.data_ptr(), many.n_seqs, stream)
    assert e.value.code == -1 and "scratch" in str(e.value)


def test_noalloc_under_graph_capture_replays_the_eager_result():
    """What the entry point is for: captured into a HIP graph (where an allocation would fail the
    capture) and replayed several times, with eager forwards of another cache -- which overwrite
    the shared scratch -- and synchronisations in between; every replay must equal the eager result.
    A captured forward is bound to the sequence lengths it was captured with: after an append the
    replay still gives the old result and the caller captures again."""
    w = synth.two_level_workload("noalloc-graph", 3, 5, 64, 256, 128, 90, n_heads=8)
    other = synth.prefix_workload("noalloc-graph-other", 7, 64, 320, 33, n_heads=8)
    attn, _ = load_workload(w)
    a_other, _ = load_workload(other)
    q = w.q()
    qd = to_dev(q)
    q_other = to_dev(other.q())
    want = attn.forward(qd).clone()
    want_other = a_other.forward(q_other).clone()
    out = torch.full_like(want, float("nan"))
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        attn.ctx.attention_noalloc(qd.data_ptr(), out.data_ptr(), w.n_seqs, side.cuda_stream)   # warm-up
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        attn.ctx.attention_noalloc(qd.data_ptr(), out.data_ptr(), w.n_seqs, torch.cuda.current_stream().cuda_stream)
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(3):
        out.fill_(float("nan"))
        got_other = torch.empty_like(want_other)
        a_other.ctx.attention_noalloc(q_other.data_ptr(), got_other.data_ptr(), other.n_seqs, stream)
        torch.cuda.synchronize()
        assert torch.equal(got_other, want_other)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
    assert_close(out, oracle_output(attn, q))
    # an append moves delta_tokens: the captured launches still carry the old value
    k, v = w.append_kv(0)
    attn.append_token(w.append_tokens(0), to_dev(k), to_dev(v))
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    fresh = torch.empty_like(out)
    attn.ctx.attention_noalloc(qd.data_ptr(), fresh.data_ptr(), w.n_seqs, stream)
    assert not torch.equal(fresh, want)
    assert_close(fresh, oracle_output(attn, q))
