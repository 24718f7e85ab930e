"""The benchmark configurations at full size: outputs against the CPU oracle, and the
size-independent properties (prefix-aware == private copies, all partitions agree)."""
import numpy as np
import pytest
import torch

import synth
from gpu_helpers import (assert_chunk_holds, assert_close, load_workload, oracle_output, oracle_tree_rows,
                         textbook_on_original, to_dev)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cfg", [0, 1, 3])
def test_config_against_oracle(cfg):
    w = synth.baseline_config(cfg)
    attn, order = load_workload(w)
    assert order == list(range(w.n_seqs))
    # independent of what the attention oracle reads back: the tree is the oracle's tree, and
    # chunks hold the rows the workload generated (a shared one, and a private one of the last sequence)
    np.testing.assert_array_equal(attn.get_chunks(), oracle_tree_rows(w))
    assert_chunk_holds(attn, w, 0, 1)
    assert_chunk_holds(attn, w, w.n_seqs - 1, w.seq_len(w.n_seqs - 1) // w.chunk_size - 1)
    q = w.q()
    qd = to_dev(q)
    out0 = attn.forward(qd)
    want = oracle_output(attn, q, partition=0)
    assert_close(out0, want)
    # every partition of the same tree agrees with the oracle too
    assert_close(attn.forward(qd, 2), want)
    assert_close(attn.forward(qd, 1), want)
    # private copies of the same K/V (no sharing) must give the same answer
    paged, _ = load_workload(synth.paged_variant(w))
    outp = paged.forward(qd)
    assert paged.ctx.plan_info().n_shared_chunks == 0
    assert_close(outp, want)
    np.testing.assert_allclose(outp.float().cpu().numpy(), out0.float().cpu().numpy(), atol=2e-3, rtol=1e-2)


SWEEP_SAMPLES = (0, 31, 63)


@pytest.mark.parametrize("fraction", [0.0, 0.25, 0.5, 0.75, 1.0])
def test_config3_sharing_sweep(fraction):
    """Batch 64, 4096 tokens of context, the given fraction of it shared (reference scenario:
    tests/benchmark_chunk_attn.py:73-97; checks as tests/test_chunk_attn_cuda.py:19-72).  4 GiB of
    K/V at fraction 0: drawn on the device; the sampled sequences are checked against float64
    attention over host copies of the very tensors that were inserted."""
    w = synth.baseline_config(2, fraction)
    shared = int(round(4096 * fraction))
    attn, order, kept = load_workload(w, keep=SWEEP_SAMPLES)
    assert order == list(range(64))
    np.testing.assert_array_equal(attn.get_chunks(), oracle_tree_rows(w))
    q = w.q()
    qd = to_dev(q)
    want = {s: textbook_on_original(w, q, s, kv=kept[s]) for s in SWEEP_SAMPLES}
    out0 = attn.forward(qd)
    info = attn.ctx.plan_info()
    assert info.n_shared_chunks == shared // 64 and info.shared_tokens == shared
    assert info.stream_tokens == 64 * (4096 - shared)
    assert (info.n_shared_items > 0) == (shared > 0)
    for s in SWEEP_SAMPLES:
        assert_close(out0[s], want[s])
    assert_chunk_holds(attn, w, 0, 0, kv=kept[0])       # first chunk (shared unless fraction 0)
    assert_chunk_holds(attn, w, 63, 63, kv=kept[63])     # last full chunk of the last sequence
    out2 = attn.forward(qd, 2)
    np.testing.assert_allclose(out2.float().cpu().numpy(), out0.float().cpu().numpy(), atol=2e-3, rtol=1e-2)
    for s in SWEEP_SAMPLES:
        assert_close(out2[s], want[s])
    if fraction == 0.5:
        ref = oracle_output(attn, q, partition=0)       # the reference's CPU path on the same cache
        assert_close(out0, ref)
        assert_close(out2, ref)
    # private copies of the same K/V (no sharing) give the same answer
    paged, _, _ = load_workload(synth.paged_variant(w), keep=())
    outp = paged.forward(qd)
    assert paged.ctx.plan_info().n_shared_chunks == 0
    np.testing.assert_allclose(outp.float().cpu().numpy(), out0.float().cpu().numpy(), atol=2e-3, rtol=1e-2)
    for s in SWEEP_SAMPLES:
        assert_close(outp[s], want[s])


@pytest.mark.parametrize("unique,fused", [(100, False), (128, False), (128, True)])
def test_config4_decode_steps(unique, fused):
    """The two-level tree and its 32 decode steps: as the configuration states it (128 private
    tokens: last chunks hold 0 tokens at the start and never fill), and with 100 private tokens,
    where every last chunk fills and rolls over at step 28.  fused: the steps go through
    decode_step (append and attention in one launch) instead of append_token + forward."""
    w = synth.two_level_workload("cfg4-%d" % unique, 8, 8, 64, 1024, 512, unique, append_steps=32)
    attn, _ = load_workload(w)
    np.testing.assert_array_equal(attn.get_chunks(), oracle_tree_rows(w))
    rng = np.random.default_rng(0)
    for step in range(32):
        k, v = w.append_kv(step)
        q = (rng.standard_normal((w.n_seqs, w.n_heads, 128))).astype(np.float16)
        if fused:
            out = attn.decode_step(w.append_tokens(step), to_dev(q), to_dev(k), to_dev(v))
        else:
            attn.append_token(w.append_tokens(step), to_dev(k), to_dev(v))
        if step in (0, 27, 28, 31):
            if not fused:
                out = attn.forward(to_dev(q))
            assert_close(out, oracle_output(attn, q))
    rows = attn.get_chunks()
    assert rows[:, 1].sum() == 1024 + 8 * 512 + 64 * (unique + 32)


CFG5_SAMPLES = (0, 63, 64, 127, 128, 129, 255)   # both sides of the 128-row boundaries of the wide items


def test_config5_large_batch_properties():
    """256 sequences over a 4096-token prompt (the chunk-first regime: wide items of 128 rows).
    K/V are drawn on the device; the sampled sequences are checked against float64 attention over
    host copies of the tensors that were inserted (never a read-back of the GPU's own pool), the
    tree against the oracle's tree, sampled chunks against the inserted rows."""
    w = synth.baseline_config(4)
    attn, order, kept = load_workload(w, keep=CFG5_SAMPLES)
    assert order == list(range(w.n_seqs))
    np.testing.assert_array_equal(attn.get_chunks(), oracle_tree_rows(w))
    assert_chunk_holds(attn, w, 0, 5, kv=kept[0])                      # a shared chunk
    assert_chunk_holds(attn, w, 255, 4096 // 64 + 2, kv=kept[255])     # a private chunk of the last sequence
    assert_chunk_holds(attn, w, 128, 4096 // 64, kv=kept[128])
    q = w.q()
    out = attn.forward(to_dev(q))
    info = attn.ctx.plan_info()
    out2 = attn.forward(to_dev(q), 2)
    np.testing.assert_allclose(out.float().cpu().numpy(), out2.float().cpu().numpy(), atol=2e-3, rtol=1e-2)
    assert info.n_shared_chunks == 64 and info.shared_tokens == 4096 and info.stream_tokens == 256 * 256
    for s in CFG5_SAMPLES:
        want = textbook_on_original(w, q, s, kv=kept[s])
        assert_close(out[s], want)
        assert_close(out2[s], want)
