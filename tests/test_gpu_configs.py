"""The benchmark configurations at full size: outputs against the CPU oracle, and the
size-independent properties (prefix-aware == private copies, all partitions agree)."""
import numpy as np
import pytest
import torch

from chunk_attn import synth
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


def test_config4_decode_steps():
    # two-level tree, 36-token private tails so that appends cross a chunk boundary
    w = synth.two_level_workload("cfg4-100", 8, 8, 64, 1024, 512, 100, append_steps=32)
    attn, _ = load_workload(w)
    rng = np.random.default_rng(0)
    for step in range(32):
        k, v = w.append_kv(step)
        attn.append_token(w.append_tokens(step), to_dev(k), to_dev(v))
        if step in (0, 27, 28, 31):
            q = (rng.standard_normal((w.n_seqs, w.n_heads, 128))).astype(np.float16)
            assert_close(attn.forward(to_dev(q)), oracle_output(attn, q))


def test_config5_large_batch_properties():
    # 256 sequences: checked on a sample of sequences against float64 textbook attention
    w = synth.baseline_config(4)
    attn, _ = load_workload(w)
    q = w.q()
    out = attn.forward(to_dev(q))
    out2 = attn.forward(to_dev(q), 2)
    np.testing.assert_allclose(out.float().cpu().numpy(), out2.float().cpu().numpy(), atol=2e-3, rtol=1e-2)
    from gpu_helpers import host_state
    from oracle.attention_ref import gather_seq_kv
    rows, kpool, vpool = host_state(attn, as_float=False)
    for s in (0, 63, 64, 129, 255):
        k, v = gather_seq_kv(rows.tolist(), s, kpool, vpool)
        sc = np.einsum("hd,htd->ht", q[s].astype(np.float64), k.astype(np.float64)) / np.sqrt(128)
        p = np.exp(sc - sc.max(axis=1, keepdims=True))
        want = np.einsum("ht,htd->hd", p / p.sum(axis=1, keepdims=True), v.astype(np.float64))
        assert_close(out[s], want)
