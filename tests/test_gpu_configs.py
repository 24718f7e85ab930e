"""The benchmark configurations at full size: outputs against the CPU oracle, and the
size-independent properties (prefix-aware == private copies, all partitions agree)."""
import numpy as np
import pytest
import torch

from chunk_attn import synth
from gpu_helpers import assert_close, load_workload, oracle_output, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cfg", [0, 1, 3])
def test_config_against_oracle(cfg):
    w = synth.baseline_config(cfg)
    attn, order = load_workload(w)
    assert order == list(range(w.n_seqs))
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
