"""Decode steps during which last chunks fill up at different steps: the device tables are
patched in place (ca_ctx_roll_tails) instead of rebuilt from a tree walk, through both hosts
(the ctypes binding and the pybind11 class); outputs, reference-form tables and the tree are
compared with the oracle at every step that rolled."""
import numpy as np
import pytest
import torch

import chunk_attn
from chunk_attn import capi
from gpu_helpers import assert_close, dev, host_state, make_attention, to_dev
from oracle.attention_ref import textbook_attention
from oracle.prefix_tree import PrefixTree, build_ref_tables

pytestmark = pytest.mark.gpu


def ragged_batch(rng, c, H, n_seqs, shared):
    sk, sv = (rng.standard_normal((shared, H, 128)).astype(np.float16) for _ in range(2))
    seqs = []
    for s in range(n_seqs):
        extra = (7 * s + 3) % (2 * c) + 1           # last chunks fill at different steps
        toks = list(range(shared)) + [10_000 * (s + 1) + j for j in range(extra)]
        k = np.concatenate([sk, rng.standard_normal((extra, H, 128)).astype(np.float16)])
        v = np.concatenate([sv, rng.standard_normal((extra, H, 128)).astype(np.float16)])
        seqs.append((toks, k, v))
    return seqs


@pytest.mark.parametrize("c,partition", [(32, 0), (64, 0), (32, 2)])
def test_tables_are_patched_not_rebuilt_while_decoding(c, partition):
    rng = np.random.default_rng(70 + c + partition)
    H, B, shared = 4, 9, 3 * c
    attn = make_attention(H, c, B * 8 + 8)
    twin = chunk_attn.Attention(n_heads=H, d_head=128, chunk_size=c, memory_mb=max(1, (B * 8 + 8) * c * H * 512 >> 20) + 1,
                                dtype=torch.float16, device=dev())
    ora = PrefixTree(c, attn.max_chunks)
    for toks, k, v in ragged_batch(rng, c, H, B, shared):
        assert attn.add_seq(toks, to_dev(k), to_dev(v)) == twin.add_seq(toks, to_dev(k), to_dev(v)) == ora.add_seq(toks)[0]
    q0 = to_dev(rng.standard_normal((B, H, 128)).astype(np.float16))
    attn.forward(q0, partition)
    twin.forward(q0, partition)
    full_refreshes = []
    real_refresh = attn.ctx.refresh
    attn.ctx.refresh = lambda *a, **k: (full_refreshes.append(1), real_refresh(*a, **k))[1]
    rolled_steps = 0
    for step in range(2 * c + 5):
        toks = [900_000 + step * 64 + s for s in range(B)]
        k = rng.standard_normal((B, H, 128)).astype(np.float16)
        v = rng.standard_normal((B, H, 128)).astype(np.float16)
        n_new = attn.append_token(toks, to_dev(k), to_dev(v))
        assert n_new == len(twin.append_token(toks, to_dev(k), to_dev(v))) == len(ora.append_token(toks))
        rolled_steps += n_new > 0
        if n_new == 0 and step % 9:
            continue
        assert attn.ctx.valid and attn.ctx.delta_tokens >= 1
        qn = rng.standard_normal((B, H, 128)).astype(np.float16)
        rows, kpool, vpool = host_state(attn)
        np.testing.assert_array_equal(rows, np.array([r.as_tuple() for r in ora.get_chunks()], np.int32))
        out = attn.forward(to_dev(qn), partition)
        assert_close(out, textbook_attention(qn.astype(np.float32), rows.tolist(), kpool, vpool))
        assert torch.equal(out, twin.forward(to_dev(qn), partition))
        if n_new:
            # reference-form tables of the patched context = tables of the tree as it was when the
            # new chunks were added (this step's token is in delta_tokens, not in the tables)
            before = rows.copy()
            tails = {}
            for i, r in enumerate(before.tolist()):
                if r[3] - r[2] == 1:
                    tails[r[2]] = i
            for i in tails.values():
                before[i, 1] -= 1
            got = attn.ctx.ref_tables()
            want = build_ref_tables(before.tolist(), B, c, 1)
            for key in ("final_idx", "slots", "begins", "ends", "offsets", "seq_n_tokens"):
                np.testing.assert_array_equal(got[key], getattr(want, key), err_msg=key)
            assert attn.ctx.delta_tokens == 1
    assert rolled_steps >= 4 and not full_refreshes
    # a forward for another partition rebuilds from the patched context's own rows
    other = 2 - partition
    qn = rng.standard_normal((B, H, 128)).astype(np.float16)
    rows, kpool, vpool = host_state(attn)
    assert_close(attn.forward(to_dev(qn), other), textbook_attention(qn.astype(np.float32), rows.tolist(), kpool, vpool))


def test_roll_tails_errors_leave_the_tables_usable():
    rng = np.random.default_rng(3)
    c, H = 32, 2
    attn = make_attention(H, c, 16)
    k, v = (rng.standard_normal((c + 5, H, 128)).astype(np.float16) for _ in range(2))
    attn.add_seq(list(range(c + 5)), to_dev(k), to_dev(v))
    qn = rng.standard_normal((1, H, 128)).astype(np.float16)
    want = attn.forward(to_dev(qn)).clone()
    assert attn.ctx.roll_tails([0], [7]) is False          # last chunk not full: not patchable, nothing changed
    assert attn.ctx.valid
    assert torch.equal(attn.forward(to_dev(qn)), want)
    with pytest.raises(capi.ChunkAttnError):
        attn.ctx.roll_tails([0], [10 ** 6])                # slot outside the pool
    assert torch.equal(attn.forward(to_dev(qn)), want)
