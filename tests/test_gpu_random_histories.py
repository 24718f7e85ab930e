"""Random add / append / remove histories on the GPU cache: after every few operations the
native tree, the reference-form device tables and the attention outputs are compared with the
oracle driven by the same operations."""
import random

import numpy as np
import pytest
import torch

from chunk_attn import capi
from gpu_helpers import assert_close, host_state, make_attention, to_dev
from oracle.attention_ref import textbook_attention
from oracle.prefix_tree import PrefixTree, build_ref_tables

pytestmark = pytest.mark.gpu


def check_tables(attn, ora, c, tpp):
    rows = attn.get_chunks()
    orows = np.array([r.as_tuple() for r in ora.get_chunks()], np.int32).reshape(-1, 4)
    np.testing.assert_array_equal(rows, orows)
    attn.refresh_kernel_context(force=True)   # tables of the tree as it is now (delta_tokens back to 0)
    got = attn.ctx.ref_tables()
    want = build_ref_tables(orows.tolist(), ora.n_seqs, c, tpp)
    assert got["n_shared"] == want.n_shared and got["partial_rows"] == want.partial_rows
    for key in ("final_idx", "slots", "begins", "ends", "offsets", "seq_n_tokens"):
        np.testing.assert_array_equal(got[key], getattr(want, key))
    np.testing.assert_array_equal(got["seq_chunk_map"], np.array(want.seq_chunk_map, np.int32).reshape(got["seq_chunk_map"].shape))


@pytest.mark.parametrize("seed,c,tpp", [(0, 32, 1), (1, 32, 1), (2, 64, 1), (3, 64, 2), (4, 128, 1), (5, 32, 0)])
def test_history(seed, c, tpp):
    rng = random.Random(seed)
    nrng = np.random.default_rng(seed)
    H = 2
    attn = make_attention(H, c, 600, tpp_threshold=tpp)
    ora = PrefixTree(c, attn.max_chunks)
    # a few prompt families so that sequences share prefixes of different depths
    families = [[rng.randint(0, 50) for _ in range(rng.randint(c, 5 * c))] for _ in range(3)]
    fam_kv = [(nrng.standard_normal((len(f), H, 128)).astype(np.float16), nrng.standard_normal((len(f), H, 128)).astype(np.float16)) for f in families]
    n = 0
    for op_i in range(60):
        r = rng.random()
        if r < 0.45 or n == 0:
            fi = rng.randrange(3)
            cut = rng.randint(1, len(families[fi]))
            extra = rng.randint(0, 2 * c)
            toks = families[fi][:cut] + [1000 + rng.randint(0, 10 ** 6) for _ in range(extra)]
            k = np.concatenate([fam_kv[fi][0][:cut], nrng.standard_normal((extra, H, 128)).astype(np.float16)])
            v = np.concatenate([fam_kv[fi][1][:cut], nrng.standard_normal((extra, H, 128)).astype(np.float16)])
            idx = attn.add_seq(toks, to_dev(k), to_dev(v))
            oidx, _ = ora.add_seq(toks)
            assert idx == oidx
            n += 1
        elif r < 0.8:
            toks = [2000000 + rng.randint(0, 10 ** 6) for _ in range(n)]
            k = nrng.standard_normal((n, H, 128)).astype(np.float16)
            v = nrng.standard_normal((n, H, 128)).astype(np.float16)
            assert attn.append_token(toks, to_dev(k), to_dev(v)) == len(ora.append_token(toks))
        else:
            i = rng.randrange(n)
            attn.remove_seq(i)
            ora.remove_seq(i)
            n -= 1
        if op_i % 6 == 5 and n > 0:
            check_tables(attn, ora, c, tpp)
            q = nrng.standard_normal((n, H, 128)).astype(np.float16)
            rows, kpool, vpool = host_state(attn)
            want = textbook_attention(q.astype(np.float32), rows.tolist(), kpool, vpool)
            for partition in (0, 2):
                assert_close(attn.forward(to_dev(q), partition), want)
    attn.clear()
    assert attn.tree.n_seqs == 0 and attn.tree.used_chunks == 0
