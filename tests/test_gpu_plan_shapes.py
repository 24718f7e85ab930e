"""The decode kernels under every work-item shape the plan can hand them: the plan's knobs
(chunks per shared segment, chunks per stream item), the partition and the launch schedule are
swept over one cache per chunk size whose tree has narrow and wide shared runs, a second sharing
level, long private runs and ragged tails.  Every combination must reproduce textbook attention
(the oracle's float64 statement) within the decode path's tolerance."""
import itertools

import numpy as np
import pytest
import torch

from gpu_helpers import assert_close, host_state, make_attention, to_dev
from oracle.attention_ref import textbook_attention

pytestmark = pytest.mark.gpu


def build(c, rng, H=2):
    attn = make_attention(H, c, 700)
    root = list(range(3 * c))                                         # shared by everyone
    rk, rv = rng.standard_normal((len(root), H, 128)).astype(np.float16), rng.standard_normal((len(root), H, 128)).astype(np.float16)
    n = 0
    for g, n_in_group in enumerate((100, 9, 1, 68)):                   # a wide group, a narrow one, a loner, a mid-sized one
        mid = [10 ** 4 * (g + 1) + i for i in range(2 * c)]
        mk, mv = rng.standard_normal((len(mid), H, 128)).astype(np.float16), rng.standard_normal((len(mid), H, 128)).astype(np.float16)
        for s in range(n_in_group):
            own = (s * 7) % (c + 5) + (70 * c if (g, s) == (1, 0) else 1)   # one sequence with 70 private chunks
            toks = root + mid + [10 ** 6 * (n + 1) + i for i in range(own)]
            k = np.concatenate([rk, mk, rng.standard_normal((own, H, 128)).astype(np.float16)])
            v = np.concatenate([rv, mv, rng.standard_normal((own, H, 128)).astype(np.float16)])
            assert attn.add_seq(toks, to_dev(k), to_dev(v)) == n
            n += 1
    return attn, n, H


@pytest.mark.parametrize("c", [32, 64, 128])
def test_plan_shapes(c):
    rng = np.random.default_rng(40 + c)
    attn, n, H = build(c, rng)
    q = rng.standard_normal((n, H, 128)).astype(np.float16)
    rows, kpool, vpool = host_state(attn)
    want = textbook_attention(q.astype(np.float32), rows.tolist(), kpool, vpool)
    tq = to_dev(q)
    worst = 0.0
    for seg, stream in itertools.product((0, 1, 2, 3, 7, 64), (0, 1, 2, 5, 63, 64)):
        attn.ctx.set_plan(seg, stream)
        for partition, schedule in ((0, 0), (0, 1), (1, 0), (2, 0), (2, 1)):
            attn.ctx.set_schedule(schedule)
            attn.refresh_kernel_context()
            info = attn.ctx.plan_info()
            assert info.n_stream_items + info.n_shared_items > 0
            out = attn.forward(tq, partition)
            worst = max(worst, assert_close(out, want))
    attn.ctx.set_schedule(0)
    attn.ctx.set_plan(0, 0)
    # and after a few decode steps on the same cache (tables kept valid by delta_tokens)
    for step in range(3):
        k = rng.standard_normal((n, H, 128)).astype(np.float16)
        v = rng.standard_normal((n, H, 128)).astype(np.float16)
        attn.append_token([5 * 10 ** 8 + step * 1000 + s for s in range(n)], to_dev(k), to_dev(v))
    rows, kpool, vpool = host_state(attn)
    want = textbook_attention(q.astype(np.float32), rows.tolist(), kpool, vpool)
    for seg, stream in ((1, 1), (64, 64), (3, 5)):
        attn.ctx.set_plan(seg, stream)
        for partition in (0, 1, 2):
            assert_close(attn.forward(tq, partition), want)
    assert worst < 2e-3


@pytest.mark.parametrize("H", [1, 5, 12, 40])
def test_head_counts_that_are_no_multiple_of_eight(H):
    """Chunk-first workgroups are mapped to (work item, head) so that the row tiles of one (segment,
    head) land on one XCD (workgroup b runs on XCD b % 8): the mapping must cover every (item, head)
    exactly once for any number of heads and items, which shows as every output row being right."""
    c = 64
    rng = np.random.default_rng(400 + H)
    attn, n, _ = build(c, rng, H)
    q = rng.standard_normal((n, H, 128)).astype(np.float16)
    rows, kpool, vpool = host_state(attn)
    want = textbook_attention(q.astype(np.float32), rows.tolist(), kpool, vpool)
    tq = to_dev(q)
    for seg in (0, 1, 3):
        attn.ctx.set_plan(seg, 0)
        for partition in (0, 1):
            out = attn.forward(tq, partition)
            assert attn.ctx.plan_info().n_shared_items > 0
            assert_close(out, want)
