"""Native prefix-tree manager (C-ABI ca_tree_*) against the reference's literal expectations
and, on random histories and the five benchmark trees, bit-exact against the oracle."""
import random

import numpy as np
import pytest

import synth
from chunk_attn import capi
from oracle.prefix_tree import PrefixTree
from kats import ADD_SEQ_STEPS, APPEND_CASE, REMOVE_CASE


def tail_slots_by_path(tree: capi.Tree, paths):
    """slot ids of the nodes at the given child-index paths, read from the dump."""
    flat = tree.dump()
    # rebuild child lists
    kids = {0: []}
    stack = [(0, 0)]
    for i, (depth, _, _, _) in enumerate(flat[1:], start=1):
        while stack[-1][0] >= depth:
            stack.pop()
        kids.setdefault(stack[-1][1], []).append(i)
        kids[i] = []
        stack.append((depth, i))
    out = []
    for p in paths:
        n = 0
        for c in p:
            n = kids[n][c]
        out.append(flat[n][3])
    return out


def test_add_seq_kat():
    t = capi.Tree(2, 64)
    want_idx = [0, 1, 2, 3, 3, 3]
    for (tokens, want_tree, want_tails), wi in zip(ADD_SEQ_STEPS, want_idx):
        idx, tok_begin, slots = t.add_seq(tokens)
        assert idx == wi
        assert t.structure() == want_tree
        assert t.tails() == tail_slots_by_path(t, want_tails)
    assert t.n_seqs == 6


def test_append_token_kat():
    t = capi.Tree(2, 64)
    for tokens in APPEND_CASE["adds"]:
        t.add_seq(tokens)
    assert t.append_token(APPEND_CASE["append"]) == 0
    assert t.structure() == APPEND_CASE["tree"]
    assert t.tails() == tail_slots_by_path(t, APPEND_CASE["tails"])


def test_remove_kat():
    t = capi.Tree(2, 64)
    for tokens in REMOVE_CASE["adds"]:
        t.add_seq(tokens)
    used = t.used_chunks
    t.remove_seq(REMOVE_CASE["remove"])
    assert t.structure() == REMOVE_CASE["tree"]
    assert t.used_chunks == used - 1


def test_errors():
    t = capi.Tree(2, 3)
    t.add_seq([1, 2, 3])              # 2 chunks
    with pytest.raises(capi.ChunkAttnError) as e:
        t.add_seq([4, 5, 6, 7])       # needs 3 more
    assert "capacity reached" in str(e.value) and e.value.code == -4
    t2 = capi.Tree(2, 16)
    t2.add_seq([1])
    with pytest.raises(capi.ChunkAttnError) as e:
        t2.append_token([1, 2])
    assert "num of seqs is not equal to num of tokens" in str(e.value)
    with pytest.raises(capi.ChunkAttnError):
        t2.remove_seq(5)


def test_max_chunks_rule():
    # reference chunk_allocator.cpp:32-35
    assert capi.max_chunks_for(1024, 64, 32, 128, 2) == 1024
    assert capi.max_chunks_for(16, 2, 2, 4, 4) == 16 * 1024 * 1024 // (2 * 2 * 4 * 4 * 2)
    assert capi.max_chunks_for(8192, 64, 32, 128, 2) == 8192


def same_state(nat: capi.Tree, ora: PrefixTree):
    assert nat.structure() == ora.structure()
    rows = nat.get_chunks()
    orows = np.array([r.as_tuple() for r in ora.get_chunks()], np.int32).reshape(-1, 4)
    np.testing.assert_array_equal(rows, orows)          # slots included: same allocation policy
    assert nat.tails() == [c.slot for c in ora.tails]
    assert nat.n_seqs == ora.n_seqs


@pytest.mark.parametrize("seed", range(10))
def test_random_histories_match_oracle(seed):
    rng = random.Random(seed)
    c = rng.choice([2, 3, 4, 8])
    nat, ora = capi.Tree(c, 2048), PrefixTree(c, 2048)
    n = 0
    for _ in range(150):
        op = rng.random()
        if op < 0.45 or n == 0:
            toks = [rng.randint(0, 2) for _ in range(rng.randint(1, 3 * c + 2))]
            i1, tb, slots = nat.add_seq(toks)
            i2, jobs = ora.add_seq(toks)
            assert i1 == i2
            assert slots == [j.slot for j in jobs]
            assert tb == (jobs[0].tok_begin if jobs else len(toks))
            n += 1
        elif op < 0.7:
            new = [rng.randint(0, 2) for _ in range(n)]
            assert nat.append_token(new) == len(ora.append_token(new))
        elif op < 0.8:
            assert nat.reserve() == len(ora.reserve())
        else:
            i = rng.randrange(n)
            nat.remove_seq(i)
            ora.remove_seq(i)
            n -= 1
        same_state(nat, ora)
    nat.clear()
    assert nat.n_seqs == 0 and nat.used_chunks == 0


@pytest.mark.parametrize("cfg,frac,want", [
    (0, None, (176, 32, 512)), (1, None, (320, 32, 1024)), (2, 0.25, (3152, 16, 1024)),
    (3, None, (272, 80, 1536)), (4, None, (1344, 64, 16384))])
def test_benchmark_trees(cfg, frac, want):
    w = synth.baseline_config(cfg, frac if frac is not None else 0.5)
    need = sum(w.seq_len(s) // w.chunk_size + 2 for s in range(w.n_seqs))
    nat, ora = capi.Tree(w.chunk_size, need), PrefixTree(w.chunk_size, need)
    for s in range(w.n_seqs):
        toks = w.tokens(s)
        assert nat.add_seq(toks)[0] == ora.add_seq(toks)[0] == s
    rows = nat.get_chunks()
    np.testing.assert_array_equal(rows, np.array([r.as_tuple() for r in ora.get_chunks()], np.int32))
    shared = rows[(rows[:, 3] - rows[:, 2]) > 1]
    assert (len(rows), len(shared), int((shared[:, 3] - shared[:, 2]).sum())) == want
    assert int((rows[:, 1] == 0).sum()) == w.n_seqs      # one empty tail per sequence


@pytest.mark.parametrize("seed", range(8))
def test_random_histories_with_beam_operations_match_oracle(seed):
    """duplicate / append_completion of the native manager against the restatement of reference
    attention.cpp:227-261, 287-313: same tree, same slots, same copy pairs and row targets."""
    rng = random.Random(900 + seed)
    c = rng.choice([2, 3, 4, 8])
    nat, ora = capi.Tree(c, 4096), PrefixTree(c, 4096)
    n = 0
    for _ in range(150):
        op = rng.random()
        if op < 0.3 or n == 0:
            toks = [rng.randint(0, 2) for _ in range(rng.randint(1, 3 * c + 2))]
            i1, _, _ = nat.add_seq(toks)
            i2, _ = ora.add_seq(toks)
            assert i1 == i2
            n += 1
        elif op < 0.5:
            new = [rng.randint(0, 2) for _ in range(n)]
            assert nat.append_token(new) == len(ora.append_token(new))
        elif op < 0.65:
            i, k = rng.randrange(n), rng.randint(0, 3)
            assert nat.duplicate(i, k) == ora.duplicate(i, k)
            n += k
        elif op < 0.85:
            i = rng.randrange(n)
            cand = [rng.randint(0, 2) for _ in range(rng.randint(1, 4))]
            p1, t1 = nat.append_completion(i, cand)
            p2, t2 = ora.append_completion(i, cand)
            assert p1 == p2 and t1 == t2
            n += len(cand) - 1
        else:
            i = rng.randrange(n)
            nat.remove_seq(i)
            ora.remove_seq(i)
            n -= 1
        same_state(nat, ora)


def test_beam_operation_errors():
    t = capi.Tree(2, 3)
    t.add_seq([1, 2, 3])
    rows = t.get_chunks().copy()
    with pytest.raises(capi.ChunkAttnError, match="capacity reached"):
        t.append_completion(0, [4, 5])
    with pytest.raises(capi.ChunkAttnError, match="capacity reached"):
        t.duplicate(0, 2)
    np.testing.assert_array_equal(t.get_chunks(), rows)     # failed calls leave the tree alone
    with pytest.raises(capi.ChunkAttnError):
        t.duplicate(5, 1)
    with pytest.raises(capi.ChunkAttnError):
        t.append_completion(-1, [1])
    assert t.duplicate(0, 0) == [] and t.append_completion(0, []) == ([], [])
