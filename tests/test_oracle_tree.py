"""Pins oracle/prefix_tree.py: the reference's own literal expectations, the hand-worked
table example, and an independently built dictionary trie."""
import random

import pytest

from oracle.prefix_tree import PrefixTree, build_ref_tables
from kats import ADD_SEQ_STEPS, APPEND_CASE, REMOVE_CASE, TABLE_KAT


def node_at(tree, path):
    node = tree.root
    for i in path:
        node = node.children[i]
    return node


def test_add_seq_kat():
    t = PrefixTree(chunk_size=2, max_chunks=64)
    expected_idx = [0, 1, 2, 3, 3, 3]
    for (tokens, want_tree, want_tails), want_idx in zip(ADD_SEQ_STEPS, expected_idx):
        idx, _ = t.add_seq(tokens)
        assert idx == want_idx
        assert t.structure() == want_tree
        assert t.tails == [node_at(t, p) for p in want_tails]


def test_append_token_kat():
    t = PrefixTree(2, 64)
    for tokens in APPEND_CASE["adds"]:
        t.add_seq(tokens)
    t.append_token(APPEND_CASE["append"])
    assert t.structure() == APPEND_CASE["tree"]
    assert t.tails == [node_at(t, p) for p in APPEND_CASE["tails"]]


def test_remove_kat():
    t = PrefixTree(2, 64)
    for tokens in REMOVE_CASE["adds"]:
        t.add_seq(tokens)
    t.remove_seq(REMOVE_CASE["remove"])
    assert t.structure() == REMOVE_CASE["tree"]


def test_table_kat():
    t = PrefixTree(2, 64)
    for tokens, _, _ in ADD_SEQ_STEPS:
        t.add_seq(tokens)
    rows = t.get_chunks()
    assert [(tuple(r.chunk.tokens), r.seq_begin, r.seq_end) for r in rows] == TABLE_KAT["rows"]
    tab = build_ref_tables([r.as_tuple() for r in rows], t.n_seqs, 2, 1)
    assert tab.n_shared == TABLE_KAT["n_shared"]
    assert tab.final_idx == TABLE_KAT["final_idx"]
    assert (tab.begins, tab.ends, tab.offsets) == (TABLE_KAT["begins"], TABLE_KAT["ends"], TABLE_KAT["offsets"])
    assert tab.partial_rows == TABLE_KAT["partial_rows"]
    assert tab.seq_n_tokens == TABLE_KAT["seq_n_tokens"]
    assert tab.max_seq_n_chunks == TABLE_KAT["max_seq_n_chunks"]
    assert tab.seq_chunk_map == TABLE_KAT["seq_chunk_map"]
    # slots follow the same renumbering
    for row, fi in zip(rows, tab.final_idx):
        assert tab.slots[fi] == row.chunk.slot


def test_boundary_crossing_append_and_reuse_of_generated_tokens():
    # behaviour observed on the reference: chunk_size 2, two sequences, three appends
    t = PrefixTree(2, 64)
    t.add_seq([1, 2, 3])
    t.add_seq([1, 2, 4, 5])
    new = [len(t.append_token(tok)) for tok in ([100, 200], [101, 201], [102, 202])]
    assert new == [0, 1, 1]
    assert t.structure() == (2, (), [(2, (1, 2), [
        (1, (3, 100), [(1, (101, 102), [])]),
        (1, (4, 5), [(1, (200, 201), [(1, (202,), [])])])])])
    t.remove_seq(1)
    assert t.structure() == (1, (), [(1, (1, 2), [(1, (3, 100), [(1, (101, 102), [])])])])
    idx, jobs = t.add_seq([1, 2, 3, 100])      # matches the former tail, now an internal node
    assert idx == 1 and jobs == []
    assert t.structure() == (2, (), [(2, (1, 2), [(2, (3, 100), [(1, (101, 102), []), (1, (), [])])])])


def test_share_prefix_false_quirk():
    t = PrefixTree(2, 64, share_prefix=False)
    assert [t.add_seq(s)[0] for s in ([1, 2, 3], [4, 5, 6], [7, 8, 9])] == [0, 0, 0]
    assert [tuple(c.tokens) for c in t.root.children] == [(1, 2), (4, 5), (7, 8)]
    assert [tuple(x.tokens) for x in t.tails] == [(9,), (6,), (3,)]


def brute_force_order(seqs, c):
    """Independent model for insert-only histories: a dict trie over full chunks; every
    sequence hangs a private leaf under its last full chunk.  Returns the left-to-right leaf
    order (sequence ids) and per-prefix sharing counts."""
    root = {"kids": [], "index": {}}
    counts = {}
    for sid, toks in enumerate(seqs):
        node = root
        n_full = len(toks) // c
        for k in range(n_full):
            key = tuple(toks[k * c:(k + 1) * c])
            prefix = tuple(toks[:(k + 1) * c])
            counts[prefix] = counts.get(prefix, 0) + 1
            if key not in node["index"]:
                child = {"kids": [], "index": {}}
                node["index"][key] = child
                node["kids"].append(child)
            node = node["index"][key]
        node["kids"].append({"leaf": sid})
    order = []

    def walk(n):
        for k in n["kids"]:
            if "leaf" in k:
                order.append(k["leaf"])
            else:
                walk(k)
    walk(root)
    return order, counts


@pytest.mark.parametrize("seed", range(6))
def test_insert_only_against_brute_force(seed):
    rng = random.Random(seed)
    c = rng.choice([2, 3, 4])
    seqs = []
    for _ in range(rng.randint(3, 24)):
        if seqs and rng.random() < 0.7:
            base = rng.choice(seqs)
            cut = rng.randint(0, len(base))
            toks = base[:cut] + [rng.randint(0, 3) for _ in range(rng.randint(0, 7))]
        else:
            toks = [rng.randint(0, 3) for _ in range(rng.randint(1, 12))]
        if not toks:
            toks = [rng.randint(0, 3)]
        seqs.append(toks)
    t = PrefixTree(c, 4096)
    order = []
    for sid, toks in enumerate(seqs):
        idx, jobs = t.add_seq(toks)
        order.insert(idx, sid)
        # copy jobs cover exactly the unmatched suffix, chunk by chunk
        if jobs:
            assert jobs[-1].tok_end == len(toks)
            assert all(j.tok_end - j.tok_begin <= c for j in jobs)
            assert all(a.tok_end == b.tok_begin for a, b in zip(jobs, jobs[1:]))
    want_order, counts = brute_force_order(seqs, c)
    assert order == want_order
    for i, sid in enumerate(order):
        assert t.seq_tokens(i) == seqs[sid]
    # sharing counts of every full-chunk prefix
    for row in t.get_chunks():
        node, prefix = row.chunk, []
        n = node
        parts = []
        while n is not None:
            parts.append(n.tokens)
            n = n.parent
        for p in reversed(parts):
            prefix.extend(p)
        if node.children:  # internal => full
            assert counts[tuple(prefix)] == node.n_seqs == row.seq_end - row.seq_begin


def check_invariants(t):
    rows = t.get_chunks()
    assert t.root.n_seqs == len(t.tails)
    seen_leaf = 0
    for r in rows:
        ch = r.chunk
        assert r.seq_end - r.seq_begin == ch.n_seqs >= 1
        if ch.children:
            assert ch.full()
            assert sum(k.n_seqs for k in ch.children) == ch.n_seqs
        else:
            assert ch.n_seqs == 1
            assert t.tails[r.seq_begin] is ch
            seen_leaf += 1
    assert seen_leaf == len(t.tails)
    assert len(rows) == t.alloc.max_chunks - len(t.alloc.free)


@pytest.mark.parametrize("seed", range(8))
def test_random_histories_keep_invariants(seed):
    rng = random.Random(100 + seed)
    c = rng.choice([2, 4])
    t = PrefixTree(c, 4096)
    model = []  # token lists in sequence order
    for _ in range(120):
        op = rng.random()
        if op < 0.45 or not model:
            toks = [rng.randint(0, 2) for _ in range(rng.randint(1, 10))]
            idx, _ = t.add_seq(toks)
            model.insert(idx, list(toks))
        elif op < 0.7:
            new = [rng.randint(0, 2) for _ in model]
            t.append_token(new)
            for m, x in zip(model, new):
                m.append(x)
        else:
            i = rng.randrange(len(model))
            t.remove_seq(i)
            del model[i]
        check_invariants(t)
        assert [t.seq_tokens(i) for i in range(len(model))] == model


# ---- beam-search operations (reference attention.cpp:227-261, 287-313; the reference's own
# ---- test_duplicate is skipped, so these are pinned by hand-worked trees, the token-list model
# ---- and the tree invariants) ------------------------------------------------------------------

def test_duplicate_hand_worked():
    t = PrefixTree(2, 64)
    t.add_seq([1, 2, 3])          # root -> [1,2] -> [3]
    t.add_seq([1, 2, 4, 5])       # [1,2] -> [4,5] -> []
    pairs = t.duplicate(0, 2)     # two more copies of sequence 0, right after it
    #   root(4) -> [1,2](4) -> { [3](1), [3](1), [3](1), [4,5](1) -> [](1) }
    assert t.structure() == (4, (), [(4, (1, 2), [(1, (3,), []), (1, (3,), []), (1, (3,), []),
                                                  (1, (4, 5), [(1, (), [])])])])
    assert [t.seq_tokens(i) for i in range(4)] == [[1, 2, 3]] * 3 + [[1, 2, 4, 5]]
    src = t.tails[0].slot
    assert pairs == [(src, t.tails[1].slot), (src, t.tails[2].slot)]
    assert len({c.slot for c in t.tails}) == 4
    assert t.duplicate(1, 0) == [] and t.n_seqs == 4
    check_invariants(t)


def test_append_completion_hand_worked():
    t = PrefixTree(2, 64)
    t.add_seq([1, 2, 3])
    t.add_seq([1, 2, 4, 5])
    # three candidates for sequence 0; its tail [3] has one free row, so every candidate fills
    # its chunk and gets an empty child at once
    pairs, targets = t.append_completion(0, [7, 8, 9])
    assert t.structure() == (4, (), [(4, (1, 2), [(1, (3, 7), [(1, (), [])]), (1, (3, 8), [(1, (), [])]),
                                                  (1, (3, 9), [(1, (), [])]), (1, (4, 5), [(1, (), [])])])])
    assert [t.seq_tokens(i) for i in range(4)] == [[1, 2, 3, 7], [1, 2, 3, 8], [1, 2, 3, 9], [1, 2, 4, 5]]
    first = t.tails[0].parent
    assert targets[0] == (first.slot, 1)                     # row 1 of the chunk that held [3]
    assert [p[0] for p in pairs] == [first.slot, first.slot]
    assert targets[1:] == [(p[1], 1) for p in pairs]
    # a full tail without a child (append_token leaves it so) first gets its empty child
    t2 = PrefixTree(2, 64)
    t2.add_seq([1])
    t2.append_token([2])
    assert t2.tails[0].full() and not t2.tails[0].children
    _, tg = t2.append_completion(0, [5, 6])
    assert [t2.seq_tokens(i) for i in range(2)] == [[1, 2, 5], [1, 2, 6]]
    assert tg[0][1] == 0 and tg[1][1] == 0
    check_invariants(t2)
    # a single candidate is an append to one sequence only
    t2.append_completion(1, [9])
    assert [t2.seq_tokens(i) for i in range(2)] == [[1, 2, 5], [1, 2, 6, 9]]
    check_invariants(t2)


def test_beam_operations_capacity():
    t = PrefixTree(2, 3)
    t.add_seq([1, 2, 3])                     # uses 2 chunks
    before = t.structure()
    with pytest.raises(RuntimeError, match="capacity reached"):
        t.append_completion(0, [4, 5])       # would need 3 more chunks
    assert t.structure() == before           # nothing changed


@pytest.mark.parametrize("seed", range(8))
def test_random_histories_with_beam_operations(seed):
    rng = random.Random(500 + seed)
    c = rng.choice([2, 3, 4])
    t = PrefixTree(c, 8192)
    model = []
    for _ in range(150):
        op = rng.random()
        if op < 0.3 or not model:
            toks = [rng.randint(0, 2) for _ in range(rng.randint(1, 10))]
            idx, _ = t.add_seq(toks)
            model.insert(idx, list(toks))
        elif op < 0.5:
            new = [rng.randint(0, 2) for _ in model]
            t.append_token(new)
            for m, x in zip(model, new):
                m.append(x)
        elif op < 0.65:
            i, n = rng.randrange(len(model)), rng.randint(0, 3)
            pairs = t.duplicate(i, n)
            assert len(pairs) == n
            for k in range(n):
                model.insert(i + 1 + k, list(model[i]))
        elif op < 0.85:
            i = rng.randrange(len(model))
            cand = [rng.randint(0, 2) for _ in range(rng.randint(1, 4))]
            pairs, targets = t.append_completion(i, cand)
            assert len(pairs) == len(cand) - 1 and len(targets) == len(cand)
            base = model[i]
            for k in range(1, len(cand)):
                model.insert(i + k, base + [cand[k]])
            model[i] = base + [cand[0]]
            for k, (slot, row) in enumerate(targets):     # the row named is where the token sits
                node = t.tails[i + k] if t.tails[i + k].n_tokens else t.tails[i + k].parent
                assert (node.slot, node.n_tokens - 1) == (slot, row) and node.tokens[-1] == cand[k]
        else:
            i = rng.randrange(len(model))
            t.remove_seq(i)
            del model[i]
        check_invariants(t)
        assert [t.seq_tokens(i) for i in range(len(model))] == model
