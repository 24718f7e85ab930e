"""Known-answer data transcribed from the reference's own tests (expectations only).

ADD_SEQ_STEPS: tests/test_chunk_attn_cpu.py:24-175 of the reference -- six inserts with
chunk_size 2; after each, the expected tree as nested (n_seqs, tokens, [children]) and the
expected tails (as the tokens of each tail chunk plus its position path in the tree).
"""

# (tokens inserted, expected tree, expected tail paths [child indices from the root])
ADD_SEQ_STEPS = [
    ([1, 2, 3, 4, 5],
     (1, (), [(1, (1, 2), [(1, (3, 4), [(1, (5,), [])])])]),
     [(0, 0, 0)]),
    ([1, 2, 3, 4, 6],
     (2, (), [(2, (1, 2), [(2, (3, 4), [(1, (5,), []), (1, (6,), [])])])]),
     [(0, 0, 0), (0, 0, 1)]),
    ([1, 2, 3, 4],
     (3, (), [(3, (1, 2), [(3, (3, 4), [(1, (5,), []), (1, (6,), []), (1, (), [])])])]),
     [(0, 0, 0), (0, 0, 1), (0, 0, 2)]),
    ([1, 7],
     (4, (), [(3, (1, 2), [(3, (3, 4), [(1, (5,), []), (1, (6,), []), (1, (), [])])]),
              (1, (1, 7), [(1, (), [])])]),
     [(0, 0, 0), (0, 0, 1), (0, 0, 2), (1, 0)]),
    ([1, 2],
     (5, (), [(4, (1, 2), [(3, (3, 4), [(1, (5,), []), (1, (6,), []), (1, (), [])]),
                           (1, (), [])]),
              (1, (1, 7), [(1, (), [])])]),
     [(0, 0, 0), (0, 0, 1), (0, 0, 2), (0, 1), (1, 0)]),
    ([1, 2, 3, 4, 5],
     (6, (), [(5, (1, 2), [(4, (3, 4), [(1, (5,), []), (1, (6,), []), (1, (), []), (1, (5,), [])]),
                           (1, (), [])]),
              (1, (1, 7), [(1, (), [])])]),
     [(0, 0, 0), (0, 0, 1), (0, 0, 2), (0, 0, 3), (0, 1), (1, 0)]),
]

# tests/test_chunk_attn_cpu.py:177-215: two inserts then one append_token([8, 9]), chunk_size 2
APPEND_CASE = {
    "adds": [[1, 2, 3, 4, 5], [1, 2, 3, 4, 6, 7]],
    "append": [8, 9],
    "tree": (2, (), [(2, (1, 2), [(2, (3, 4), [(1, (5, 8), []), (1, (6, 7), [(1, (9,), [])])])])]),
    "tails": [(0, 0, 0), (0, 0, 1, 0)],
}

# tests/test_chunk_attn_cpu.py:267-303: two inserts, remove_seq(0), chunk_size 2
REMOVE_CASE = {
    "adds": [[1, 2, 3, 4, 5], [1, 2, 3, 4, 6]],
    "remove": 0,
    "tree": (1, (), [(1, (1, 2), [(1, (3, 4), [(1, (6,), [])])])]),
}

# Tables of the tree after ADD_SEQ_STEPS, derived by hand from the reference's table builder
# (cpp/chunk_attn/kernel_cuda.cu:1343-1410), tpp_threshold 1, chunk_size 2.  Rows are listed
# as (tokens, seq_begin, seq_end) in get_chunks order (children visited last-to-first).
TABLE_KAT = {
    "rows": [((1, 7), 5, 6), ((), 5, 6), ((1, 2), 0, 5), ((), 4, 5), ((3, 4), 0, 4),
             ((5,), 3, 4), ((), 2, 3), ((6,), 1, 2), ((5,), 0, 1)],
    "n_shared": 2,
    "final_idx": [2, 3, 0, 4, 1, 5, 6, 7, 8],
    "begins": [0, 0], "ends": [5, 4], "offsets": [0, 5], "partial_rows": 9,
    "seq_n_tokens": [5, 5, 4, 5, 2, 2],
    "max_seq_n_chunks": 3,
    "seq_chunk_map": [[0, 1, 8], [0, 1, 7], [0, 1, 6], [0, 1, 5], [0, 4, -1], [2, 3, -1]],
}
