"""Shared test helpers: build a host-side (numpy) KV pool from an oracle tree."""
import numpy as np

from oracle.prefix_tree import PrefixTree


def build_host_case(seq_tokens, seq_kv, chunk_size, n_heads, d_head, max_chunks=None, dtype=np.float32):
    """Inserts sequences into an oracle tree and fills numpy pools [max_chunks, H, c, d] the way
    add_seq copies K/V in.  seq_kv[s] = (k, v) as [T, H, d].  Returns (tree, kpool, vpool, order)
    where order[i] is the id of the sequence sitting at index i."""
    if max_chunks is None:
        max_chunks = sum(len(t) // chunk_size + 2 for t in seq_tokens)
    tree = PrefixTree(chunk_size, max_chunks)
    kpool = np.zeros((max_chunks, n_heads, chunk_size, d_head), dtype)
    vpool = np.zeros((max_chunks, n_heads, chunk_size, d_head), dtype)
    order = []
    for sid, toks in enumerate(seq_tokens):
        idx, jobs = tree.add_seq(toks)
        order.insert(idx, sid)
        k, v = seq_kv[sid]
        for j in jobs:
            n = j.tok_end - j.tok_begin
            kpool[j.slot][:, :n, :] = np.transpose(k[j.tok_begin:j.tok_end], (1, 0, 2))
            vpool[j.slot][:, :n, :] = np.transpose(v[j.tok_begin:j.tok_end], (1, 0, 2))
    return tree, kpool, vpool, order


def rows_of(tree):
    return [r.as_tuple() for r in tree.get_chunks()]
