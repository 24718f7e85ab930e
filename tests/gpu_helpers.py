"""Helpers for the GPU parity tests: drive the HIP path through the C-ABI (ctypes) and mirror
its state into numpy for the oracle."""
import numpy as np
import torch

import synth
from chunk_attn import capi
from oracle.attention_ref import CpuAttention, textbook_attention

ATOL, RTOL = 2e-3, 1e-2   # fp16 out, fp32 accumulate: tolerance of the decode path


def dev():
    return torch.device("cuda:0")


def to_dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev())


def make_attention(n_heads, chunk_size, n_chunks_needed, tpp_threshold=1, share_prefix=True):
    per_chunk = chunk_size * n_heads * 128 * 2 * 2
    memory_mb = max(1, -(-(n_chunks_needed + 4) * per_chunk // (1 << 20)))
    return capi.Attention(n_heads=n_heads, d_head=128, chunk_size=chunk_size, memory_mb=memory_mb,
                          share_prefix=share_prefix, tpp_threshold=tpp_threshold,
                          dtype=torch.float16, device=dev())


def load_workload(w: synth.Workload, seed=0, tpp_threshold=1, keep=None):
    """Inserts every sequence of the workload; returns (attn, order).  keep: None draws all K/V
    on the host (w.kv).  Otherwise (workloads of several GiB) K/V are drawn on the device with
    the same generator (w.kv_torch) and host copies of the tensors handed to add_seq are kept for
    the sequences in `keep`: returns (attn, order, {seq: (k, v)})."""
    need = sum(w.seq_len(s) // w.chunk_size + 2 for s in range(w.n_seqs)) + w.n_seqs * (w.append_steps // w.chunk_size + 1)
    attn = make_attention(w.n_heads, w.chunk_size, need, tpp_threshold)
    order, kept = [], {}
    for s in range(w.n_seqs):
        if keep is None:
            k, v = (to_dev(a) for a in w.kv(s, seed))
        else:
            k, v = w.kv_torch(s, seed, dev())
            if s in keep:
                kept[s] = (k.cpu().numpy(), v.cpu().numpy())
        idx = attn.add_seq(w.tokens(s), k, v)
        order.insert(idx, s)
    return (attn, order) if keep is None else (attn, order, kept)


def oracle_tree_rows(w: synth.Workload):
    """get_chunks rows of the oracle's prefix tree after the same insertions (slots included:
    both managers hand out the lowest free slot)."""
    from oracle.prefix_tree import PrefixTree
    need = sum(w.seq_len(s) // w.chunk_size + 2 for s in range(w.n_seqs))
    tree = PrefixTree(w.chunk_size, need + 4)
    for s in range(w.n_seqs):
        tree.add_seq(w.tokens(s))
    return np.asarray([r.as_tuple() for r in tree.get_chunks()], np.int32).reshape(-1, 4)


def assert_chunk_holds(attn, w: synth.Workload, seq: int, path_pos: int, seed=0, kv=None):
    """The chunk at position path_pos of sequence seq's root->leaf path holds exactly the K/V
    rows the workload generates for those tokens (bit-exact: checks the copy-in independently
    of anything read back for the attention oracle)."""
    rows = attn.get_chunks()
    path = [r for r in rows.tolist() if r[2] <= seq < r[3]]
    slot, n_tok = path[path_pos][0], path[path_pos][1]
    assert n_tok > 0
    k, v = kv if kv is not None else w.kv(seq, seed)
    c = w.chunk_size
    kp, vp = attn.pool_views()
    torch.cuda.synchronize()
    got_k = kp[slot].cpu().numpy()[:, :n_tok, :]
    got_v = vp[slot].cpu().numpy()[:, :n_tok, :]
    np.testing.assert_array_equal(got_k, np.transpose(k[path_pos * c: path_pos * c + n_tok], (1, 0, 2)))
    np.testing.assert_array_equal(got_v, np.transpose(v[path_pos * c: path_pos * c + n_tok], (1, 0, 2)))


def textbook_on_original(w: synth.Workload, q_np: np.ndarray, seq: int, seed=0, kv=None) -> np.ndarray:
    """float64 softmax attention of sequence seq over the K/V the workload generates for it
    (kv: the tensors handed to add_seq; never anything read back from the cache).  Returns [H, d]."""
    k, v = kv if kv is not None else w.kv(seq, seed)
    k = np.transpose(k, (1, 0, 2)).astype(np.float64)
    v = np.transpose(v, (1, 0, 2)).astype(np.float64)
    sc = np.einsum("hd,htd->ht", q_np[seq].astype(np.float64), k) / np.sqrt(q_np.shape[2])
    p = np.exp(sc - sc.max(axis=1, keepdims=True))
    return np.einsum("ht,htd->hd", p / p.sum(axis=1, keepdims=True), v)


def host_state(attn, as_float=True):
    """(rows, kpool, vpool) of the GPU cache as numpy (fp32 unless as_float=False), for the oracle."""
    rows = attn.get_chunks()
    top = int(rows[:, 0].max()) + 1 if len(rows) else 0
    kp, vp = attn.pool_views()
    torch.cuda.synchronize()
    if not as_float:
        return rows, kp[:top].cpu().numpy(), vp[:top].cpu().numpy()
    return rows, kp[:top].float().cpu().numpy(), vp[:top].float().cpu().numpy()


def oracle_output(attn, q_np: np.ndarray, partition=0, exact=False):
    rows, kpool, vpool = host_state(attn)
    # tail rows beyond n_tokens may hold stale data on the GPU; the oracle never reads them
    if exact:
        return textbook_attention(q_np.astype(np.float32), rows.tolist(), kpool, vpool)
    return CpuAttention().attention(q_np.astype(np.float32), rows.tolist(), kpool, vpool, partition)


def assert_close(got: torch.Tensor, want: np.ndarray, atol=ATOL, rtol=RTOL):
    g = got.float().cpu().numpy()
    assert np.isfinite(g).all()
    err = np.abs(g - want)
    tol = atol + rtol * np.abs(want)
    bad = err > tol
    assert not bad.any(), "max abs err %.3e at %s (want %.4f got %.4f), %d bad" % (
        err.max(), np.unravel_index(err.argmax(), err.shape), want.flat[err.argmax()], g.flat[err.argmax()], bad.sum())
    return float(err.max())
