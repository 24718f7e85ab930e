"""Helpers for the GPU parity tests: drive the HIP path through the C-ABI (ctypes) and mirror
its state into numpy for the oracle."""
import numpy as np
import torch

from chunk_attn import capi, synth
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


def load_workload(w: synth.Workload, seed=0, tpp_threshold=1):
    need = sum(w.seq_len(s) // w.chunk_size + 2 for s in range(w.n_seqs)) + w.n_seqs * (w.append_steps // w.chunk_size + 1)
    attn = make_attention(w.n_heads, w.chunk_size, need, tpp_threshold)
    order = []
    for s in range(w.n_seqs):
        k, v = w.kv(s, seed)
        idx = attn.add_seq(w.tokens(s), to_dev(k), to_dev(v))
        order.insert(idx, s)
    return attn, order


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
