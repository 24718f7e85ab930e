"""Numeric side of the oracle: TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

  * textbook_attention / textbook_partials: float64 closed-form softmax attention, the
    check the reference's own tests apply (tests/test_chunk_attn_cpu.py:234-265,333-385,
    tests/test_chunk_attn_cuda.py:37-44, cpp/tests/test_gpu_kernel.cpp:36-62).
  * CpuAttention: ctypes handle on oracle/libca_oracle.so, the C restatement of the
    reference's fp32 two-phase CPU path (cpp/chunk_attn/kernel_cpu_mkl.cpp).
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess
from typing import Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libca_oracle.so")


def build(force: bool = False) -> str:
    """Compile oracle/cpu_attn.c with gcc (a checker build, not a product build)."""
    if force or not os.path.exists(_LIB) or os.path.getmtime(_LIB) < os.path.getmtime(
            os.path.join(_HERE, "cpu_attn.c")):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libca_oracle.so"])
    return _LIB


def gather_seq_kv(rows: Sequence[Tuple[int, int, int, int]], seq: int, kpool: np.ndarray,
                  vpool: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """Concatenate the K/V of every chunk covering `seq`, in get_chunks (root->leaf) order.
    kpool/vpool: [max_chunks, H, c, d].  Returns [H, T, d] arrays."""
    ks, vs = [], []
    for (slot, nt, b, e) in rows:
        if b <= seq < e and nt > 0:
            ks.append(kpool[slot][:, :nt, :])
            vs.append(vpool[slot][:, :nt, :])
    H, d = kpool.shape[1], kpool.shape[3]
    if not ks:
        return np.zeros((H, 0, d), kpool.dtype), np.zeros((H, 0, d), vpool.dtype)
    return np.concatenate(ks, axis=1), np.concatenate(vs, axis=1)


def textbook_attention(q: np.ndarray, rows, kpool: np.ndarray, vpool: np.ndarray) -> np.ndarray:
    """softmax(q k^T / sqrt(d)) v per sequence and head in float64.  q: [B, H, d]."""
    B, H, d = q.shape
    out = np.zeros((B, H, d), np.float64)
    for s in range(B):
        k, v = gather_seq_kv(rows, s, kpool, vpool)
        k = k.astype(np.float64)
        v = v.astype(np.float64)
        sc = np.einsum("hd,htd->ht", q[s].astype(np.float64), k) / math.sqrt(d)
        sc -= sc.max(axis=1, keepdims=True)
        p = np.exp(sc)
        p /= p.sum(axis=1, keepdims=True)
        out[s] = np.einsum("ht,htd->hd", p, v)
    return out


def textbook_partials(q: np.ndarray, slot: int, n_tokens: int, b: int, e: int, kpool, vpool):
    """Per-chunk (max, sum, unnormalised P.V) for sequences [b, e), natural-log units, as
    cpp/tests/test_gpu_kernel.cpp:36-62 computes them.  Returns ([H,n], [H,n], [H,n,d])."""
    d = q.shape[2]
    k = kpool[slot][:, :n_tokens, :].astype(np.float64)
    v = vpool[slot][:, :n_tokens, :].astype(np.float64)
    qq = q[b:e].astype(np.float64).transpose(1, 0, 2)       # [H, n, d]
    sc = np.einsum("hnd,htd->hnt", qq, k) / math.sqrt(d)
    m = sc.max(axis=2)
    p = np.exp(sc - m[:, :, None])
    return m, p.sum(axis=2), np.einsum("hnt,htd->hnd", p, v)


class CpuAttention:
    """ctypes view of the C restatement.  `blas`: 'auto' hands MKL's sgemm_/vsExp from the
    PyTorch wheel's libtorch_cpu.so to the C code when they can be found, 'none' keeps the
    plain C loops."""

    def __init__(self, blas: str = "auto"):
        self.lib = ctypes.CDLL(build())
        fp = ctypes.POINTER(ctypes.c_float)
        ip = ctypes.POINTER(ctypes.c_int)
        for name in ("ca_oracle_chunk_first", "ca_oracle_seq_first"):
            fn = getattr(self.lib, name)
            fn.argtypes = [fp, fp, fp, ip] + [ctypes.c_int] * 5 + [fp, ctypes.c_int]
            fn.restype = ctypes.c_int
        self.lib.ca_oracle_attention.argtypes = [fp, fp, fp, ip] + [ctypes.c_int] * 5 + [
            fp, ctypes.c_int, ctypes.c_int]
        self.lib.ca_oracle_attention.restype = ctypes.c_int
        self.lib.ca_oracle_set_blas.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.blas_source = "plain C loops"
        self._keep = None
        if blas == "auto":
            self._try_mkl()
        else:
            self.lib.ca_oracle_set_blas(None, None)

    def _try_mkl(self) -> None:
        try:
            import torch  # only to locate the wheel's MKL-carrying library
            path = os.path.join(os.path.dirname(torch.__file__), "lib", "libtorch_cpu.so")
            mkl = ctypes.CDLL(path)
            sgemm = ctypes.cast(mkl.sgemm_, ctypes.c_void_p).value
            vsexp = ctypes.cast(mkl.vsExp, ctypes.c_void_p).value
            self.lib.ca_oracle_set_blas(sgemm, vsexp)
            self._keep = mkl
            self.blas_source = "MKL sgemm_/vsExp from " + path
        except (OSError, AttributeError, ImportError):
            self.lib.ca_oracle_set_blas(None, None)

    @property
    def max_threads(self) -> int:
        return int(self.lib.ca_oracle_max_threads())

    def attention(self, q: np.ndarray, rows, kpool: np.ndarray, vpool: np.ndarray,
                  partition: int = 0, n_threads: int = 0) -> np.ndarray:
        """q [B,H,d] fp32; pools [max_chunks,H,c,d] fp32; rows (slot,n_tokens,b,e)."""
        q = np.ascontiguousarray(q, np.float32)
        kpool = np.ascontiguousarray(kpool, np.float32)
        vpool = np.ascontiguousarray(vpool, np.float32)
        rows_a = np.ascontiguousarray(np.asarray(rows, np.int32).reshape(-1, 4))
        B, H, d = q.shape
        c = kpool.shape[2]
        out = np.empty((B, H, d), np.float32)
        fp = ctypes.POINTER(ctypes.c_float)
        rc = self.lib.ca_oracle_attention(
            q.ctypes.data_as(fp), kpool.ctypes.data_as(fp), vpool.ctypes.data_as(fp),
            rows_a.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), rows_a.shape[0], B, H, d, c,
            out.ctypes.data_as(fp), partition, n_threads)
        if rc != 0:
            raise RuntimeError("Unsupported partition type")
        return out
