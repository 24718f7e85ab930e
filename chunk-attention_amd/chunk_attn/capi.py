"""ctypes binding of libchunkattn_hip.so (the C-ABI declared in include/chunk_attn_hip.h).

`Tree` wraps the prefix-tree manager handle, `KernelContext` the device-side context, and
`Attention` composes both over a torch-allocated fp16 KV pool with the same methods as the
pybind11 class (add_seq / append_token / forward / remove_seq / reserve /
refresh_kernel_context), for hosts that cannot load the C++ extension module.

There is no CPU fallback: loading fails if the library has not been built, and every device
entry point reports an error when no HIP device is present.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Optional, Sequence, Tuple

import numpy as np

_LIB_PATH = os.environ.get("CHUNK_ATTN_HIP_LIB") or os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "lib", "libchunkattn_hip.so")
_lib = None

c_int_p = ctypes.POINTER(ctypes.c_int)
c_i32_p = ctypes.POINTER(ctypes.c_int32)
c_f32_p = ctypes.POINTER(ctypes.c_float)


class ChunkRow(ctypes.Structure):
    _fields_ = [("slot", ctypes.c_int32), ("n_tokens", ctypes.c_int32),
                ("seq_begin", ctypes.c_int32), ("seq_end", ctypes.c_int32)]


class PlanInfo(ctypes.Structure):
    _fields_ = [("n_seqs", ctypes.c_int32), ("n_chunks", ctypes.c_int32),
                ("n_shared_chunks", ctypes.c_int32), ("ref_partial_rows", ctypes.c_int32),
                ("max_seq_n_chunks", ctypes.c_int32), ("n_shared_items", ctypes.c_int32),
                ("n_stream_items", ctypes.c_int32), ("n_part_rows", ctypes.c_int32),
                ("shared_tokens", ctypes.c_int64), ("stream_tokens", ctypes.c_int64),
                ("stream_per_wave", ctypes.c_int32), ("reserved", ctypes.c_int32)]


# name -> (restype, argtypes); every symbol include/chunk_attn_hip.h declares
SIGNATURES = {
    "ca_last_error": (ctypes.c_char_p, []),
    "ca_ctx_create": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_int,
                                     ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                     ctypes.c_int]),
    "ca_ctx_destroy": (None, [ctypes.c_void_p]),
    "ca_refresh_kernel_context": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ChunkRow),
                                                 ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "ca_ctx_roll_tails": (ctypes.c_int, [ctypes.c_void_p, c_i32_p, c_i32_p, ctypes.c_int, ctypes.c_void_p]),
    "ca_ctx_valid": (ctypes.c_int, [ctypes.c_void_p]),
    "ca_ctx_invalidate": (None, [ctypes.c_void_p]),
    "ca_ctx_delta_tokens": (ctypes.c_int, [ctypes.c_void_p]),
    "ca_ctx_set_delta_tokens": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "ca_attention": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                    ctypes.c_int, ctypes.c_void_p]),
    "ca_attention_noalloc": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                            ctypes.c_void_p]),
    "ca_attn_chunks_first": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                            ctypes.c_void_p]),
    "ca_attn_seqs_first": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                          ctypes.c_int, ctypes.c_void_p]),
    "ca_append_kv": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                    ctypes.c_void_p]),
    "ca_decode_step": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                      ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]),
    "ca_rotary_embedding": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                           ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                           ctypes.c_void_p]),
    "ca_rms_norm": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float,
                                   ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]),
    "ca_fused_add_rms_norm": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float,
                                             ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]),
    "ca_rope_append_kv": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                         ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "ca_scatter_kv": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                     ctypes.c_int, c_i32_p, ctypes.c_int, ctypes.c_void_p]),
    "ca_copy_chunk": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "ca_copy_chunks": (ctypes.c_int, [ctypes.c_void_p, c_i32_p, ctypes.c_int, ctypes.c_void_p]),
    "ca_copy_chunks_put_rows": (ctypes.c_int, [ctypes.c_void_p, c_i32_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                               ctypes.c_int, c_i32_p, ctypes.c_void_p]),
    "ca_put_kv_rows": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, c_i32_p,
                                      ctypes.c_void_p]),
    "ca_ctx_set_plan": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]),
    "ca_ctx_set_replan": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "ca_ctx_table_stats": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64)]),
    "ca_ctx_set_schedule": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "ca_ctx_set_stream_hint": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "ca_set_markers": (ctypes.c_int, [ctypes.c_int]),
    "ca_ctx_set_timing": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "ca_bench_decode_launch": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                              ctypes.c_int, ctypes.c_void_p]),
    "ca_bench_read_probe": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int,
                                           ctypes.c_void_p]),
    "ca_ctx_read_timing": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_double),
                                          ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double),
                                          ctypes.POINTER(ctypes.c_int64), ctypes.c_int]),
    "ca_ctx_plan_info": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(PlanInfo)]),
    "ca_ctx_ref_tables": (ctypes.c_int, [ctypes.c_void_p] + [c_i32_p] * 7),
    "ca_ctx_export_partials": (ctypes.c_int, [ctypes.c_void_p, c_f32_p, c_f32_p, c_f32_p,
                                              ctypes.c_void_p]),
    "ca_ctx_read_partials_raw": (ctypes.c_int, [ctypes.c_void_p, c_f32_p, ctypes.c_int64, ctypes.c_void_p]),
    "ca_tables_build": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ChunkRow)] +
                        [ctypes.c_int] * 9),
    "ca_tables_build_like": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p,
                                            ctypes.POINTER(ChunkRow), ctypes.c_int, ctypes.c_int]),
    "ca_tables_roll_tails": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, c_i32_p, c_i32_p, ctypes.c_int]),
    "ca_tables_stale": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_int64]),
    "ca_tables_destroy": (None, [ctypes.c_void_p]),
    "ca_tables_info": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(PlanInfo)]),
    "ca_tables_plan_sizes": (ctypes.c_int, [ctypes.c_void_p, c_int_p]),
    "ca_tables_ref": (ctypes.c_int, [ctypes.c_void_p] + [c_i32_p] * 7),
    "ca_tables_plan": (ctypes.c_int, [ctypes.c_void_p] + [c_i32_p] * 7),
    "ca_tree_create": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_int,
                                      ctypes.c_int]),
    "ca_tree_destroy": (None, [ctypes.c_void_p]),
    "ca_tree_max_chunks_for": (ctypes.c_int, [ctypes.c_int] * 5),
    "ca_tree_add_seq": (ctypes.c_int, [ctypes.c_void_p, c_i32_p, ctypes.c_int, c_int_p, c_int_p,
                                       c_i32_p, ctypes.c_int, c_int_p]),
    "ca_tree_remove_seq": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "ca_tree_clear": (ctypes.c_int, [ctypes.c_void_p]),
    "ca_tree_reserve": (ctypes.c_int, [ctypes.c_void_p, c_int_p]),
    "ca_tree_reserve_tails": (ctypes.c_int, [ctypes.c_void_p, c_i32_p, c_i32_p, ctypes.c_int, c_int_p]),
    "ca_tree_append_token": (ctypes.c_int, [ctypes.c_void_p, c_i32_p, ctypes.c_int, c_int_p]),
    "ca_tree_get_chunks": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ChunkRow), ctypes.c_int,
                                          c_int_p]),
    "ca_tree_n_seqs": (ctypes.c_int, [ctypes.c_void_p]),
    "ca_tree_used_chunks": (ctypes.c_int, [ctypes.c_void_p]),
    "ca_tree_version": (ctypes.c_uint64, [ctypes.c_void_p]),
    "ca_tree_tails": (ctypes.c_int, [ctypes.c_void_p, c_i32_p, ctypes.c_int, c_int_p]),
    "ca_tree_duplicate": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, c_i32_p, ctypes.c_int,
                                         c_int_p]),
    "ca_tree_append_completion": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, c_i32_p, ctypes.c_int, c_i32_p,
                                                 ctypes.c_int, c_int_p, c_i32_p]),
    "ca_tree_dump": (ctypes.c_int, [ctypes.c_void_p, c_i32_p, ctypes.c_int, c_int_p, c_i32_p,
                                    ctypes.c_int, c_int_p]),
}


def load() -> ctypes.CDLL:
    """The C-ABI library, with argument types set.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(
                f"{_LIB_PATH} is missing: build it with `python chunk-attention_amd/build.py` "
                "(the decode path has no fallback implementation)")
        lib = ctypes.CDLL(_LIB_PATH)
        # CHUNK_ATTN_HOST_ONLY=1: the library is a checking build of the host-only half (tables and
        # prefix tree, e.g. the sanitizer build): device entry points are absent and stay unbound
        host_only = os.environ.get("CHUNK_ATTN_HOST_ONLY") == "1"
        for name, (res, args) in SIGNATURES.items():
            if host_only and not hasattr(lib, name):
                continue
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class ChunkAttnError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


def _check(rc: int) -> None:
    if rc != 0:
        raise ChunkAttnError(rc, load().ca_last_error().decode())


def set_markers(enable: bool) -> None:
    """Named ranges (roctx) around refreshes, patches, attention calls and appends; off by default."""
    _check(load().ca_set_markers(1 if enable else 0))


def _i32(values: Sequence[int]):
    arr = np.ascontiguousarray(np.asarray(values, dtype=np.int32))
    return arr, arr.ctypes.data_as(c_i32_p)


class Tree:
    """Prefix-tree chunk manager handle (ca_tree_*)."""

    def __init__(self, chunk_size: int, max_chunks: int, share_prefix: bool = True):
        self._lib = load()
        self._h = ctypes.c_void_p()
        _check(self._lib.ca_tree_create(ctypes.byref(self._h), chunk_size, max_chunks, int(share_prefix)))
        self.chunk_size = chunk_size
        self.max_chunks = max_chunks

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h is not None and h.value:
            self._lib.ca_tree_destroy(h)

    def add_seq(self, tokens: Sequence[int]) -> Tuple[int, int, List[int]]:
        """Returns (seq_idx, tok_begin, slots): tokens[tok_begin:] need their K/V copied into
        `slots`, chunk_size rows each."""
        arr, ptr = _i32(tokens)
        cap = len(tokens) // self.chunk_size + 2
        slots = (ctypes.c_int32 * cap)()
        idx, tb, n_new = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        _check(self._lib.ca_tree_add_seq(self._h, ptr, len(tokens), ctypes.byref(idx), ctypes.byref(tb),
                                         slots, cap, ctypes.byref(n_new)))
        return idx.value, tb.value, list(slots[: n_new.value])

    def remove_seq(self, seq_idx: int) -> None:
        _check(self._lib.ca_tree_remove_seq(self._h, seq_idx))

    def clear(self) -> None:
        _check(self._lib.ca_tree_clear(self._h))

    def reserve(self) -> int:
        n = ctypes.c_int()
        _check(self._lib.ca_tree_reserve(self._h, ctypes.byref(n)))
        return n.value

    def reserve_tails(self) -> Tuple[List[int], List[int]]:
        """reserve() that reports what it added: (sequence indices, slots of their new last chunks)."""
        cap = max(self.n_seqs, 1)
        seqs, slots = (ctypes.c_int32 * cap)(), (ctypes.c_int32 * cap)()
        n = ctypes.c_int()
        _check(self._lib.ca_tree_reserve_tails(self._h, seqs, slots, cap, ctypes.byref(n)))
        return list(seqs[: n.value]), list(slots[: n.value])

    def append_token(self, tokens: Sequence[int]) -> int:
        arr, ptr = _i32(tokens)
        n = ctypes.c_int()
        _check(self._lib.ca_tree_append_token(self._h, ptr, len(tokens), ctypes.byref(n)))
        return n.value

    def duplicate(self, seq_idx: int, copies: int) -> List[Tuple[int, int]]:
        """`copies` more sequences identical to seq_idx right after it; returns the (source slot,
        destination slot) pairs whose K/V chunks the caller copies."""
        if copies < 1:
            return []
        pairs = (ctypes.c_int32 * (2 * copies))()
        n = ctypes.c_int()
        _check(self._lib.ca_tree_duplicate(self._h, seq_idx, copies, pairs, copies, ctypes.byref(n)))
        return [(pairs[2 * i], pairs[2 * i + 1]) for i in range(n.value)]

    def append_completion(self, seq_idx: int, tokens: Sequence[int]):
        """One beam-search step on seq_idx.  Returns (copy pairs, targets): chunk copies to make
        first, then targets[i] = (slot, row) of the K/V row of candidate i (sequence seq_idx + i)."""
        n_tok = len(tokens)
        if n_tok < 1:
            return [], []
        arr, ptr = _i32(tokens)
        pairs = (ctypes.c_int32 * (2 * max(n_tok - 1, 1)))()
        targets = (ctypes.c_int32 * (2 * n_tok))()
        n = ctypes.c_int()
        _check(self._lib.ca_tree_append_completion(self._h, seq_idx, ptr, n_tok, pairs, n_tok - 1, ctypes.byref(n),
                                                   targets))
        return ([(pairs[2 * i], pairs[2 * i + 1]) for i in range(n.value)],
                [(targets[2 * i], targets[2 * i + 1]) for i in range(n_tok)])

    def get_chunks(self) -> np.ndarray:
        """[n_rows, 4] int32: slot, n_tokens, seq_begin, seq_end in get_chunks order."""
        n = ctypes.c_int()
        _check(self._lib.ca_tree_get_chunks(self._h, None, 0, ctypes.byref(n)))
        rows = np.zeros((max(n.value, 1), 4), np.int32)
        _check(self._lib.ca_tree_get_chunks(self._h, rows.ctypes.data_as(ctypes.POINTER(ChunkRow)),
                                            n.value, ctypes.byref(n)))
        return rows[: n.value]

    @property
    def n_seqs(self) -> int:
        return self._lib.ca_tree_n_seqs(self._h)

    @property
    def used_chunks(self) -> int:
        return self._lib.ca_tree_used_chunks(self._h)

    @property
    def version(self) -> int:
        return self._lib.ca_tree_version(self._h)

    def tails(self) -> List[int]:
        n = ctypes.c_int()
        cap = max(self.n_seqs, 1)
        buf = (ctypes.c_int32 * cap)()
        _check(self._lib.ca_tree_tails(self._h, buf, cap, ctypes.byref(n)))
        return list(buf[: n.value])

    def dump(self):
        """Pre-order list of (depth, n_seqs, tokens, slot), children first-to-last."""
        nn, nt = ctypes.c_int(), ctypes.c_int()
        _check(self._lib.ca_tree_dump(self._h, None, 0, ctypes.byref(nn), None, 0, ctypes.byref(nt)))
        nodes = np.zeros((max(nn.value, 1), 4), np.int32)
        toks = np.zeros(max(nt.value, 1), np.int32)
        _check(self._lib.ca_tree_dump(self._h, nodes.ctypes.data_as(c_i32_p), nn.value, ctypes.byref(nn),
                                      toks.ctypes.data_as(c_i32_p), nt.value, ctypes.byref(nt)))
        out, pos = [], 0
        for depth, n_seqs, n_tok, slot in nodes[: nn.value].tolist():
            out.append((depth, n_seqs, toks[pos: pos + n_tok].tolist(), slot))
            pos += n_tok
        return out

    def structure(self):
        """Nested (n_seqs, tokens, [children]) like the oracle's PrefixTree.structure()."""
        flat = self.dump()
        root = (flat[0][1], tuple(flat[0][2]), [])
        stack = [(0, root)]
        for depth, n_seqs, toks, _ in flat[1:]:
            node = (n_seqs, tuple(toks), [])
            while stack[-1][0] >= depth:
                stack.pop()
            stack[-1][1][2].append(node)
            stack.append((depth, node))
        return root


def rotary_embedding(positions, query, key, head_size: int, cos_sin_cache, is_neox: bool = True) -> None:
    """In-place rotary embedding of torch fp16 tensors, the operator the reference exports as
    `chunk_attn.ops.rotary_embedding` (python_exports_ops.cpp:13): positions int64 [n_tokens] (or
    [batch, seq]), query [..., n_heads*head_size], key [..., n_kv_heads*head_size], rows
    contiguous, cos_sin_cache [max_position, rot_dim]."""
    import torch
    for name, t in (("query", query), ("key", key), ("cos_sin_cache", cos_sin_cache)):
        if t.dtype != torch.float16 or t.device.type != "cuda":
            raise RuntimeError(f"{name} must be an fp16 tensor on the GPU")
    if positions.dtype != torch.int64 or positions.device != query.device or not positions.is_contiguous():
        raise RuntimeError("positions must be a contiguous int64 tensor on the query's device")
    if query.stride(-1) != 1 or key.stride(-1) != 1 or not cos_sin_cache.is_contiguous():
        raise RuntimeError("query/key rows and cos_sin_cache must be contiguous")
    n_tokens = query.numel() // query.shape[-1]
    if positions.numel() != n_tokens or key.numel() // key.shape[-1] != n_tokens:
        raise RuntimeError("positions, query and key disagree on the number of tokens")
    if query.shape[-1] % head_size or key.shape[-1] % head_size:
        raise RuntimeError("row width is not a multiple of head_size")
    q2 = query.view(n_tokens, query.shape[-1]) if query.is_contiguous() else None
    k2 = key.view(n_tokens, key.shape[-1]) if key.is_contiguous() else None
    q_stride = query.shape[-1] if q2 is not None else query.stride(-2)
    k_stride = key.shape[-1] if k2 is not None else key.stride(-2)
    if (q2 is None or k2 is None) and query.dim() != 2:
        raise RuntimeError("strided query/key must be two-dimensional")
    with torch.cuda.device(query.device):
        stream = torch.cuda.current_stream(query.device).cuda_stream
        _check(load().ca_rotary_embedding(positions.data_ptr(), query.data_ptr(), key.data_ptr(),
                                          cos_sin_cache.data_ptr(), n_tokens, query.shape[-1] // head_size,
                                          key.shape[-1] // head_size, head_size, cos_sin_cache.shape[1],
                                          cos_sin_cache.shape[0], q_stride, k_stride, int(is_neox), stream))


def _norm_args(name, tensors, weight):
    import torch
    hidden = weight.numel()
    for t in tensors + [weight]:
        if t.dtype != torch.float16 or t.device.type != "cuda" or not t.is_contiguous():
            raise RuntimeError(f"{name}: contiguous fp16 tensors on the GPU only")
    for t in tensors:
        if t.shape[-1] != hidden or t.shape != tensors[0].shape:
            raise RuntimeError(f"{name}: rows must be {hidden} wide and of one shape")
    return tensors[0].numel() // hidden, hidden


def rms_norm(out, input, weight, epsilon: float) -> None:
    """out = rms_norm(input) * weight on torch fp16 tensors, the reference's
    `chunk_attn.ops.rms_norm` (python_exports_ops.cpp:16)."""
    import torch
    n, hidden = _norm_args("rms_norm", [input, out], weight)
    with torch.cuda.device(input.device):
        _check(load().ca_rms_norm(out.data_ptr(), input.data_ptr(), weight.data_ptr(), float(epsilon), n, hidden,
                                  torch.cuda.current_stream(input.device).cuda_stream))


def fused_add_rms_norm(input, residual, weight, epsilon: float) -> None:
    """In place: residual += input; input = rms_norm(residual) * weight, the reference's
    `chunk_attn.ops.fused_add_rms_norm` (python_exports_ops.cpp:17)."""
    import torch
    n, hidden = _norm_args("fused_add_rms_norm", [input, residual], weight)
    with torch.cuda.device(input.device):
        _check(load().ca_fused_add_rms_norm(input.data_ptr(), residual.data_ptr(), weight.data_ptr(), float(epsilon),
                                            n, hidden, torch.cuda.current_stream(input.device).cuda_stream))


def max_chunks_for(memory_mb: int, chunk_size: int, n_heads: int, d_head: int, elem_bytes: int = 2) -> int:
    return load().ca_tree_max_chunks_for(memory_mb, chunk_size, n_heads, d_head, elem_bytes)


class HostTables:
    """Host-only table set (ca_tables_*): the flattening ca_refresh_kernel_context performs, and
    the patch ca_ctx_roll_tails applies, without a device."""

    def __init__(self, rows: np.ndarray, n_seqs: int, chunk_size: int = 0, tpp_threshold: int = 1,
                 partition: int = 0, shared_seg_chunks: int = 0, stream_chunks: int = 0,
                 n_heads: int = 32, n_cus: int = 256, like: Optional["HostTables"] = None):
        """like: build for other rows with the parameters and the work-item sizes of that table set
        (what a patched table keeps) instead of the ones given here."""
        self._lib = load()
        rows = np.ascontiguousarray(rows, np.int32).reshape(-1, 4)
        self._h = ctypes.c_void_p()
        rp = rows.ctypes.data_as(ctypes.POINTER(ChunkRow))
        if like is not None:
            _check(self._lib.ca_tables_build_like(ctypes.byref(self._h), like._h, rp, rows.shape[0], n_seqs))
        else:
            _check(self._lib.ca_tables_build(ctypes.byref(self._h), rp, rows.shape[0], n_seqs, chunk_size,
                                             tpp_threshold, partition, shared_seg_chunks, stream_chunks,
                                             n_heads, n_cus))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h is not None and h.value:
            self._lib.ca_tables_destroy(h)

    def roll_tails(self, delta_tokens: int, seqs: Sequence[int], slots: Sequence[int]) -> None:
        a, ap = _i32(seqs)
        b, bp = _i32(slots)
        _check(self._lib.ca_tables_roll_tails(self._h, delta_tokens, ap, bp, len(seqs)))

    def stale(self, percent: int = 25, extra_tokens: int = 0) -> bool:
        """Would the re-planning policy rebuild these tables (attended tokens drifted by more than
        `percent` per cent since their last full build)?"""
        return bool(self._lib.ca_tables_stale(self._h, percent, extra_tokens))

    def info(self) -> PlanInfo:
        info = PlanInfo()
        _check(self._lib.ca_tables_info(self._h, ctypes.byref(info)))
        return info

    def ref(self) -> dict:
        info = self.info()
        t = {
            "final_idx": np.zeros(info.n_chunks, np.int32),
            "slots": np.zeros(info.n_chunks, np.int32),
            "begins": np.zeros(info.n_shared_chunks, np.int32),
            "ends": np.zeros(info.n_shared_chunks, np.int32),
            "offsets": np.zeros(info.n_shared_chunks, np.int32),
            "seq_n_tokens": np.zeros(info.n_seqs, np.int32),
            "seq_chunk_map": np.zeros((info.n_seqs, info.max_seq_n_chunks), np.int32),
        }
        _check(self._lib.ca_tables_ref(self._h, *[t[k].ctypes.data_as(c_i32_p) for k in (
            "final_idx", "slots", "begins", "ends", "offsets", "seq_n_tokens", "seq_chunk_map")]))
        t["n_shared"] = info.n_shared_chunks
        t["partial_rows"] = info.ref_partial_rows
        t["max_seq_n_chunks"] = info.max_seq_n_chunks
        return t

    def plan(self) -> dict:
        info = self.info()
        n_slots = ctypes.c_int()
        _check(self._lib.ca_tables_plan_sizes(self._h, ctypes.byref(n_slots)))
        p = {
            "shared_items": np.zeros((info.n_shared_items, 16), np.int32),
            "stream_items": np.zeros((info.n_stream_items, 16), np.int32),
            "slots": np.zeros(n_slots.value, np.int32),
            "seq_len": np.zeros(info.n_seqs, np.int32),
            "part_ptr": np.zeros(info.n_seqs + 1, np.int32),
            "tail_slot": np.zeros(info.n_seqs, np.int32),
            "tail_fill": np.zeros(info.n_seqs, np.int32),
        }
        _check(self._lib.ca_tables_plan(self._h, *[p[k].ctypes.data_as(c_i32_p) for k in (
            "shared_items", "stream_items", "slots", "seq_len", "part_ptr", "tail_slot", "tail_fill")]))
        p["n_part_rows"] = info.n_part_rows
        p["shared_tokens"] = info.shared_tokens
        p["stream_tokens"] = info.stream_tokens
        p["stream_per_wave"] = info.stream_per_wave
        return p


def build_tables(rows: np.ndarray, n_seqs: int, chunk_size: int, tpp_threshold: int = 1,
                 partition: int = 0, shared_seg_chunks: int = 0, stream_chunks: int = 0,
                 n_heads: int = 32, n_cus: int = 256) -> dict:
    """Host-only flattening of get_chunks rows: reference-form tables and the packed work list
    (work items as [n, 16] int32: seq_begin, n_rows, slot_first, n_chunks, part_row, pos0,
    len0, flags (1 = wide shared item), 8 inline slots; an item writes partial row part_ptr[seq] + part_row of each covered seq)."""
    t = HostTables(rows, n_seqs, chunk_size, tpp_threshold, partition, shared_seg_chunks, stream_chunks,
                   n_heads, n_cus)
    return {"ref": t.ref(), "plan": t.plan()}


class KernelContext:
    """Device-side context handle (ca_ctx_*).  Pointers are raw device addresses."""

    def __init__(self, n_heads: int, d_head: int, chunk_size: int, k_pool_ptr: int, v_pool_ptr: int,
                 max_chunks: int, tpp_threshold: int = 1):
        self._lib = load()
        self._h = ctypes.c_void_p()
        _check(self._lib.ca_ctx_create(ctypes.byref(self._h), n_heads, d_head, chunk_size, k_pool_ptr,
                                       v_pool_ptr, max_chunks, tpp_threshold))
        self.n_heads, self.d_head, self.chunk_size = n_heads, d_head, chunk_size

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h is not None and h.value:
            self._lib.ca_ctx_destroy(h)

    def refresh(self, rows: np.ndarray, n_seqs: int, stream: int = 0) -> None:
        rows = np.ascontiguousarray(rows, np.int32).reshape(-1, 4)
        _check(self._lib.ca_refresh_kernel_context(
            self._h, rows.ctypes.data_as(ctypes.POINTER(ChunkRow)), rows.shape[0], n_seqs, stream))

    def roll_tails(self, seqs: Sequence[int], slots: Sequence[int], stream: int = 0) -> bool:
        """Patches the tables after reserve() gave the sequences `seqs` the new last chunks `slots`
        (and folds delta_tokens in).  False when the tables cannot be patched (they are untouched)."""
        a, ap = _i32(seqs)
        b, bp = _i32(slots)
        rc = self._lib.ca_ctx_roll_tails(self._h, ap, bp, len(seqs), stream)
        if rc == -3:
            return False
        _check(rc)
        return True

    @property
    def valid(self) -> bool:
        return bool(self._lib.ca_ctx_valid(self._h))

    def invalidate(self) -> None:
        self._lib.ca_ctx_invalidate(self._h)

    @property
    def delta_tokens(self) -> int:
        return self._lib.ca_ctx_delta_tokens(self._h)

    @delta_tokens.setter
    def delta_tokens(self, v: int) -> None:
        _check(self._lib.ca_ctx_set_delta_tokens(self._h, v))

    def attention(self, q_ptr: int, out_ptr: int, n_seqs: int, partition: int = 0, stream: int = 0) -> None:
        _check(self._lib.ca_attention(self._h, q_ptr, out_ptr, n_seqs, partition, stream))

    def attention_noalloc(self, q_ptr: int, out_ptr: int, n_seqs: int, stream: int = 0) -> None:
        """ca_attention (partition 0) with the partial rows in the library's static device scratch:
        allocates nothing; fails when the tables need more rows than the scratch holds."""
        _check(self._lib.ca_attention_noalloc(self._h, q_ptr, out_ptr, n_seqs, stream))

    def attn_chunks_first(self, q_ptr: int, n_seqs: int, stream: int = 0) -> None:
        _check(self._lib.ca_attn_chunks_first(self._h, q_ptr, n_seqs, stream))

    def attn_seqs_first(self, q_ptr: int, out_ptr: int, n_seqs: int, stream: int = 0) -> None:
        _check(self._lib.ca_attn_seqs_first(self._h, q_ptr, out_ptr, n_seqs, stream))

    def append_kv(self, k_ptr: int, v_ptr: int, n_seqs: int, stream: int = 0) -> None:
        _check(self._lib.ca_append_kv(self._h, k_ptr, v_ptr, n_seqs, stream))

    def decode_step(self, q_ptr: int, k_ptr: int, v_ptr: int, out_ptr: int, n_seqs: int, stream: int = 0) -> None:
        """append_kv + delta_tokens += 1 + attention (partition 0) in one call, one launch fewer."""
        _check(self._lib.ca_decode_step(self._h, q_ptr, k_ptr, v_ptr, out_ptr, n_seqs, stream))

    def rope_append_kv(self, positions_ptr: int, q_ptr: int, k_ptr: int, v_ptr: int, cache_ptr: int,
                       max_position: int, rot_dim: int, is_neox: bool, n_seqs: int, stream: int = 0) -> None:
        _check(self._lib.ca_rope_append_kv(self._h, positions_ptr or None, q_ptr, k_ptr, v_ptr, cache_ptr,
                                           max_position, rot_dim, int(is_neox), n_seqs, stream))

    def scatter_kv(self, k_ptr: int, v_ptr: int, n_tokens: int, tok_begin: int, slots: Sequence[int],
                   stream: int = 0) -> None:
        arr, ptr = _i32(slots)
        _check(self._lib.ca_scatter_kv(self._h, k_ptr, v_ptr, n_tokens, tok_begin, ptr, len(slots), stream))

    def put_kv_rows(self, k_ptr: int, v_ptr: int, targets: Sequence[Tuple[int, int]], stream: int = 0) -> None:
        """Row i of k/v to row targets[i][1] of chunk targets[i][0]."""
        flat = [x for t in targets for x in t]
        arr, ptr = _i32(flat)
        _check(self._lib.ca_put_kv_rows(self._h, k_ptr, v_ptr, len(targets), ptr, stream))

    def copy_chunk(self, src_slot: int, dst_slot: int, stream: int = 0) -> None:
        _check(self._lib.ca_copy_chunk(self._h, src_slot, dst_slot, stream))

    def copy_chunks(self, pairs: Sequence[Tuple[int, int]], stream: int = 0) -> None:
        """Chunk pairs[i][0] copied onto chunk pairs[i][1], all pairs in one launch."""
        if not pairs:
            return
        arr, ptr = _i32([x for p in pairs for x in p])
        _check(self._lib.ca_copy_chunks(self._h, ptr, len(pairs), stream))

    def copy_chunks_put_rows(self, pairs: Sequence[Tuple[int, int]], k_ptr: int, v_ptr: int,
                             targets: Sequence[Tuple[int, int]], stream: int = 0) -> None:
        """copy_chunks(pairs) then put_kv_rows(targets): one beam-search step's device work, in one
        launch when the rows can be left out of the copies."""
        pa, pp = _i32([x for p in pairs for x in p])
        ta, tp = _i32([x for t in targets for x in t])
        _check(self._lib.ca_copy_chunks_put_rows(self._h, pp, len(pairs), k_ptr, v_ptr, len(targets), tp, stream))

    def set_plan(self, shared_seg_chunks: int = 0, stream_chunks: int = 0) -> None:
        _check(self._lib.ca_ctx_set_plan(self._h, shared_seg_chunks, stream_chunks))

    def set_stream_hint(self, mode: int) -> None:
        """Non-temporal loads of private chunks: 0 by working-set size (default), 1 always, 2 never."""
        _check(self._lib.ca_ctx_set_stream_hint(self._h, int(mode)))

    def set_replan(self, percent: int) -> None:
        """Patched tables are rebuilt once the attended tokens drifted by more than `percent` per cent
        since the last full build (default 25; 0: never)."""
        _check(self._lib.ca_ctx_set_replan(self._h, int(percent)))

    def table_stats(self) -> Tuple[int, int]:
        """(full builds, patches) of the device tables since the context was created."""
        a, b = ctypes.c_int64(), ctypes.c_int64()
        _check(self._lib.ca_ctx_table_stats(self._h, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value

    def set_schedule(self, mode: int) -> None:
        """0: producer launch + merge launch (default); 1: single launch, last finisher merges."""
        _check(self._lib.ca_ctx_set_schedule(self._h, int(mode)))

    def set_timing(self, mode: int) -> None:
        """0 off, 1 time the forward's launches, 2 run and time the three phases separately."""
        _check(self._lib.ca_ctx_set_timing(self._h, int(mode)))

    def bench_decode_launch(self, q_ptr: int, out_ptr: int, n_seqs: int, what: int = 0, stream: int = 0) -> None:
        """Measurement aid: the decode launch alone (0), its stream items alone (1) or its shared items
        alone (2); the output is not complete afterwards."""
        _check(self._lib.ca_bench_decode_launch(self._h, q_ptr, out_ptr, n_seqs, what, stream))

    def bench_read_probe(self, dev_ptr: int, n_bytes: int, wgs_per_cu: int = 1, stream: int = 0) -> None:
        """Measurement aid: one launch that reads n_bytes of device memory and keeps nothing."""
        _check(self._lib.ca_bench_read_probe(self._h, dev_ptr, n_bytes, wgs_per_cu, stream))

    def read_timing(self, reset: bool = True) -> dict:
        """Accumulated per-phase milliseconds of the timed ca_attention calls."""
        a, b, c = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        n = ctypes.c_int64()
        _check(self._lib.ca_ctx_read_timing(self._h, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c),
                                            ctypes.byref(n), int(reset)))
        return {"shared_ms": a.value, "stream_ms": b.value, "merge_ms": c.value, "calls": n.value}

    def plan_info(self) -> PlanInfo:
        info = PlanInfo()
        _check(self._lib.ca_ctx_plan_info(self._h, ctypes.byref(info)))
        return info

    def ref_tables(self) -> dict:
        info = self.plan_info()
        t = {
            "final_idx": np.zeros(info.n_chunks, np.int32),
            "slots": np.zeros(info.n_chunks, np.int32),
            "begins": np.zeros(info.n_shared_chunks, np.int32),
            "ends": np.zeros(info.n_shared_chunks, np.int32),
            "offsets": np.zeros(info.n_shared_chunks, np.int32),
            "seq_n_tokens": np.zeros(info.n_seqs, np.int32),
            "seq_chunk_map": np.zeros((info.n_seqs, info.max_seq_n_chunks), np.int32),
        }
        _check(self._lib.ca_ctx_ref_tables(self._h, *[t[k].ctypes.data_as(c_i32_p) for k in (
            "final_idx", "slots", "begins", "ends", "offsets", "seq_n_tokens", "seq_chunk_map")]))
        t["n_shared"] = info.n_shared_chunks
        t["partial_rows"] = info.ref_partial_rows
        return t

    def read_partials_raw(self, stream: int = 0) -> np.ndarray:
        """[n_part_rows, n_heads, 160] float32 copy of the partial-row buffer."""
        info = self.plan_info()
        out = np.zeros((info.n_part_rows, self.n_heads, 160), np.float32)
        _check(self._lib.ca_ctx_read_partials_raw(self._h, out.ctypes.data_as(c_f32_p), out.size, stream))
        return out

    def export_partials(self, stream: int = 0):
        """(maxs, sums [rows*H], attns [rows*H, d]) in the reference's partial layout."""
        info = self.plan_info()
        n = info.ref_partial_rows * self.n_heads
        maxs = np.zeros(n, np.float32)
        sums = np.zeros(n, np.float32)
        attns = np.zeros((n, self.d_head), np.float32)
        _check(self._lib.ca_ctx_export_partials(self._h, maxs.ctypes.data_as(c_f32_p),
                                                sums.ctypes.data_as(c_f32_p),
                                                attns.ctypes.data_as(c_f32_p), stream))
        return maxs, sums, attns


class Attention:
    """Prefix-tree KV cache + decode attention over the C-ABI, torch tensors in and out.

    Same methods and argument meaning as the pybind11 `Attention` class; chunks are reported
    as pool slot ids instead of node objects."""

    def __init__(self, n_heads: int = 12, d_head: int = 64, chunk_size: int = 64, memory_mb: int = 1024,
                 share_prefix: bool = True, tpp_threshold: int = 1, dtype=None, device=None):
        import torch
        dtype = dtype or torch.get_default_dtype()
        device = torch.device(device) if device is not None else torch.randn(1).device
        if dtype != torch.float16:
            raise RuntimeError(f"unsupported data type {dtype}")
        if device.type != "cuda":
            raise RuntimeError("GPUKernel is enabled. But the device is not CUDA.")
        self.n_heads, self.d_head, self.chunk_size = n_heads, d_head, chunk_size
        self.device = device
        self.max_chunks = max_chunks_for(memory_mb, chunk_size, n_heads, d_head, 2)
        elems = chunk_size * n_heads * d_head * self.max_chunks
        with torch.cuda.device(device):
            # one allocation, V pool right behind the K pool: the distance between a chunk's K and V
            # rows in memory is then the same in every process (it is worth a few percent of the
            # streaming rate, and two allocations leave it to the driver)
            pools = torch.empty(2 * elems, dtype=dtype, device=device)
            self.key_storage, self.value_storage = pools[:elems], pools[elems:]
            self.ctx = KernelContext(n_heads, d_head, chunk_size, self.key_storage.data_ptr(),
                                     self.value_storage.data_ptr(), self.max_chunks, tpp_threshold)
        self.tree = Tree(chunk_size, self.max_chunks, share_prefix)
        self._tables_version = 0

    def _stream(self) -> int:
        import torch
        return torch.cuda.current_stream(self.device).cuda_stream

    def _check_kv(self, t, rows: int, name: str):
        import torch
        if t.dtype != torch.float16 or t.device != self.device or tuple(t.shape) != (rows, self.n_heads, self.d_head):
            raise RuntimeError(f"{name} must be fp16 [{rows}, {self.n_heads}, {self.d_head}] on {self.device}")
        return t.contiguous()

    def add_seq(self, tokens: Sequence[int], k, v) -> int:
        k = self._check_kv(k, len(tokens), "k")
        v = self._check_kv(v, len(tokens), "v")
        idx, tok_begin, slots = self.tree.add_seq(tokens)
        if slots:
            self.ctx.scatter_kv(k.data_ptr(), v.data_ptr(), len(tokens), tok_begin, slots, self._stream())
        self.ctx.invalidate()
        return idx

    def remove_seq(self, seq_idx: int) -> None:
        self.tree.remove_seq(seq_idx)
        self.ctx.invalidate()

    def clear(self) -> None:
        self.tree.clear()
        self.ctx.invalidate()

    def reserve(self) -> int:
        seqs, slots = self.tree.reserve_tails()
        if seqs:
            # full last chunks got an empty successor and nothing else changed since the tables
            # were built: patch them; anything else is rebuilt from a tree walk at the next refresh
            if not (self.ctx.valid and self.ctx.roll_tails(seqs, slots, self._stream())):
                self.ctx.invalidate()
        return len(seqs)

    def refresh_kernel_context(self, force: bool = False) -> None:
        if force or not self.ctx.valid:
            self.ctx.refresh(self.tree.get_chunks(), self.tree.n_seqs, self._stream())

    def append_token(self, tokens: Sequence[int], k, v, fused: bool = True) -> int:
        if self.tree.n_seqs != len(tokens):
            raise RuntimeError("num of seqs is not equal to num of tokens")
        k = self._check_kv(k, len(tokens), "k")
        v = self._check_kv(v, len(tokens), "v")
        n_new = self.reserve()
        self.refresh_kernel_context()
        self.ctx.append_kv(k.data_ptr(), v.data_ptr(), len(tokens), self._stream())
        self.tree.append_token(tokens)  # reserve inside is a no-op now
        self.ctx.delta_tokens = self.ctx.delta_tokens + 1
        return n_new

    def decode_step(self, tokens: Sequence[int], q, k, v):
        """append_token(tokens, k, v) followed by forward(q) as one call (same results, bit for bit):
        the new K/V rows are written by the attention launch itself.  Returns the output."""
        import torch
        n = len(tokens)
        if self.tree.n_seqs != n:
            raise RuntimeError("num of seqs is not equal to num of tokens")
        k = self._check_kv(k, n, "k")
        v = self._check_kv(v, n, "v")
        q = self._check_kv(q, n, "q")
        self.reserve()
        self.refresh_kernel_context()
        out = torch.empty((n, self.n_heads, self.d_head), dtype=q.dtype, device=q.device)
        self.ctx.decode_step(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), n, self._stream())
        self.tree.append_token(tokens)  # reserve inside is a no-op now
        return out

    def append_token_rotary(self, tokens: Sequence[int], q, k, v, cos_sin_cache, is_neox: bool = True,
                            positions=None) -> int:
        """append_token with the rotary embedding of the new rows folded in: q is rotated in
        place, k is rotated on its way into the cache (k itself is left as it is), v is copied.
        Without `positions` (int64 [n_seqs] on the device) a sequence's position is its length."""
        import torch
        if self.tree.n_seqs != len(tokens):
            raise RuntimeError("num of seqs is not equal to num of tokens")
        n = len(tokens)
        k = self._check_kv(k, n, "k")
        v = self._check_kv(v, n, "v")
        if not q.is_contiguous() or q.dtype != torch.float16 or q.device != self.device or \
                tuple(q.shape) != (n, self.n_heads, self.d_head):
            raise RuntimeError(f"q must be contiguous fp16 [{n}, {self.n_heads}, {self.d_head}] on {self.device}")
        if cos_sin_cache.dtype != torch.float16 or cos_sin_cache.device != self.device or \
                cos_sin_cache.dim() != 2 or not cos_sin_cache.is_contiguous():
            raise RuntimeError("cos_sin_cache must be contiguous fp16 [max_position, rot_dim] on the cache's device")
        pos_ptr = 0
        if positions is not None:
            if positions.dtype != torch.int64 or positions.device != self.device or tuple(positions.shape) != (n,) \
                    or not positions.is_contiguous():
                raise RuntimeError(f"positions must be contiguous int64 [{n}] on {self.device}")
            pos_ptr = positions.data_ptr()
        n_new = self.reserve()
        self.refresh_kernel_context()
        self.ctx.rope_append_kv(pos_ptr, q.data_ptr(), k.data_ptr(), v.data_ptr(), cos_sin_cache.data_ptr(),
                                cos_sin_cache.shape[0], cos_sin_cache.shape[1], is_neox, n, self._stream())
        self.tree.append_token(tokens)
        self.ctx.delta_tokens = self.ctx.delta_tokens + 1
        return n_new

    def duplicate(self, seq_idx: int, copies: int) -> None:
        """Beam search: `copies` more sequences identical to seq_idx, right after it (reference
        attention.cpp:287-313); each owns a device copy of the tail chunk."""
        self.ctx.copy_chunks(self.tree.duplicate(seq_idx, copies), self._stream())
        self.ctx.invalidate()

    def append_completion(self, seq_idx: int, tokens: Sequence[int], k, v) -> int:
        """One beam-search step (reference attention.cpp:227-261): candidate 0 continues seq_idx
        with tokens[0] and row 0 of k/v, candidates 1.. become sequences seq_idx+1.. ."""
        n = len(tokens)
        if n < 1:
            return seq_idx
        k = self._check_kv(k, n, "k")
        v = self._check_kv(v, n, "v")
        pairs, targets = self.tree.append_completion(seq_idx, tokens)
        self.ctx.copy_chunks_put_rows(pairs, k.data_ptr(), v.data_ptr(), targets, self._stream())
        self.ctx.invalidate()
        return seq_idx

    def forward(self, q, partition: int = 0):
        import torch
        if not q.is_contiguous():
            raise RuntimeError("q is not contiguous")
        if q.dtype != torch.float16 or q.device != self.device or q.dim() != 3 or \
                q.shape[1] != self.n_heads or q.shape[2] != self.d_head:
            raise RuntimeError(f"q must be fp16 [n_seqs, {self.n_heads}, {self.d_head}] on {self.device}")
        out = torch.empty((q.shape[0], self.n_heads, self.d_head), dtype=q.dtype, device=q.device)
        self.refresh_kernel_context()
        self.ctx.attention(q.data_ptr(), out.data_ptr(), q.shape[0], partition, self._stream())
        return out

    def get_chunks(self) -> np.ndarray:
        return self.tree.get_chunks()

    def pool_views(self):
        """(K, V) pool tensors viewed as [max_chunks, H, c, d]."""
        shape = (self.max_chunks, self.n_heads, self.chunk_size, self.d_head)
        return self.key_storage.view(shape), self.value_storage.view(shape)
