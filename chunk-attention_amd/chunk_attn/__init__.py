"""ChunkAttention decode path for MI355X.

`from chunk_attn import Attention` gives the pybind11/libtorch class with the reference
project's constructor and methods; `chunk_attn.capi` is the ctypes binding of the C-ABI
library underneath it.  Both need the native libraries built in-tree
(`python chunk-attention_amd/build.py`); there is no pure-Python or CPU fallback.
"""
import os as _os

_libdir = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "lib")
try:
    import torch as _torch  # noqa: F401  (loads libtorch before the extension module)
    from .lib.chunk_attn_c import Attention, Chunk, IntFuture, ops  # noqa: F401
except ImportError as _e:  # pragma: no cover
    raise ImportError(
        "chunk_attn: the native module is missing or does not load (%s). Build it with "
        "`python chunk-attention_amd/build.py`; the decode path has no fallback." % _e) from _e

__all__ = ["Attention", "Chunk", "IntFuture", "ops"]
