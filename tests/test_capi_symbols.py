"""The C-ABI library loads and exports every symbol include/chunk_attn_hip.h declares."""
import os
import re

from chunk_attn import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "chunk_attn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ca_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = capi.load()
    names = declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), f"{name} declared but not exported"
        assert name in capi.SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(capi.SIGNATURES) == names


def test_device_entry_points_fail_loudly_without_a_gpu():
    import ctypes
    import pytest
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(capi.ChunkAttnError) as e:
        capi.KernelContext(2, 128, 64, 0, 0, 0)
    assert "no HIP device" in str(e.value)
    h = ctypes.c_void_p()
    assert capi.load().ca_ctx_create(ctypes.byref(h), 0, 64, 64, None, None, 0, 1) == -1
    assert b"bad shape" in capi.load().ca_last_error()


def test_markers_switch_on_and_off():
    """Marker ranges are off by default; switching them on loads the roctx library at run time
    (an error that says so where the image has none), and host-only calls still work inside them."""
    import numpy as np
    try:
        capi.set_markers(True)
    except capi.ChunkAttnError as e:
        assert "marker library" in str(e)
        return
    try:
        tree = capi.Tree(2, 16)
        tree.add_seq([1, 2, 3])
        rows = tree.get_chunks()
        assert np.asarray(rows).shape[1] == 4
    finally:
        capi.set_markers(False)
