"""GPU parity of the RMS-norm operators (ca_rms_norm, ca_fused_add_rms_norm) through the C-ABI
and through the pybind `ops` module, against the numpy oracle (oracle/norm.py).

Tolerance: the kernels round where the reference's do (normalised value to fp16, product with
the weight in fp16); only the fp32 summation order and the hardware's reciprocal square root
differ, so results agree to one fp16 unit in the last place of either rounding (rtol 2e-3)."""
import numpy as np
import pytest
import torch

from chunk_attn import capi
from gpu_helpers import to_dev
from oracle.norm import fused_add_rms_norm, rms_norm

pytestmark = pytest.mark.gpu


def close(got: torch.Tensor, want: np.ndarray):
    np.testing.assert_allclose(got.float().cpu().numpy(), want.astype(np.float32), rtol=2e-3, atol=1e-6)


@pytest.mark.parametrize("n,hidden", [(1, 8), (7, 100), (33, 4096), (3, 8200), (5, 4099)])
def test_rms_norm(n, hidden):
    rng = np.random.default_rng(hidden + n)
    x = (rng.standard_normal((n, hidden)) * 2).astype(np.float16)
    w = (1 + 0.2 * rng.standard_normal(hidden)).astype(np.float16)
    tx, tw = to_dev(x), to_dev(w)
    out = torch.empty_like(tx)
    capi.rms_norm(out, tx, tw, 1e-6)
    close(out, rms_norm(x, w, 1e-6))
    assert np.array_equal(tx.cpu().numpy(), x)          # input untouched
    capi.rms_norm(tx, tx, tw, 1e-6)                     # in place is allowed
    close(tx, rms_norm(x, w, 1e-6))


@pytest.mark.parametrize("n,hidden", [(2, 16), (9, 4096), (4, 1001)])
def test_fused_add_rms_norm(n, hidden):
    rng = np.random.default_rng(hidden)
    x = rng.standard_normal((n, 3, hidden)).astype(np.float16)     # leading dims are flattened
    r = rng.standard_normal((n, 3, hidden)).astype(np.float16)
    w = (1 + 0.2 * rng.standard_normal(hidden)).astype(np.float16)
    tx, tr, tw = to_dev(x), to_dev(r), to_dev(w)
    capi.fused_add_rms_norm(tx, tr, tw, 1e-5)
    want_out, want_res = fused_add_rms_norm(x, r, w, 1e-5)
    assert np.array_equal(tr.cpu().numpy(), want_res)   # the sum is one exact fp32 add, rounded once
    close(tx, want_out)


def test_pybind_ops_and_errors():
    import chunk_attn
    rng = np.random.default_rng(3)
    x = rng.standard_normal((6, 512)).astype(np.float16)
    r = rng.standard_normal((6, 512)).astype(np.float16)
    w = np.ones(512, np.float16)
    tx, tr, tw = to_dev(x), to_dev(r), to_dev(w)
    out = torch.empty_like(tx)
    chunk_attn.ops.rms_norm(out, tx, tw, 1e-6)
    close(out, rms_norm(x, w, 1e-6))
    chunk_attn.ops.fused_add_rms_norm(tx, tr, tw, 1e-6)
    want_out, want_res = fused_add_rms_norm(x, r, w, 1e-6)
    close(tx, want_out)
    assert np.array_equal(tr.cpu().numpy(), want_res)
    with pytest.raises(RuntimeError):
        chunk_attn.ops.rms_norm(out, tx.float(), tw, 1e-6)
    with pytest.raises(RuntimeError):
        capi.rms_norm(out[:, :256], tx, tw, 1e-6)
    with pytest.raises(capi.ChunkAttnError, match="different buffers"):
        capi.fused_add_rms_norm(tx, tx, tw, 1e-6)
