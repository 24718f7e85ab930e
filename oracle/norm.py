"""CPU restatement of the reference's RMS-norm operators.  TEST INFRASTRUCTURE ONLY: nothing on
the product path may import this module.

Follows cpp/chunk_attn/layernorm_kernels.cu:
  :23-47   rms_norm_kernel            out = fp16(x * rsqrt(mean(x^2) + eps)) * weight (fp16 product)
  :50-79   fused_add_rms_norm_kernel  residual = fp16(input + residual), mean over the unrounded
                                      fp32 sums, input = fp16(residual * rsqrt(...)) * weight
Pinned by tests/test_oracle_norm.py against the reference's other statement of the operator
(src/chunk_attn/models/llama_hf/layernorm.py:17-22, weight * (x * rsqrt(var + eps)).to(dtype))
in float64, by closed forms (constant rows, scale invariance, unit weights give unit RMS) and by
the fused form equalling add-then-norm.
"""
from __future__ import annotations

import numpy as np


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """x [..., hidden] fp16, weight [hidden] fp16 -> fp16."""
    xf = x.astype(np.float32)
    var = (xf * xf).sum(-1, keepdims=True, dtype=np.float32) / np.float32(x.shape[-1])
    inv = (np.float32(1.0) / np.sqrt(var + np.float32(eps))).astype(np.float32)
    return ((xf * inv).astype(np.float16) * weight.astype(np.float16)).astype(np.float16)


def fused_add_rms_norm(x: np.ndarray, residual: np.ndarray, weight: np.ndarray, eps: float):
    """Returns (new input, new residual), both fp16."""
    s = x.astype(np.float32) + residual.astype(np.float32)
    new_res = s.astype(np.float16)
    var = (s * s).sum(-1, keepdims=True, dtype=np.float32) / np.float32(x.shape[-1])
    inv = (np.float32(1.0) / np.sqrt(var + np.float32(eps))).astype(np.float32)
    out = ((new_res.astype(np.float32) * inv).astype(np.float16) * weight.astype(np.float16)).astype(np.float16)
    return out, new_res
