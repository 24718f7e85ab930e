"""CPU restatement of the reference's rotary position embedding.  TEST INFRASTRUCTURE ONLY:
nothing on the product path may import this module.

Follows
  cpp/chunk_attn/pos_encoding_kernels.cu:24-50   apply_rotary_embedding (pairing, arithmetic in
                                                 the tensor's own type: every product and the
                                                 sum round to fp16)
  cpp/chunk_attn/pos_encoding_kernels.cu:52-92   rotary_embedding_kernel (cache row = position,
                                                 cosines then sines, all query heads then all
                                                 key heads)
  src/chunk_attn/models/llama_hf/rotary_embedding_vllm.py:58-93   the cos/sin cache (fp32 math,
                                                 stored as fp16)

Pinned by tests/test_oracle_rotary.py against the reference's other, independent statement of
the same operator (x*cos + rotate(x)*sin, rotary_embedding_vllm.py:29-40,95-135), evaluated in
float64, and by what a rotation fixes: position 0 is the identity, pair norms are preserved, and
q_m . k_n depends on m - n only.
"""
from __future__ import annotations

import numpy as np


def cos_sin_cache(rot_dim: int, max_position: int, base: float = 10000.0) -> np.ndarray:
    """[max_position, rot_dim] fp16: cos(p * f_r) for r < rot_dim/2, then sin(p * f_r);
    f_r = base ** (-2r / rot_dim), computed in fp32 (rotary_embedding_vllm.py:58-93)."""
    exponent = np.arange(0, rot_dim, 2, dtype=np.float32) / np.float32(rot_dim)
    inv_freq = (np.float32(1.0) / np.power(np.float32(base), exponent)).astype(np.float32)
    t = np.arange(max_position, dtype=np.float32)
    freqs = np.einsum("i,j->ij", t, inv_freq).astype(np.float32)
    return np.concatenate([np.cos(freqs), np.sin(freqs)], axis=-1).astype(np.float16)


def _rotate_rows(rows: np.ndarray, cos: np.ndarray, sin: np.ndarray, rot_dim: int, is_neox: bool,
                 step_dtype) -> np.ndarray:
    """rows [..., n_heads, head_size]; cos, sin [..., 1, rot_dim/2] already gathered by position.
    step_dtype: the type every product and sum is rounded to (fp16 = the reference's kernel)."""
    out = rows.copy()
    embed = rot_dim // 2
    if is_neox:
        xi, yi = slice(0, embed), slice(embed, rot_dim)          # pos_encoding_kernels.cu:33-36
    else:
        xi, yi = slice(0, rot_dim, 2), slice(1, rot_dim, 2)      # pos_encoding_kernels.cu:40-43
    x = rows[..., xi].astype(step_dtype)
    y = rows[..., yi].astype(step_dtype)
    c = cos.astype(step_dtype)
    s = sin.astype(step_dtype)
    # x*cos - y*sin ; y*cos + x*sin   (pos_encoding_kernels.cu:46-49), one rounding per operation
    out[..., xi] = ((x * c).astype(step_dtype) - (y * s).astype(step_dtype)).astype(rows.dtype)
    out[..., yi] = ((y * c).astype(step_dtype) + (x * s).astype(step_dtype)).astype(rows.dtype)
    return out


def rotary_embedding(positions, query, key, head_size: int, cache: np.ndarray, is_neox: bool = True,
                     step_dtype=np.float16):
    """positions [n_tokens] ints; query [n_tokens, n_heads*head_size], key [n_tokens,
    n_kv_heads*head_size] fp16 (key may be None).  Returns rotated copies (the reference
    rotates in place)."""
    positions = np.asarray(positions, dtype=np.int64)
    rot_dim = cache.shape[1]
    embed = rot_dim // 2
    cs = cache[positions]                       # [n_tokens, rot_dim]
    cos = cs[:, None, :embed]
    sin = cs[:, None, embed:]
    outs = []
    for t in (query, key):
        if t is None:
            outs.append(None)
            continue
        n_tokens = t.shape[0]
        rows = np.asarray(t).reshape(n_tokens, -1, head_size)
        outs.append(_rotate_rows(rows, cos, sin, rot_dim, is_neox, step_dtype).reshape(np.asarray(t).shape))
    return outs[0], outs[1]
