"""The caller of the decode path: one Llama attention layer over the prefix-tree KV cache.

Mirrors the reference's `LlamaChunkAttention`
(src/chunk_attn/models/llama_hf/modeling_llama.py:16-113) and its rotary module
(src/chunk_attn/models/llama_hf/rotary_embedding_vllm.py:43-147) with the same argument
meaning.  The projections are plain torch matmuls; what differs is the decode branch: the
rotary embedding of the new query/key rows and the KV append are one launch
(`Attention.append_token_rotary`) instead of a rotary launch followed by an append launch.
Weights are whatever the caller loads; tests use seeded random ones.
"""
from __future__ import annotations

import math
from typing import List, Sequence

import torch
from torch import nn

from . import capi


class RotaryEmbedding(nn.Module):
    """cos/sin cache [max_position, rotary_dim] (fp32 math, stored fp16) and the in-place operator."""

    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int = 10240,
                 base: float = 10000.0, is_neox_style: bool = True, device="cuda"):
        super().__init__()
        self.head_size, self.rotary_dim = head_size, rotary_dim
        self.max_position_embeddings, self.base, self.is_neox_style = max_position_embeddings, base, is_neox_style
        inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float, device=device) / rotary_dim))
        t = torch.arange(max_position_embeddings, dtype=torch.float, device=device)
        freqs = torch.einsum("i,j -> ij", t, inv_freq)
        cache = torch.cat((freqs.cos(), freqs.sin()), dim=-1).to(torch.float16)
        self.register_buffer("cos_sin_cache", cache.contiguous(), persistent=False)

    def forward(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor):
        capi.rotary_embedding(positions, query, key, self.head_size, self.cos_sin_cache, self.is_neox_style)
        return query, key


class LlamaChunkAttention(nn.Module):
    """q/k/v projections -> rotary -> (prefill: causal attention + add_seq | decode: append +
    chunk attention) -> output projection."""

    def __init__(self, hidden_size: int, num_heads: int, max_position_embeddings: int = 10240,
                 rope_base: float = 10000.0, dtype=torch.float16, device="cuda"):
        super().__init__()
        if hidden_size % num_heads:
            raise ValueError(f"hidden_size must be divisible by num_heads (got `hidden_size`: {hidden_size}"
                             f" and `num_heads`: {num_heads}).")
        self.hidden_size, self.num_heads, self.head_dim = hidden_size, num_heads, hidden_size // num_heads
        kw = dict(bias=False, dtype=dtype, device=device)
        self.q_proj = nn.Linear(hidden_size, hidden_size, **kw)
        self.k_proj = nn.Linear(hidden_size, hidden_size, **kw)
        self.v_proj = nn.Linear(hidden_size, hidden_size, **kw)
        self.o_proj = nn.Linear(hidden_size, hidden_size, **kw)
        self.rotary_emb = RotaryEmbedding(self.head_dim, self.head_dim, max_position_embeddings, rope_base,
                                          True, device)

    def forward(self, hidden_states: torch.Tensor, seqs: List[Sequence[int]], position_ids: torch.Tensor,
                kv_cache: capi.Attention, prefill: bool) -> torch.Tensor:
        """hidden_states [n_seqs, n_tokens, hidden]; seqs: each sequence's token ids so far (the
        new token last); position_ids int64 [n_seqs, n_tokens].  Prefill inserts the sequences
        into kv_cache (their cache indices are returned in self.last_indices); decode expects
        batch row i to be cache sequence i."""
        batch, n_tokens, d_hidden = hidden_states.shape
        q = self.q_proj(hidden_states)
        k = self.k_proj(hidden_states)
        v = self.v_proj(hidden_states)
        if prefill:
            q, k = self.rotary_emb(position_ids.contiguous(), q, k)
            shape = (batch, n_tokens, self.num_heads, self.head_dim)
            q4, k4, v4 = q.view(shape), k.view(shape), v.view(shape)
            # causal attention over the prompt (not the decode path: plain fp32 torch math)
            qh, kh, vh = (t.transpose(1, 2).float() for t in (q4, k4, v4))
            scores = qh @ kh.transpose(-1, -2) / math.sqrt(self.head_dim)
            future = torch.ones(n_tokens, n_tokens, dtype=torch.bool, device=scores.device).triu(1)
            attn = torch.softmax(scores.masked_fill(future, float("-inf")), dim=-1) @ vh
            attn_output = attn.transpose(1, 2).reshape(batch, n_tokens, d_hidden).to(hidden_states.dtype)
            self.last_indices = [kv_cache.add_seq(list(seqs[i]), k4[i].contiguous(), v4[i].contiguous())
                                 for i in range(batch)]
        else:
            assert n_tokens == 1
            shape = (batch, self.num_heads, self.head_dim)
            q3, k3, v3 = q.view(shape), k.view(shape), v.view(shape)
            kv_cache.append_token_rotary([s[-1] for s in seqs], q3, k3, v3, self.rotary_emb.cos_sin_cache,
                                         self.rotary_emb.is_neox_style, position_ids.reshape(batch).contiguous())
            attn_output = kv_cache.forward(q3).view(batch, 1, d_hidden)
        output = self.o_proj(attn_output)
        kv_cache.reserve()
        kv_cache.refresh_kernel_context(force=False)
        return output
