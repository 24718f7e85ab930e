"""A small attention-only language model over the prefix-tree KV caches: embedding, a stack of
pre-norm `LlamaChunkAttention` layers with residuals, final norm and output head.  It has the
call signature of the reference's `LlamaForCausalLM.forward(seqs, kv_caches, prefill)`
(src/chunk_attn/models/llama_hf/modeling_llama.py:288-299, 206-235) and exists to drive the
scheduler and the decode path end to end with seeded weights; it is not a trained model.
"""
from __future__ import annotations

import math
from typing import List

import torch
from torch import nn

from .. import capi
from ..llama_layer import LlamaChunkAttention
from .sequence import Sequence


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6, dtype=torch.float16, device="cuda"):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype, device=device))
        self.eps = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        x = x.contiguous()
        out = torch.empty_like(x)
        capi.rms_norm(out, x, self.weight.detach(), self.eps)
        return out


class AttentionOnlyLM(nn.Module):
    def __init__(self, vocab_size: int, hidden_size: int, num_heads: int, num_layers: int,
                 max_position_embeddings: int = 4096, chunk_size: int = 64, memory_mb: int = 256,
                 seed: int = 0, dtype=torch.float16, device="cuda"):
        super().__init__()
        self.vocab_size, self.hidden_size, self.num_heads = vocab_size, hidden_size, num_heads
        self.chunk_size, self.memory_mb, self.device = chunk_size, memory_mb, torch.device(device)
        self.embed_tokens = nn.Embedding(vocab_size, hidden_size, dtype=dtype, device=device)
        self.layers = nn.ModuleList([LlamaChunkAttention(hidden_size, num_heads, max_position_embeddings,
                                                         dtype=dtype, device=device) for _ in range(num_layers)])
        self.input_norms = nn.ModuleList([RMSNorm(hidden_size, dtype=dtype, device=device) for _ in range(num_layers)])
        self.norm = RMSNorm(hidden_size, dtype=dtype, device=device)
        self.lm_head = nn.Linear(hidden_size, vocab_size, bias=False, dtype=dtype, device=device)
        g = torch.Generator().manual_seed(seed)
        with torch.no_grad():
            self.embed_tokens.weight.copy_(torch.randn(vocab_size, hidden_size, generator=g))
            self.lm_head.weight.copy_(torch.randn(vocab_size, hidden_size, generator=g) / math.sqrt(hidden_size))
            for layer in self.layers:
                for p in (layer.q_proj, layer.k_proj, layer.v_proj, layer.o_proj):
                    p.weight.copy_(torch.randn(hidden_size, hidden_size, generator=g) / math.sqrt(hidden_size))

    def create_kv_caches(self) -> List[capi.Attention]:
        """One cache per layer, same configuration (reference modeling_llama.py:252-270)."""
        dev = self.device if self.device.index is not None else torch.device("cuda", torch.cuda.current_device())
        return [capi.Attention(n_heads=self.num_heads, d_head=self.hidden_size // self.num_heads,
                               chunk_size=self.chunk_size, memory_mb=self.memory_mb, share_prefix=True,
                               tpp_threshold=1, dtype=torch.float16, device=dev) for _ in self.layers]

    def logits(self, seqs: List[Sequence], kv_caches, prefill: bool) -> torch.Tensor:
        """[n_seqs, vocab] logits of every sequence's last position."""
        if prefill:
            lens = {len(s) for s in seqs}
            if len(lens) != 1:
                raise ValueError("prefill takes prompts of one length at a time")
            input_ids = [list(s.tokens) for s in seqs]
            position_ids = [list(range(len(s))) for s in seqs]
        else:
            input_ids = [[s[-1]] for s in seqs]
            position_ids = [[len(s) - 1] for s in seqs]
        dev = self.embed_tokens.weight.device
        ids = torch.tensor(input_ids, dtype=torch.long, device=dev)
        pos = torch.tensor(position_ids, dtype=torch.int64, device=dev)
        hidden = self.embed_tokens(ids)
        token_lists = [s.tokens for s in seqs]
        for i, layer in enumerate(self.layers):
            hidden = hidden + layer(self.input_norms[i](hidden), token_lists, pos, kv_caches[i], prefill)
            if prefill:
                for s, idx in zip(seqs, layer.last_indices):
                    s.index = idx
        return self.lm_head(self.norm(hidden[:, -1]))

    @torch.no_grad()
    def forward(self, seqs: List[Sequence], kv_caches, prefill: bool) -> List[int]:
        return torch.argmax(self.logits(seqs, kv_caches, prefill), dim=-1).tolist()
