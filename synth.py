"""Synthetic decode-attention workloads: token ids that produce exactly the intended chunk
sharing, and seeded N(0, sigma) Q/K/V drawn from a counter-based generator (so any slice of
any tensor can be regenerated independently, on any machine).

Test and benchmark infrastructure (bench.py, tests/, the smoke run), not part of the package;
nothing here touches the GPU.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Tuple

import numpy as np

# stream ids of the generator, one per tensor family
STREAM_Q = 1
STREAM_K_SHARED = 2
STREAM_V_SHARED = 3
STREAM_K_GROUP = 20      # + group index
STREAM_V_GROUP = 60      # + group index
STREAM_K_UNIQUE = 1000   # + sequence index
STREAM_V_UNIQUE = 5000   # + sequence index
STREAM_K_APPEND = 10000  # + step
STREAM_V_APPEND = 20000  # + step


def _mix64(x: np.ndarray) -> np.ndarray:
    """splitmix64 finaliser on uint64 arrays."""
    x = (x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    x = (x ^ (x >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return x ^ (x >> np.uint64(31))


def normal(seed: int, stream: int, count: int, sigma: float = 1.0, offset: int = 0) -> np.ndarray:
    """`count` float32 draws of N(0, sigma) for counters offset .. offset+count-1 of
    (seed, stream): hash -> two uniforms -> Box-Muller."""
    with np.errstate(over="ignore"):
        key = _mix64(np.uint64(seed) * np.uint64(0x9E3779B97F4A7C15) + np.uint64(stream))
        ctr = np.arange(offset, offset + count, dtype=np.uint64)
        bits = _mix64(ctr * np.uint64(0xD1342543DE82EF95) + key)
    u1 = ((bits >> np.uint64(40)).astype(np.float64) + 0.5) / float(1 << 24)
    u2 = ((bits & np.uint64(0xFFFFFF)).astype(np.float64) + 0.5) / float(1 << 24)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (z * sigma).astype(np.float32)


def normal_fp16(seed: int, stream: int, shape: Tuple[int, ...], sigma: float = 1.0) -> np.ndarray:
    n = int(np.prod(shape))
    return normal(seed, stream, n, sigma).astype(np.float16).reshape(shape)


def _signed64(x: int) -> int:
    x &= (1 << 64) - 1
    return x - (1 << 64) if x >= (1 << 63) else x


def normal_fp16_torch(seed: int, stream: int, shape: Tuple[int, ...], sigma: float, device):
    """normal_fp16 evaluated on `device` with torch: the same counters, hash and Box-Muller
    transform (int64 arithmetic wraps like uint64; right shifts are made logical by masking),
    so that large workloads need not be drawn on the host.  The float64 log/cos of the device
    may differ from numpy's in the last place, which survives the rounding to fp16 for at most
    a handful of elements per tensor: use normal_fp16 where bit-identical values matter."""
    import torch

    def mix(x):
        x = (x ^ ((x >> 30) & ((1 << 34) - 1))) * _signed64(0xBF58476D1CE4E5B9)
        x = (x ^ ((x >> 27) & ((1 << 37) - 1))) * _signed64(0x94D049BB133111EB)
        return x ^ ((x >> 31) & ((1 << 33) - 1))

    n = int(np.prod(shape))
    with np.errstate(over="ignore"):
        key = int(_mix64(np.uint64(seed) * np.uint64(0x9E3779B97F4A7C15) + np.uint64(stream)))
    out = torch.empty(n, dtype=torch.float16, device=device)
    step = 1 << 24   # bounded temporaries
    for o in range(0, n, step):
        m = min(step, n - o)
        ctr = torch.arange(o, o + m, dtype=torch.int64, device=device)
        bits = mix(ctr * _signed64(0xD1342543DE82EF95) + _signed64(key))
        u1 = (((bits >> 40) & 0xFFFFFF).to(torch.float64) + 0.5) / float(1 << 24)
        u2 = ((bits & 0xFFFFFF).to(torch.float64) + 0.5) / float(1 << 24)
        z = torch.sqrt(-2.0 * torch.log(u1)) * torch.cos(2.0 * np.pi * u2)
        out[o:o + m] = (z * sigma).to(torch.float32).to(torch.float16)
    return out.reshape(shape)


@dataclass
class Segment:
    """A run of tokens of one sequence: ids plus the generator stream of its K and V."""
    ids: np.ndarray
    k_stream: int
    v_stream: int


@dataclass
class Workload:
    name: str
    n_heads: int
    d_head: int
    chunk_size: int
    sigma: float
    seqs: List[List[Segment]] = field(default_factory=list)
    append_steps: int = 0
    _cache: Dict[Tuple[int, int, int], np.ndarray] = field(default_factory=dict, repr=False)

    @property
    def n_seqs(self) -> int:
        return len(self.seqs)

    def tokens(self, s: int) -> List[int]:
        return np.concatenate([seg.ids for seg in self.seqs[s]]).astype(np.int64).tolist()

    def seq_len(self, s: int) -> int:
        return int(sum(len(seg.ids) for seg in self.seqs[s]))

    def kv(self, s: int, seed: int = 0) -> Tuple[np.ndarray, np.ndarray]:
        """K, V of sequence s as fp16 [T, H, d].  Shared segments regenerate the same values
        for every sequence that contains them."""
        def draw(stream: int, n: int) -> np.ndarray:
            if stream >= STREAM_K_UNIQUE:
                return normal_fp16(seed, stream, (n, self.n_heads, self.d_head), self.sigma)
            key = (seed, stream, n)  # shared segments are drawn once
            if key not in self._cache:
                self._cache[key] = normal_fp16(seed, stream, (n, self.n_heads, self.d_head), self.sigma)
            return self._cache[key]

        ks = [draw(seg.k_stream, len(seg.ids)) for seg in self.seqs[s]]
        vs = [draw(seg.v_stream, len(seg.ids)) for seg in self.seqs[s]]
        return np.concatenate(ks, axis=0), np.concatenate(vs, axis=0)

    def kv_torch(self, s: int, seed: int = 0, device="cuda:0"):
        """kv(s) drawn on the device (see normal_fp16_torch): fp16 torch tensors [T, H, d]."""
        import torch

        def draw(stream: int, n: int):
            if stream >= STREAM_K_UNIQUE:
                return normal_fp16_torch(seed, stream, (n, self.n_heads, self.d_head), self.sigma, device)
            key = ("torch", str(device), seed, stream, n)
            if key not in self._cache:
                self._cache[key] = normal_fp16_torch(seed, stream, (n, self.n_heads, self.d_head), self.sigma, device)
            return self._cache[key]

        ks = [draw(seg.k_stream, len(seg.ids)) for seg in self.seqs[s]]
        vs = [draw(seg.v_stream, len(seg.ids)) for seg in self.seqs[s]]
        return torch.cat(ks, dim=0), torch.cat(vs, dim=0)

    def q(self, seed: int = 0) -> np.ndarray:
        return normal_fp16(seed, STREAM_Q, (self.n_seqs, self.n_heads, self.d_head), self.sigma)

    def append_kv(self, step: int, seed: int = 0) -> Tuple[np.ndarray, np.ndarray]:
        shape = (self.n_seqs, self.n_heads, self.d_head)
        return (normal_fp16(seed, STREAM_K_APPEND + step, shape, self.sigma),
                normal_fp16(seed, STREAM_V_APPEND + step, shape, self.sigma))

    def append_tokens(self, step: int) -> List[int]:
        return [2_000_000_000 - step * 4096 - s for s in range(self.n_seqs)]

    # sizes -------------------------------------------------------------------------------
    def shared_tokens_physical(self) -> int:
        """Tokens stored once although several sequences attend them (whole chunks only)."""
        seen: Dict[int, int] = {}
        total = 0
        for s in range(self.n_seqs):
            pos = 0
            for seg in self.seqs[s]:
                if seg.k_stream < STREAM_K_UNIQUE and seg.k_stream not in seen:
                    seen[seg.k_stream] = 1
                    total += (len(seg.ids) // self.chunk_size) * self.chunk_size
                pos += len(seg.ids)
        return total

    def logical_tokens(self) -> int:
        return sum(self.seq_len(s) for s in range(self.n_seqs))


def _unique_ids(s: int, n: int) -> np.ndarray:
    return 1_000_000 * (s + 1) + np.arange(n, dtype=np.int64)


def prefix_workload(name: str, batch: int, chunk_size: int, shared: int, unique: int,
                    n_heads: int = 32, d_head: int = 128, sigma: float = 1.0) -> Workload:
    """`batch` sequences = one shared prefix of `shared` tokens + `unique` private tokens."""
    w = Workload(name, n_heads, d_head, chunk_size, sigma)
    for s in range(batch):
        segs = []
        if shared:
            segs.append(Segment(np.arange(shared, dtype=np.int64), STREAM_K_SHARED, STREAM_V_SHARED))
        if unique:
            segs.append(Segment(_unique_ids(s, unique), STREAM_K_UNIQUE + s, STREAM_V_UNIQUE + s))
        w.seqs.append(segs)
    return w


def two_level_workload(name: str, groups: int, per_group: int, chunk_size: int, root: int, mid: int,
                       unique: int, n_heads: int = 32, d_head: int = 128, sigma: float = 1.0,
                       append_steps: int = 32) -> Workload:
    """root prefix shared by all, a further prefix per group, then private tokens."""
    w = Workload(name, n_heads, d_head, chunk_size, sigma, append_steps=append_steps)
    for g in range(groups):
        for r in range(per_group):
            s = g * per_group + r
            segs = [Segment(np.arange(root, dtype=np.int64), STREAM_K_SHARED, STREAM_V_SHARED),
                    Segment(10_000 * (g + 1) + np.arange(mid, dtype=np.int64), STREAM_K_GROUP + g, STREAM_V_GROUP + g)]
            if unique:
                segs.append(Segment(_unique_ids(s, unique), STREAM_K_UNIQUE + s, STREAM_V_UNIQUE + s))
            w.seqs.append(segs)
    return w


def paged_variant(w: Workload) -> Workload:
    """Same K/V values, but every sequence's first token id is made distinct so that no
    chunk matches: the non-prefix-aware baseline in which each sequence owns private copies."""
    p = Workload(w.name + "-paged", w.n_heads, w.d_head, w.chunk_size, w.sigma, append_steps=w.append_steps)
    for s, segs in enumerate(w.seqs):
        new = []
        for i, seg in enumerate(segs):
            ids = seg.ids.copy()
            if i == 0 and len(ids):
                ids[0] = -(s + 1)
            new.append(Segment(ids, seg.k_stream, seg.v_stream))
        p.seqs.append(new)
    return p


def baseline_config(idx: int, fraction: float = 0.5, n_heads: int = 32) -> Workload:
    """The five benchmark configurations (0-based index).  `fraction` is the shared-prefix
    fraction of configuration 2 (the sharing sweep).  n_heads other than the configurations' 32
    gives the same workload with that many heads (its name says so): for measurements of what
    depends on the number of heads."""
    if n_heads != 32:
        w = baseline_config(idx, fraction)
        return Workload("%s-h%d" % (w.name, n_heads), n_heads, w.d_head, w.chunk_size, w.sigma, seqs=w.seqs,
                        append_steps=w.append_steps)
    if idx == 0:
        return prefix_workload("cfg1-b16-c32-1024+256", 16, 32, 1024, 256)
    if idx == 1:
        return prefix_workload("cfg2-b32-c64-2048+512", 32, 64, 2048, 512, sigma=0.5)
    if idx == 2:
        shared = int(round(4096 * fraction))
        return prefix_workload("cfg3-b64-c64-f%.2f" % fraction, 64, 64, shared, 4096 - shared)
    if idx == 3:
        return two_level_workload("cfg4-b64-c64-1024+512+128", 8, 8, 64, 1024, 512, 128)
    if idx == 4:
        return prefix_workload("cfg5-b256-c64-4096+256", 256, 64, 4096, 256)
    raise ValueError("configuration index must be 0..4")
