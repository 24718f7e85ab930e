"""CPU restatement of the reference prefix-tree chunk manager.

TEST INFRASTRUCTURE ONLY.  Nothing shipped may import this module: it exists so that
tests can compare the native manager (and the device tables derived from it) with an
independent, readable restatement of the reference algorithm.

Each function cites the reference file:line it follows (paths relative to the
reference checkout, cpp/chunk_attn/...).  Pure-Python loops: meant for small cases
and for the five benchmark trees (a few thousand chunks), not for timing.

Pinned by (see tests/test_oracle_tree.py):
  * the literal expectations of the reference's own tests
    (tests/test_chunk_attn_cpu.py:24-175 add, :177-215 append, :267-303 remove),
  * the hand-worked table example for the tree after those six inserts,
  * a brute-force model that recomputes sharing from the raw token lists,
  * for the beam-search operations (duplicate, append_completion), which the reference's own
    test suite skips: the list-of-token-lists model (every sequence's root-to-tail tokens), the
    tree invariants, and hand-worked trees.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple


@dataclass(eq=False)
class Chunk:
    """Tree node (chunk.h:9-65).  `slot` replaces the K/V tensor views: chunk i's K/V
    live at element offset slot*H*c*d of the two pool tensors (chunk_allocator.cpp:43-55)."""
    capacity: int
    slot: int = -1
    tokens: List[int] = field(default_factory=list)
    children: List["Chunk"] = field(default_factory=list)
    n_seqs: int = 1
    parent: Optional["Chunk"] = None

    @property
    def n_tokens(self) -> int:
        return len(self.tokens)

    def full(self) -> bool:  # chunk.h:22
        return len(self.tokens) == self.capacity

    def equal(self, ids: Sequence[int], start: int, end: int) -> bool:  # chunk.cpp:50-61
        n = end - start
        if self.n_tokens != n or end > len(ids):
            return False
        return all(self.tokens[i] == ids[start + i] for i in range(n))

    def append_tokens(self, ids: Sequence[int], start: int, end: int) -> None:  # chunk.cpp:83-91
        if end - start > self.capacity - self.n_tokens:
            raise RuntimeError("no enough space in Chunk")
        self.tokens.extend(ids[start:end])

    def add_child(self, child: "Chunk") -> "Chunk":  # chunk.cpp:109-113
        self.children.append(child)
        child.parent = self
        return child

    def clear(self) -> None:  # chunk.h:38-44
        self.tokens = []
        self.n_seqs = 1
        self.children = []
        self.parent = None


class ChunkAllocator:
    """Fixed-capacity slab (chunk_allocator.cpp:8-120).  Which free chunk is handed out is
    not part of the parity contract (the reference pops the lowest Chunk* address); this
    restatement and the native manager both hand out the lowest free slot id."""

    def __init__(self, max_chunks: int, chunk_size: int):
        self.max_chunks = max_chunks
        self.chunk_size = chunk_size
        self.chunks = [Chunk(capacity=chunk_size, slot=i) for i in range(max_chunks)]
        self.free = set(range(max_chunks))
        self.peak_chunks = 0

    @staticmethod
    def max_chunks_for(memory_mb: int, chunk_size: int, n_heads: int, d_head: int, elem_bytes: int) -> int:
        # chunk_allocator.cpp:32-35 (float arithmetic as the reference does it)
        import numpy as np
        total = np.float32(memory_mb) * np.float32(1024) * np.float32(1024)
        per_chunk = chunk_size * n_heads * d_head * elem_bytes * 2
        return int(np.floor(total / np.float32(per_chunk)))

    def allocate(self) -> Chunk:  # chunk_allocator.cpp:58-84
        if not self.free:
            raise RuntimeError("ChunkAllocator: capacity reached")
        slot = min(self.free)
        self.free.remove(slot)
        self.peak_chunks = max(self.peak_chunks, self.max_chunks - len(self.free))
        return self.chunks[slot]

    def release(self, chunk: Chunk) -> None:  # chunk_allocator.cpp:109-116
        if chunk.slot in self.free:
            raise RuntimeError("free is called, but chunk is in free list")
        chunk.clear()
        self.free.add(chunk.slot)


@dataclass
class ChunkRow:
    """One flattened-tree row (chunk_info.h:6-15) with the chunk pointer replaced by
    (slot, n_tokens)."""
    chunk: Chunk
    seq_begin: int
    seq_end: int

    def as_tuple(self) -> Tuple[int, int, int, int]:
        return (self.chunk.slot, self.chunk.n_tokens, self.seq_begin, self.seq_end)


@dataclass
class CopyJob:
    """K/V rows [tok_begin, tok_end) of an inserted sequence go to chunk `slot`, starting
    at row 0 of that chunk (chunk.cpp:63-72 via chunk_allocator.cpp:92-100)."""
    slot: int
    tok_begin: int
    tok_end: int


class PrefixTree:
    """Host side of GPT::Attention (attention.cpp), without tensors."""

    def __init__(self, chunk_size: int, max_chunks: int, share_prefix: bool = True):
        self.chunk_size = chunk_size
        self.share_prefix = share_prefix
        self.root = Chunk(capacity=0)  # attention.cpp:28-29
        self.root.n_seqs = 0
        self.tails: List[Chunk] = []
        self.alloc = ChunkAllocator(max_chunks, chunk_size)
        self.valid = False       # KernelContext::valid
        self.delta_tokens = 0    # KernelContext::delta_tokens

    # attention.cpp:141-193
    def add_seq(self, tokens: Sequence[int]) -> Tuple[int, List[CopyJob]]:
        seq_idx = 0
        total = len(tokens)
        prev = self.root
        start = 0
        if self.share_prefix:
            while start < total:
                prev.n_seqs += 1
                start += prev.n_tokens
                found = False
                for child in prev.children:
                    if child.children and child.equal(tokens, start, start + child.n_tokens):
                        prev = child
                        found = True
                        break
                    seq_idx += child.n_seqs
                if not found:
                    break
        else:
            prev.n_seqs += 1
        jobs: List[CopyJob] = []
        while start < total:
            end = min(start + self.chunk_size, total)
            child = self.alloc.allocate()
            child.append_tokens(tokens, start, end)
            jobs.append(CopyJob(child.slot, start, end))
            prev = prev.add_child(child)
            start += self.chunk_size
        if prev.full():  # attention.cpp:182-188
            prev = prev.add_child(self.alloc.allocate())
        self.tails.insert(seq_idx, prev)
        self.valid = False
        return seq_idx, jobs

    # attention.cpp:116-131
    def reserve(self) -> List[Chunk]:
        new_chunks = []
        for i, tail in enumerate(self.tails):
            if tail.full():
                child = self.alloc.allocate()
                new_chunks.append(child)
                self.tails[i] = tail.add_child(child)
        if new_chunks:
            self.valid = False
        return new_chunks

    # attention.cpp:80-114 (host bookkeeping only; K/V rows go through append_kv)
    def append_token(self, tokens: Sequence[int]) -> List[Chunk]:
        if len(self.tails) != len(tokens):
            raise RuntimeError("num of seqs is not equal to num of tokens")
        new_chunks = self.reserve()
        for i, tail in enumerate(self.tails):
            tail.append_tokens(tokens, i, i + 1)
        self.delta_tokens += 1
        return new_chunks

    # attention.cpp:263-278
    def remove_seq(self, seq_idx: int) -> None:
        node = self.tails[seq_idx]
        while node is not None:
            node.n_seqs -= 1
            parent = node.parent
            if node.n_seqs <= 0 and parent is not None:
                parent.children = [c for c in parent.children if c is not node]
                self.alloc.release(node)
            node = parent
        del self.tails[seq_idx]
        self.valid = False

    # attention.cpp:211-226
    def at(self, seq_idx: int) -> Chunk:
        if not 0 <= seq_idx < self.root.n_seqs:
            raise IndexError("no such sequence")
        chunk = self.root
        start = 0
        while chunk.children:
            for child in chunk.children:
                end = start + child.n_seqs
                if start <= seq_idx < end:
                    chunk = child
                    break
                start = end
        return chunk

    def _copy_of_tail(self, tail: Chunk) -> Chunk:
        """chunk_allocator.cpp:87-91 -> Chunk::deep_copy (chunk.cpp:93-107): tokens copied,
        n_seqs = 1; copying a chunk with children is refused."""
        if tail.children:
            raise RuntimeError("Copy a non tailing chunk is forbidden")
        copy = self.alloc.allocate()
        copy.tokens = list(tail.tokens)
        copy.n_seqs = 1
        return copy

    # attention.cpp:287-313.  Every node above the tail counts `copies` more sequences, and
    # `copies` deep copies of the tail go in right after it (Chunk::insert_child,
    # chunk.cpp:115-120).  The reference stops there, leaving tails() and the kernel context
    # stale; here the tail list gains the copies at seq_idx+1.. and the context is
    # invalidated.  Returns the (source slot, copy slot) pairs whose K/V must be copied.
    def duplicate(self, seq_idx: int, copies: int) -> List[Tuple[int, int]]:
        if copies < 1:
            return []
        tail = self.at(seq_idx)
        node = tail.parent
        while node is not None:
            node.n_seqs += copies
            node = node.parent
        distance = tail.parent.children.index(tail) + 1
        pairs = []
        for i in range(copies):
            copy = self._copy_of_tail(tail)
            tail.parent.children.insert(distance, copy)
            copy.parent = tail.parent
            distance += 1
            self.tails.insert(seq_idx + 1 + i, copy)
            pairs.append((tail.slot, copy.slot))
        self.valid = False
        return pairs

    # attention.cpp:227-261, one beam-search step: candidates 1.. are copies of the tail (taken
    # before candidate 0's token is appended) that continue with their own token and go in right
    # after it; then the tail takes tokens[0]; a chunk that fills up gets its empty child at once
    # ("make sure full chunks are not the tails").  The reference leaves the ancestors' n_seqs
    # and tails() untouched, which makes the tree inconsistent, and asserts that the tail is not
    # full; here the counts and the tail list follow, and a full tail first gets its empty child
    # (what reserve() would do for it).  Returns (copy pairs, [(slot, row) of each candidate's
    # K/V row]); candidate i is sequence seq_idx + i afterwards.
    def append_completion(self, seq_idx: int, tokens: Sequence[int]):
        n = len(tokens)
        if n < 1:
            return [], []
        chunk = self.at(seq_idx)
        need = (1 if chunk.full() else 0)
        fills = (0 if chunk.full() else chunk.n_tokens) + 1 == self.chunk_size
        need += (n - 1) * (2 if fills else 1) + (1 if fills else 0)
        if need > len(self.alloc.free):
            raise RuntimeError("ChunkAllocator: capacity reached")
        if chunk.full():
            chunk = chunk.add_child(self.alloc.allocate())
            self.tails[seq_idx] = chunk
        pairs, targets = [], [None] * n
        if n > 1:
            node = chunk.parent
            while node is not None:
                node.n_seqs += n - 1
                node = node.parent
            distance = chunk.parent.children.index(chunk) + 1
            for i in range(1, n):
                copy = self._copy_of_tail(chunk)
                pairs.append((chunk.slot, copy.slot))
                targets[i] = (copy.slot, copy.n_tokens)
                copy.append_tokens(tokens, i, i + 1)
                chunk.parent.children.insert(distance, copy)
                copy.parent = chunk.parent
                distance += 1
                tail = copy
                if copy.full():
                    tail = copy.add_child(self.alloc.allocate())
                self.tails.insert(seq_idx + i, tail)
        targets[0] = (chunk.slot, chunk.n_tokens)
        chunk.append_tokens(tokens, 0, 1)
        if chunk.full():
            self.tails[seq_idx] = chunk.add_child(self.alloc.allocate())
        self.valid = False
        return pairs, targets

    # attention.cpp:342-372: pre-order walk with an explicit stack, so the children of a
    # node are visited in REVERSE order; the root itself is not listed; empty chunks are.
    def get_chunks(self) -> List[ChunkRow]:
        rows: List[ChunkRow] = []
        stack: List[Tuple[int, Chunk]] = [(0, self.root)]
        while stack:
            seq_begin, chunk = stack.pop()
            seq_end = seq_begin + chunk.n_seqs
            start = seq_begin
            for child in chunk.children:
                stack.append((start, child))
                start += child.n_seqs
            if chunk is self.root:
                continue
            rows.append(ChunkRow(chunk, seq_begin, seq_end))
        return rows

    @property
    def n_seqs(self) -> int:
        return self.root.n_seqs

    # helpers for tests -----------------------------------------------------------------
    def structure(self, node: Optional[Chunk] = None):
        """Nested (n_seqs, tokens, [children...]) description of the tree."""
        node = node or self.root
        return (node.n_seqs, tuple(node.tokens), [self.structure(c) for c in node.children])

    def seq_tokens(self, seq_idx: int) -> List[int]:
        out: List[int] = []
        node = self.tails[seq_idx]
        parts = []
        while node is not None:
            parts.append(node.tokens)
            node = node.parent
        for p in reversed(parts):
            out.extend(p)
        return out


@dataclass
class RefTables:
    """Reference-form device tables (kernel_cuda.cu:1331-1445) with K/V pointers replaced
    by slot ids.  Cells of seq_chunk_map the reference leaves unwritten are -1 here."""
    n_chunks: int
    n_shared: int
    final_idx: List[int]           # per get_chunks row
    slots: List[int]               # indexed by final chunk id (replaces keys_values)
    begins: List[int]
    ends: List[int]
    offsets: List[int]
    partial_rows: int
    seq_n_tokens: List[int]
    max_seq_n_chunks: int
    seq_chunk_map: List[List[int]]


def build_ref_tables(rows: Sequence[Tuple[int, int, int, int]], n_seqs: int, chunk_size: int,
                     tpp_threshold: int = 1) -> RefTables:
    """rows: (slot, n_tokens, seq_begin, seq_end) in get_chunks order."""
    n_chunks = len(rows)
    # kernel_cuda.cu:1343-1349
    n_shared = sum(1 for (_, _, b, e) in rows if e - b > tpp_threshold)
    # kernel_cuda.cu:1351-1369
    begins, ends, offsets = [], [], []
    partial = 0
    for (_, _, b, e) in rows:
        n = e - b
        if n <= tpp_threshold:
            continue
        begins.append(b)
        ends.append(e)
        offsets.append(partial)
        partial += n
    # kernel_cuda.cu:1371-1381
    seq_n_tokens = [0] * n_seqs
    for (_, nt, b, e) in rows:
        for j in range(b, e):
            seq_n_tokens[j] += nt
    max_len = max(seq_n_tokens) if n_seqs > 0 else 0
    width = max_len // chunk_size + 1
    # kernel_cuda.cu:1383-1410
    slots = [-1] * n_chunks
    final_idx = []
    cmap = [[-1] * width for _ in range(n_seqs)]
    count = [0] * n_seqs
    s1, s2 = 0, n_shared
    for (slot, _, b, e) in rows:
        n = e - b
        if n <= tpp_threshold:
            fi = s2
            s2 += 1
        else:
            fi = s1
            s1 += 1
        final_idx.append(fi)
        slots[fi] = slot
        for j in range(b, e):
            cmap[j][count[j]] = fi
            count[j] += 1
    return RefTables(n_chunks, n_shared, final_idx, slots, begins, ends, offsets, partial,
                     seq_n_tokens, width, cmap)
