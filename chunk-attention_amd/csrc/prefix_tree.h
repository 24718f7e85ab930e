// Prefix-tree chunk manager: host-side bookkeeping of which KV chunks exist, which
// sequences share them and where each chunk's K/V live in the pool.  No tensors, no GPU
// calls: a chunk is identified by its pool slot (chunk i's K and V are the [H, c, d] blocks
// at element offset slot*H*c*d of the two pool buffers).
//
// Behaviour follows the reference manager (cpp/chunk_attn/attention.cpp, chunk.cpp,
// chunk_allocator.cpp); each method cites the lines it mirrors.
#pragma once

#include <cstdint>
#include <set>
#include <string>
#include <vector>

namespace GPT {

// Tree node (reference chunk.h:9-65).  Public members keep the reference's names because
// the Python binding exposes them.
class Chunk {
  public:
    std::vector<int> tokens;
    std::vector<Chunk*> children;  // non-owning; nodes are owned by ChunkAllocator
    int n_seqs = 1;
    Chunk* parent = nullptr;

    int capacity() const { return capacity_; }
    int n_tokens() const { return static_cast<int>(tokens.size()); }
    int slot() const { return slot_; }  // -1 for the root
    bool full() const { return n_tokens() == capacity_; }
    bool equal(const std::vector<int>& ids, int start, int end) const;
    void append_tokens(const std::vector<int>& ids, int start, int end);
    Chunk* add_child(Chunk* child);
    Chunk* insert_child(int idx, Chunk* child);
    void clear();
    std::string to_string(bool brief = false) const;

  private:
    friend class ChunkAllocator;
    friend class PrefixTree;
    int capacity_ = 0;
    int slot_ = -1;
};

// Flattened-tree row (reference chunk_info.h:6-15).
struct ChunkInfo {
    Chunk* chunk;
    int seq_idx_begin;
    int seq_idx_end;
};

// Fixed-capacity slab of chunk nodes (reference chunk_allocator.cpp:8-120).  The lowest
// free slot is handed out first.
class ChunkAllocator {
  public:
    ChunkAllocator(int max_chunks, int chunk_size, int64_t chunk_total_bytes);
    ChunkAllocator(const ChunkAllocator&) = delete;
    ChunkAllocator& operator=(const ChunkAllocator&) = delete;

    // reference chunk_allocator.cpp:32-35
    static int max_chunks_for(int memory_mb, int chunk_size, int n_heads, int d_head,
                              int elem_bytes);

    Chunk* allocate();
    void free(Chunk* chunk);
    bool full() const { return free_.empty(); }
    int max_chunks() const { return static_cast<int>(nodes_.size()); }
    int used_chunks() const { return max_chunks() - static_cast<int>(free_.size()); }
    int64_t peak_memory_allocated() const { return peak_bytes_; }

  private:
    std::vector<Chunk> nodes_;  // never resized: node addresses are stable
    std::set<int> free_;
    int64_t chunk_total_bytes_;
    int64_t peak_bytes_ = 0;
};

// "copy K/V rows [tok_begin, tok_end) of the inserted sequence into chunk `slot`, starting
// at row `dst_row`" -- what reference Chunk::append_tokens (chunk.cpp:63-72) does with
// tensor slices, recorded so that the caller can do all copies in one device pass.
struct CopyJob {
    int slot;
    int tok_begin;
    int tok_end;
    int dst_row;
};

class PrefixTree {
  public:
    PrefixTree(int chunk_size, int max_chunks, bool share_prefix, int64_t chunk_total_bytes);

    // reference attention.cpp:141-193.  Returns the index the sequence was inserted at.
    int add_seq(const std::vector<int>& tokens, std::vector<CopyJob>* jobs);
    // reference attention.cpp:263-278
    void remove_seq(int seq_idx);
    // every sequence, highest index first (reference attention.cpp:280-285 intends this)
    void clear();
    // reference attention.cpp:116-131.  seq_idx (optional): the index of the sequence each
    // returned chunk became the last chunk of
    std::vector<Chunk*> reserve(std::vector<int>* seq_idx = nullptr);
    // host half of reference attention.cpp:80-114: one token id per sequence.  Call
    // reserve() first; the K/V rows are written by the append kernel.
    void append_token_ids(const std::vector<int>& tokens);
    // reference attention.cpp:342-372 (pre-order, children visited last-to-first)
    std::vector<ChunkInfo> get_chunks() const;
    // reference attention.cpp:211-226
    Chunk* at(int seq_idx) const;
    // tree half of reference attention.cpp:287-313: `copies` more sequences identical to
    // seq_idx, inserted right after it.  Each new tail's K/V must be copied from the
    // source tail by the caller (src slot -> dst slot pairs are appended to `copy_slots`).
    void duplicate(int seq_idx, int copies, std::vector<std::pair<int, int>>* copy_slots);
    // tree half of reference attention.cpp:227-261, one beam-search step on sequence seq_idx:
    // candidate 0 continues the sequence with tokens[0]; candidates 1.. become copies of its tail,
    // inserted right after it, each continued with its own token; a tail that fills up gets its
    // empty child at once.  The caller copies K/V chunk src -> dst for every pair appended to
    // `copy_slots`, then writes candidate i's K/V row at (*targets)[i] (sequence seq_idx + i).
    // Differences from the reference, which leaves the tree inconsistent: the ancestors'
    // sequence counts and the tail list are updated, and a full tail (which the reference only
    // asserts against) first gets its empty child.
    struct RowTarget {
        int slot;
        int row;
    };
    void append_completion(int seq_idx, const std::vector<int>& tokens,
                           std::vector<std::pair<int, int>>* copy_slots, std::vector<RowTarget>* targets);

    Chunk* root() { return &root_; }
    const std::vector<Chunk*>& tails() const { return tails_; }
    int n_seqs() const { return root_.n_seqs; }
    int chunk_size() const { return chunk_size_; }
    ChunkAllocator& allocator() { return alloc_; }
    const ChunkAllocator& allocator() const { return alloc_; }
    // bumped by every change that alters the flattened tree (what the reference tracks as
    // KernelContext::valid = false)
    uint64_t version() const { return version_; }

  private:
    int chunk_size_;
    bool share_prefix_;
    Chunk root_;
    std::vector<Chunk*> tails_;
    ChunkAllocator alloc_;
    uint64_t version_ = 1;
};

}  // namespace GPT
