#include "prefix_tree.h"

#include <algorithm>
#include <cmath>
#include <stdexcept>
#include <tuple>

namespace GPT {

// ---- Chunk ---------------------------------------------------------------------------------

// reference chunk.cpp:50-61
bool Chunk::equal(const std::vector<int>& ids, int start, int end) const {
    const int n = end - start;
    if (n_tokens() != n || end > static_cast<int>(ids.size())) return false;
    return std::equal(tokens.begin(), tokens.end(), ids.begin() + start);
}

// reference chunk.cpp:83-91
void Chunk::append_tokens(const std::vector<int>& ids, int start, int end) {
    if (end - start > capacity_ - n_tokens()) throw std::runtime_error("no enough space in Chunk");
    tokens.insert(tokens.end(), ids.begin() + start, ids.begin() + end);
}

// reference chunk.cpp:109-113
Chunk* Chunk::add_child(Chunk* child) {
    children.push_back(child);
    child->parent = this;
    return child;
}

// reference chunk.cpp:115-120
Chunk* Chunk::insert_child(int idx, Chunk* child) {
    children.insert(children.begin() + idx, child);
    child->parent = this;
    return child;
}

// reference chunk.h:38-44
void Chunk::clear() {
    tokens.clear();
    n_seqs = 1;
    children.clear();
    parent = nullptr;
}

// reference chunk.cpp:122-135: "<n_seqs>: [t0,t1,...]", long lists abbreviated when brief
std::string Chunk::to_string(bool brief) const {
    std::string s = std::to_string(n_seqs) + ": [";
    if (brief && tokens.size() > 3) {
        s += std::to_string(tokens.front()) + ",...," + std::to_string(tokens.back());
    } else {
        for (size_t i = 0; i < tokens.size(); i++) {
            if (i) s += ",";
            s += std::to_string(tokens[i]);
        }
    }
    return s + "]";
}

// ---- ChunkAllocator ------------------------------------------------------------------------

ChunkAllocator::ChunkAllocator(int max_chunks, int chunk_size, int64_t chunk_total_bytes)
  : nodes_(static_cast<size_t>(std::max(max_chunks, 0))), chunk_total_bytes_(chunk_total_bytes) {
    for (int i = 0; i < static_cast<int>(nodes_.size()); i++) {
        nodes_[i].capacity_ = chunk_size;
        nodes_[i].slot_ = i;
        nodes_[i].tokens.reserve(chunk_size);
        free_.insert(free_.end(), i);
    }
}

int ChunkAllocator::max_chunks_for(int memory_mb, int chunk_size, int n_heads, int d_head,
                                   int elem_bytes) {
    // float arithmetic on purpose: the reference computes
    // floor(float(memory_mb) * 1024 * 1024 / chunk_total_bytes)
    const int64_t chunk_total = int64_t(chunk_size) * n_heads * d_head * elem_bytes * 2;
    return static_cast<int>(std::floor(float(memory_mb) * 1024 * 1024 / chunk_total));
}

// reference chunk_allocator.cpp:58-84
Chunk* ChunkAllocator::allocate() {
    if (free_.empty()) throw std::runtime_error("ChunkAllocator: capacity reached");
    const int slot = *free_.begin();
    free_.erase(free_.begin());
    peak_bytes_ = std::max(peak_bytes_, int64_t(used_chunks()) * chunk_total_bytes_);
    return &nodes_[slot];
}

// reference chunk_allocator.cpp:109-116
void ChunkAllocator::free(Chunk* chunk) {
    if (free_.count(chunk->slot_)) {
        throw std::runtime_error("free is called, but chunk is in free list");
    }
    chunk->clear();
    free_.insert(chunk->slot_);
}

// ---- PrefixTree ----------------------------------------------------------------------------

PrefixTree::PrefixTree(int chunk_size, int max_chunks, bool share_prefix,
                       int64_t chunk_total_bytes)
  : chunk_size_(chunk_size)
  , share_prefix_(share_prefix)
  , alloc_(max_chunks, chunk_size, chunk_total_bytes) {
    root_.n_seqs = 0;  // reference attention.cpp:28-29: the root holds no tokens
}

int PrefixTree::add_seq(const std::vector<int>& tokens, std::vector<CopyJob>* jobs) {
    int seq_idx = 0;
    const int total = static_cast<int>(tokens.size());
    Chunk* prev = &root_;
    int start = 0;

    if (share_prefix_) {
        // walk down while a non-leaf child holds exactly the next tokens
        // (reference attention.cpp:152-171); leaves are private and never matched
        while (start < total) {
            prev->n_seqs += 1;
            start += prev->n_tokens();
            Chunk* match = nullptr;
            for (Chunk* child : prev->children) {
                if (!child->children.empty() &&
                    child->equal(tokens, start, start + child->n_tokens())) {
                    match = child;
                    break;
                }
                seq_idx += child->n_seqs;
            }
            if (match == nullptr) break;
            prev = match;
        }
    } else {
        prev->n_seqs += 1;  // reference attention.cpp:172-174
    }

    // unmatched suffix -> new chunks (reference attention.cpp:176-180)
    for (; start < total; start += chunk_size_) {
        const int end = std::min(start + chunk_size_, total);
        Chunk* child = alloc_.allocate();
        child->append_tokens(tokens, start, end);
        if (jobs) jobs->push_back({ child->slot_, start, end, 0 });
        prev = prev->add_child(child);
    }
    // a full chunk may be shared later, so a sequence always ends in a private,
    // non-full tail (reference attention.cpp:182-188)
    if (prev->full()) prev = prev->add_child(alloc_.allocate());

    tails_.insert(tails_.begin() + seq_idx, prev);
    version_++;
    return seq_idx;
}

void PrefixTree::remove_seq(int seq_idx) {
    if (seq_idx < 0 || seq_idx >= static_cast<int>(tails_.size())) {
        throw std::out_of_range("remove_seq: no such sequence");
    }
    Chunk* node = tails_[seq_idx];
    while (node != nullptr) {
        node->n_seqs -= 1;
        Chunk* parent = node->parent;
        if (node->n_seqs <= 0 && parent != nullptr) {
            auto& sib = parent->children;
            sib.erase(std::remove(sib.begin(), sib.end(), node), sib.end());
            alloc_.free(node);
        }
        node = parent;
    }
    tails_.erase(tails_.begin() + seq_idx);
    version_++;
}

void PrefixTree::clear() {
    while (!tails_.empty()) remove_seq(static_cast<int>(tails_.size()) - 1);
}

std::vector<Chunk*> PrefixTree::reserve(std::vector<int>* seq_idx) {
    std::vector<Chunk*> fresh;
    for (size_t i = 0; i < tails_.size(); i++) {
        Chunk*& tail = tails_[i];
        if (tail->full()) {
            Chunk* child = alloc_.allocate();
            fresh.push_back(child);
            if (seq_idx) seq_idx->push_back(static_cast<int>(i));
            tail = tail->add_child(child);
        }
    }
    if (!fresh.empty()) version_++;
    return fresh;
}

void PrefixTree::append_token_ids(const std::vector<int>& tokens) {
    if (tails_.size() != tokens.size()) {
        throw std::runtime_error("num of seqs is not equal to num of tokens");
    }
    for (size_t i = 0; i < tails_.size(); i++) {
        tails_[i]->append_tokens(tokens, static_cast<int>(i), static_cast<int>(i) + 1);
    }
}

std::vector<ChunkInfo> PrefixTree::get_chunks() const {
    std::vector<ChunkInfo> rows;
    rows.reserve(alloc_.used_chunks());
    std::vector<std::pair<int, const Chunk*>> stack;
    stack.emplace_back(0, &root_);
    while (!stack.empty()) {
        const auto [seq_begin, chunk] = stack.back();
        stack.pop_back();
        int start = seq_begin;
        for (const Chunk* child : chunk->children) {
            stack.emplace_back(start, child);
            start += child->n_seqs;
        }
        // empty chunks are listed too: they are the reserved landing place of the next
        // appended token.  The root is not a chunk.
        if (chunk == &root_) continue;
        rows.push_back({ const_cast<Chunk*>(chunk), seq_begin, seq_begin + chunk->n_seqs });
    }
    return rows;
}

Chunk* PrefixTree::at(int seq_idx) const {
    if (seq_idx < 0 || seq_idx >= root_.n_seqs) throw std::out_of_range("no such sequence");
    const Chunk* chunk = &root_;
    int start = 0;
    while (!chunk->children.empty()) {
        const Chunk* next = nullptr;
        for (const Chunk* child : chunk->children) {
            const int end = start + child->n_seqs;
            if (start <= seq_idx && seq_idx < end) {
                next = child;
                break;
            }
            start = end;
        }
        if (next == nullptr) throw std::logic_error("prefix tree: sequence counts inconsistent");
        chunk = next;
    }
    return const_cast<Chunk*>(chunk);
}

void PrefixTree::duplicate(int seq_idx, int copies, std::vector<std::pair<int, int>>* copy_slots) {
    if (copies < 1) return;
    Chunk* tail = at(seq_idx);
    if (tail->parent == nullptr) throw std::runtime_error("duplicate: empty tree");
    if (copies > alloc_.max_chunks() - alloc_.used_chunks()) {
        throw std::runtime_error("ChunkAllocator: capacity reached");  // before anything changes
    }
    for (Chunk* node = tail->parent; node != nullptr; node = node->parent) node->n_seqs += copies;
    auto& sib = tail->parent->children;
    int pos = static_cast<int>(std::find(sib.begin(), sib.end(), tail) - sib.begin()) + 1;
    for (int i = 0; i < copies; i++) {
        Chunk* copy = alloc_.allocate();
        copy->tokens = tail->tokens;  // reference chunk.cpp:93-107 (deep copy of a tail)
        copy->n_seqs = 1;
        tail->parent->insert_child(pos + i, copy);
        tails_.insert(tails_.begin() + seq_idx + 1 + i, copy);
        if (copy_slots) copy_slots->emplace_back(tail->slot_, copy->slot_);
    }
    version_++;
}

void PrefixTree::append_completion(int seq_idx, const std::vector<int>& tokens,
                                   std::vector<std::pair<int, int>>* copy_slots,
                                   std::vector<RowTarget>* targets) {
    const int n = static_cast<int>(tokens.size());
    if (seq_idx < 0 || seq_idx >= static_cast<int>(tails_.size())) {
        throw std::out_of_range("append_completion: no such sequence");
    }
    if (targets) targets->assign(n, RowTarget{ -1, -1 });
    if (n < 1) return;
    Chunk* chunk = tails_[seq_idx];
    // chunks this step takes, so that running out of them leaves the tree as it was
    const bool was_full = chunk->full();
    const bool fills = (was_full ? 0 : chunk->n_tokens()) + 1 == chunk_size_;  // this token fills the tail
    const int need = (was_full ? 1 : 0) + (n - 1) * (fills ? 2 : 1) + (fills ? 1 : 0);
    if (need > alloc_.max_chunks() - alloc_.used_chunks()) {
        throw std::runtime_error("ChunkAllocator: capacity reached");
    }
    if (was_full) {
        chunk = chunk->add_child(alloc_.allocate());
        tails_[seq_idx] = chunk;
    }
    if (n > 1) {
        for (Chunk* node = chunk->parent; node != nullptr; node = node->parent) node->n_seqs += n - 1;
        auto& sib = chunk->parent->children;
        int pos = static_cast<int>(std::find(sib.begin(), sib.end(), chunk) - sib.begin()) + 1;
        for (int i = 1; i < n; i++) {
            Chunk* copy = alloc_.allocate();
            copy->tokens = chunk->tokens;  // reference chunk.cpp:93-107 (deep copy of a tail)
            copy->n_seqs = 1;
            if (copy_slots) copy_slots->emplace_back(chunk->slot_, copy->slot_);
            if (targets) (*targets)[i] = RowTarget{ copy->slot_, copy->n_tokens() };
            copy->append_tokens(tokens, i, i + 1);
            chunk->parent->insert_child(pos++, copy);
            Chunk* tail = copy;
            if (copy->full()) tail = copy->add_child(alloc_.allocate());  // full chunks are not tails
            tails_.insert(tails_.begin() + seq_idx + i, tail);
        }
    }
    if (targets) (*targets)[0] = RowTarget{ chunk->slot_, chunk->n_tokens() };
    chunk->append_tokens(tokens, 0, 1);
    if (chunk->full()) tails_[seq_idx] = chunk->add_child(alloc_.allocate());
    version_++;
}

}  // namespace GPT
