// GPT::Attention: prefix-tree KV cache with decode attention on MI355X.
//
// Drop-in for the reference class of the same name (cpp/chunk_attn/attention.h:16-75 there):
// same constructor arguments, methods and error messages.  The tree lives in the torch-free
// PrefixTree; K/V live in two pool tensors indexed by chunk slot; all device work goes
// through the C-ABI of libchunkattn_hip.so (include/chunk_attn_hip.h).
#pragma once

#include <torch/torch.h>

#include <future>
#include <memory>
#include <vector>

#include "chunk_attn_hip.h"
#include "prefix_tree.h"

namespace GPT {

class Attention {
  public:
    Attention(int n_heads, int d_head, int chunk_size, int memory_mb = 2048,
              bool share_prefix = true, int tpp_threshold = 1,
              torch::Dtype dtype = torch::kFloat16,
              torch::Device device = torch::Device(torch::kCUDA));
    // same configuration, fresh (empty) cache: one cache per model layer
    Attention(Attention& other);
    ~Attention();
    void operator=(Attention const&) = delete;

    // k, v: [n_tokens, n_heads, d_head].  Returns the index the sequence was inserted at.
    int add_seq(const std::vector<int>& tokens, torch::Tensor k, torch::Tensor v);
    std::shared_ptr<std::future<int>> add_seq_async(const std::vector<int>& tokens,
                                                    torch::Tensor k, torch::Tensor v);
    void remove_seq(int seq_idx);
    // one token per sequence; k, v: [n_seqs, n_heads, d_head]
    std::vector<Chunk*> append_token(const std::vector<int>& tokens, torch::Tensor k,
                                     torch::Tensor v, bool fused = true);
    // append_token with the rotary embedding of the new rows folded into the same launch
    // (the reference's layer runs rotary_embedding, then append_token:
    // src/chunk_attn/models/llama_hf/modeling_llama.py:62,91-95).  q [n_seqs, n_heads, d_head] is
    // rotated in place; k is rotated on its way into the cache and itself left unchanged.
    // positions: int64 [n_seqs] on the device, or an undefined tensor = each sequence's length.
    std::vector<Chunk*> append_token_rotary(const std::vector<int>& tokens, torch::Tensor q,
                                            torch::Tensor k, torch::Tensor v,
                                            torch::Tensor cos_sin_cache, bool is_neox = true,
                                            c10::optional<torch::Tensor> positions = c10::nullopt);
    // One decode step: append_token(tokens, k, v) followed by forward(q), with the same results
    // bit for bit, as one call: the attention launch writes the new K/V rows itself (one launch
    // fewer per step).  q, k, v: [n_seqs, n_heads, d_head].  Returns the output.
    torch::Tensor decode_step(const std::vector<int>& tokens, torch::Tensor q, torch::Tensor k,
                              torch::Tensor v);
    void refresh_kernel_context(bool force = false);
    std::vector<Chunk*> reserve();
    void clear();
    int64_t peak_memory_allocated() const { return tree_->allocator().peak_memory_allocated(); }
    void duplicate(int seq_idx, int copies);
    int append_completion(int seq_idx, std::vector<int>& tokens, torch::Tensor k, torch::Tensor v);
    // q: [n_seqs, n_heads, d_head], contiguous.  partition 0: shared chunks chunk-first, the
    // rest per sequence; 1: all chunk-first; 2: all per sequence.
    torch::Tensor forward(torch::Tensor q, int partition = 0);

    Chunk* get_trie() { return tree_->root(); }
    std::vector<Chunk*> tails() { return tree_->tails(); }
    void print(Chunk* root = nullptr, int level = 0);
    std::vector<ChunkInfo> get_chunks() { return tree_->get_chunks(); }

    // K / V of one chunk as [n_heads, chunk_size, d_head] views of the pool
    torch::Tensor key(const Chunk* chunk);
    torch::Tensor value(const Chunk* chunk);

  private:
    void init();
    void* stream() const;
    void check(int rc) const;
    torch::Tensor checked_kv(const torch::Tensor& t, int64_t rows, const char* name) const;
    void copy_chunks(const std::vector<std::pair<int, int>>& pairs);  // (source slot, destination slot)

    int n_heads_, d_head_, chunk_size_, memory_mb_;
    bool share_prefix_;
    int tpp_threshold_;
    torch::TensorOptions t_options_;
    int max_chunks_ = 0;
    torch::Tensor key_storage_, value_storage_;
    std::unique_ptr<PrefixTree> tree_;
    ca_ctx* ctx_ = nullptr;
    uint64_t tables_version_ = 0;  // tree version the device tables were built from
    // reserve() on a tree the tables were current for: the chunks it added, so that the next
    // refresh patches the tables (ca_ctx_roll_tails) instead of rebuilding them from a tree walk
    std::vector<Chunk*> reserve_and_note();
    std::vector<int32_t> rolled_seqs_, rolled_slots_;
    uint64_t rolled_version_ = 0;  // tree version right after that reserve(); 0 = nothing noted
};

// In-place rotary embedding of fp16 query/key rows: the operator the reference exports as
// chunk_attn.ops.rotary_embedding (cpp/chunk_attn/pos_encoding_kernels.cu:94-139).
void rotary_embedding(torch::Tensor& positions, torch::Tensor& query, torch::Tensor& key, int head_size,
                      torch::Tensor& cos_sin_cache, bool is_neox);

// The reference's rms_norm / fused_add_rms_norm (cpp/chunk_attn/layernorm_kernels.cu:66-117), fp16.
void rms_norm(torch::Tensor& out, torch::Tensor& input, torch::Tensor& weight, float epsilon);
void fused_add_rms_norm(torch::Tensor& input, torch::Tensor& residual, torch::Tensor& weight, float epsilon);

}  // namespace GPT
