#include "attention.h"

#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPFunctions.h>

#include <iostream>
#include <stdexcept>

namespace GPT {

Attention::Attention(int n_heads, int d_head, int chunk_size, int memory_mb, bool share_prefix,
                     int tpp_threshold, torch::Dtype dtype, torch::Device device)
  : n_heads_(n_heads)
  , d_head_(d_head)
  , chunk_size_(chunk_size)
  , memory_mb_(memory_mb)
  , share_prefix_(share_prefix)
  , tpp_threshold_(tpp_threshold)
  , t_options_(torch::TensorOptions().dtype(dtype).layout(torch::kStrided).device(device).requires_grad(false)) {
    init();
}

Attention::Attention(Attention& other)
  : n_heads_(other.n_heads_)
  , d_head_(other.d_head_)
  , chunk_size_(other.chunk_size_)
  , memory_mb_(other.memory_mb_)
  , share_prefix_(other.share_prefix_)
  , tpp_threshold_(other.tpp_threshold_)
  , t_options_(other.t_options_) {
    init();
}

void Attention::init() {
    // the only kernels are HIP kernels: same check as the reference's GPU KernelContext
    if (!t_options_.device().is_cuda()) {
        throw std::runtime_error("GPUKernel is enabled. But the device is not CUDA.");
    }
    if (t_options_.dtype() != torch::kFloat16) {
        throw std::runtime_error("unsupported data type: the HIP kernels take float16 K/V/Q");
    }
    if (!t_options_.device().has_index()) {
        t_options_ = t_options_.device(torch::Device(torch::kCUDA, c10::hip::current_device()));
    }
    c10::DeviceGuard guard(t_options_.device());
    max_chunks_ = ChunkAllocator::max_chunks_for(memory_mb_, chunk_size_, n_heads_, d_head_, 2);
    const int64_t chunk_elems = int64_t(chunk_size_) * n_heads_ * d_head_;
    // One allocation, the V pool right behind the K pool: how far a chunk's V rows lie from its K
    // rows in memory decides a few percent of the streaming rate, and with two allocations that
    // distance is whatever the driver makes of them (the reference allocates the two pools
    // separately, chunk_allocator.cpp:43-55; the kernels only see the two base pointers).
    const int64_t pool_elems = chunk_elems * max_chunks_;
    torch::Tensor pools = torch::empty({ 2 * pool_elems }, t_options_);
    key_storage_ = pools.narrow(0, 0, pool_elems);
    value_storage_ = pools.narrow(0, pool_elems, pool_elems);
    tree_ = std::make_unique<PrefixTree>(chunk_size_, max_chunks_, share_prefix_, chunk_elems * 2 * 2);
    check(ca_ctx_create(&ctx_, n_heads_, d_head_, chunk_size_, key_storage_.data_ptr(),
                        value_storage_.data_ptr(), max_chunks_, tpp_threshold_));
}

Attention::~Attention() { ca_ctx_destroy(ctx_); }

void* Attention::stream() const {
    return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t_options_.device().index()).stream();
}

void Attention::check(int rc) const {
    if (rc != CA_OK) throw std::runtime_error(ca_last_error());
}

torch::Tensor Attention::checked_kv(const torch::Tensor& t, int64_t rows, const char* name) const {
    if (t.dim() != 3 || t.size(0) != rows || t.size(1) != n_heads_ || t.size(2) != d_head_) {
        throw std::runtime_error(std::string(name) + " must have shape [n, n_heads, d_head] with n = number of tokens");
    }
    if (t.scalar_type() != torch::kFloat16) throw std::runtime_error("unsupported data type");
    if (t.device() != t_options_.device()) throw std::runtime_error(std::string(name) + " is on a different device than the cache");
    return t.contiguous();
}

int Attention::add_seq(const std::vector<int>& tokens, torch::Tensor k, torch::Tensor v) {
    const int n = static_cast<int>(tokens.size());
    k = checked_kv(k, n, "k");
    v = checked_kv(v, n, "v");
    std::vector<CopyJob> jobs;
    const int seq_idx = tree_->add_seq(tokens, &jobs);
    if (!jobs.empty()) {
        c10::DeviceGuard guard(t_options_.device());
        std::vector<int32_t> slots;
        slots.reserve(jobs.size());
        for (const auto& j : jobs) slots.push_back(j.slot);
        check(ca_scatter_kv(ctx_, k.data_ptr(), v.data_ptr(), n, jobs.front().tok_begin, slots.data(),
                            static_cast<int>(slots.size()), stream()));
    }
    return seq_idx;
}

std::shared_ptr<std::future<int>> Attention::add_seq_async(const std::vector<int>&, torch::Tensor,
                                                           torch::Tensor) {
    // the reference's asynchronous insert is disabled the same way (attention.cpp:195-198 there)
    throw std::runtime_error("the implementation has bugs, still have problem in capturing torch tensors in lambda");
}

void Attention::remove_seq(int seq_idx) { tree_->remove_seq(seq_idx); }

void Attention::clear() { tree_->clear(); }

std::vector<Chunk*> Attention::reserve() { return reserve_and_note(); }

std::vector<Chunk*> Attention::reserve_and_note() {
    const uint64_t before = tree_->version();
    std::vector<int> seqs;
    std::vector<Chunk*> fresh = tree_->reserve(&seqs);
    if (fresh.empty()) return fresh;
    rolled_version_ = 0;
    if (ca_ctx_valid(ctx_) && tables_version_ == before) {
        // the only change since the tables were built: full last chunks got an empty successor
        rolled_seqs_.assign(seqs.begin(), seqs.end());
        rolled_slots_.clear();
        for (const Chunk* c : fresh) rolled_slots_.push_back(c->slot());
        rolled_version_ = tree_->version();
    }
    return fresh;
}

void Attention::refresh_kernel_context(bool force) {
    if (!force && ca_ctx_valid(ctx_) && tables_version_ == tree_->version()) return;
    c10::DeviceGuard guard(t_options_.device());
    if (!force && rolled_version_ != 0 && rolled_version_ == tree_->version() && ca_ctx_valid(ctx_)) {
        rolled_version_ = 0;
        const int rc = ca_ctx_roll_tails(ctx_, rolled_seqs_.data(), rolled_slots_.data(),
                                         static_cast<int>(rolled_seqs_.size()), stream());
        if (rc == CA_OK) {
            tables_version_ = tree_->version();
            return;
        }
        if (rc != CA_ERR_STATE) check(rc);  // CA_ERR_STATE: not patchable, tables untouched: rebuild
    }
    rolled_version_ = 0;
    const auto infos = tree_->get_chunks();
    std::vector<ca_chunk_row> rows(infos.size());
    for (size_t i = 0; i < infos.size(); i++) {
        rows[i] = { infos[i].chunk->slot(), infos[i].chunk->n_tokens(), infos[i].seq_idx_begin, infos[i].seq_idx_end };
    }
    check(ca_refresh_kernel_context(ctx_, rows.data(), static_cast<int>(rows.size()), tree_->n_seqs(), stream()));
    tables_version_ = tree_->version();
}

std::vector<Chunk*> Attention::append_token(const std::vector<int>& tokens, torch::Tensor k,
                                            torch::Tensor v, bool /*fused*/) {
    if (tree_->tails().size() != tokens.size()) {
        throw std::runtime_error("num of seqs is not equal to num of tokens");
    }
    const int n = static_cast<int>(tokens.size());
    k = checked_kv(k, n, "k");
    v = checked_kv(v, n, "v");
    std::vector<Chunk*> fresh = reserve_and_note();
    refresh_kernel_context();
    {
        c10::DeviceGuard guard(t_options_.device());
        check(ca_append_kv(ctx_, k.data_ptr(), v.data_ptr(), n, stream()));
    }
    tree_->append_token_ids(tokens);
    check(ca_ctx_set_delta_tokens(ctx_, ca_ctx_delta_tokens(ctx_) + 1));
    return fresh;
}

std::vector<Chunk*> Attention::append_token_rotary(const std::vector<int>& tokens, torch::Tensor q,
                                                   torch::Tensor k, torch::Tensor v,
                                                   torch::Tensor cos_sin_cache, bool is_neox,
                                                   c10::optional<torch::Tensor> positions) {
    if (tree_->tails().size() != tokens.size()) {
        throw std::runtime_error("num of seqs is not equal to num of tokens");
    }
    const int n = static_cast<int>(tokens.size());
    k = checked_kv(k, n, "k");
    v = checked_kv(v, n, "v");
    if (!q.is_contiguous() || q.scalar_type() != torch::kFloat16 || q.device() != t_options_.device() ||
        q.dim() != 3 || q.size(0) != n || q.size(1) != n_heads_ || q.size(2) != d_head_) {
        throw std::runtime_error("q must be contiguous float16 [n_seqs, n_heads, d_head] on the cache's device");
    }
    if (!cos_sin_cache.is_contiguous() || cos_sin_cache.scalar_type() != torch::kFloat16 ||
        cos_sin_cache.device() != t_options_.device() || cos_sin_cache.dim() != 2) {
        throw std::runtime_error("cos_sin_cache must be contiguous float16 [max_position, rot_dim] on the cache's device");
    }
    const int64_t* pos = nullptr;
    if (positions.has_value() && positions->defined()) {
        if (!positions->is_contiguous() || positions->scalar_type() != torch::kInt64 ||
            positions->device() != t_options_.device() || positions->numel() != n) {
            throw std::runtime_error("positions must be contiguous int64 [n_seqs] on the cache's device");
        }
        pos = positions->data_ptr<int64_t>();
    }
    std::vector<Chunk*> fresh = reserve_and_note();
    refresh_kernel_context();
    {
        c10::DeviceGuard guard(t_options_.device());
        check(ca_rope_append_kv(ctx_, pos, q.data_ptr(), k.data_ptr(), v.data_ptr(), cos_sin_cache.data_ptr(),
                                static_cast<int>(cos_sin_cache.size(0)), static_cast<int>(cos_sin_cache.size(1)),
                                is_neox ? 1 : 0, n, stream()));
    }
    tree_->append_token_ids(tokens);
    check(ca_ctx_set_delta_tokens(ctx_, ca_ctx_delta_tokens(ctx_) + 1));
    return fresh;
}

torch::Tensor Attention::decode_step(const std::vector<int>& tokens, torch::Tensor q, torch::Tensor k,
                                     torch::Tensor v) {
    if (tree_->tails().size() != tokens.size()) {
        throw std::runtime_error("num of seqs is not equal to num of tokens");
    }
    const int n = static_cast<int>(tokens.size());
    k = checked_kv(k, n, "k");
    v = checked_kv(v, n, "v");
    q = checked_kv(q, n, "q");
    reserve_and_note();
    refresh_kernel_context();
    c10::DeviceGuard guard(t_options_.device());
    torch::Tensor output = torch::empty({ q.size(0), n_heads_, d_head_ }, t_options_);
    check(ca_decode_step(ctx_, q.data_ptr(), k.data_ptr(), v.data_ptr(), output.data_ptr(), n, stream()));
    tree_->append_token_ids(tokens);
    return output;
}

torch::Tensor Attention::forward(torch::Tensor q, int partition) {
    if (!q.is_contiguous()) throw std::runtime_error("q is not contiguous");
    if (q.dim() != 3 || q.size(1) != n_heads_ || q.size(2) != d_head_) {
        throw std::runtime_error("q must have shape [n_seqs, n_heads, d_head]");
    }
    if (q.scalar_type() != torch::kFloat16) throw std::runtime_error("unsupported data type");
    if (q.device() != t_options_.device()) throw std::runtime_error("q is on a different device than the cache");
    c10::DeviceGuard guard(t_options_.device());
    torch::Tensor output = torch::empty({ q.size(0), n_heads_, d_head_ }, t_options_);
    refresh_kernel_context();
    check(ca_attention(ctx_, q.data_ptr(), output.data_ptr(), static_cast<int>(q.size(0)), partition, stream()));
    return output;
}

void Attention::duplicate(int seq_idx, int copies) {
    std::vector<std::pair<int, int>> pairs;
    tree_->duplicate(seq_idx, copies, &pairs);
    c10::DeviceGuard guard(t_options_.device());
    copy_chunks(pairs);
}

void Attention::copy_chunks(const std::vector<std::pair<int, int>>& pairs) {
    std::vector<int32_t> flat;
    flat.reserve(2 * pairs.size());
    for (const auto& [src, dst] : pairs) {
        flat.push_back(src);
        flat.push_back(dst);
    }
    check(ca_copy_chunks(ctx_, flat.data(), static_cast<int>(pairs.size()), stream()));
}

int Attention::append_completion(int seq_idx, std::vector<int>& tokens, torch::Tensor k, torch::Tensor v) {
    // beam search step (reference attention.cpp:227-261): candidate 0 continues the sequence,
    // candidates 1.. become copies of its tail inserted right after it, each with its own token
    const int n = static_cast<int>(tokens.size());
    if (n < 1) return seq_idx;
    if (seq_idx < 0 || seq_idx >= tree_->n_seqs()) throw std::out_of_range("no such sequence");
    k = checked_kv(k, n, "k");
    v = checked_kv(v, n, "v");
    std::vector<std::pair<int, int>> pairs;
    std::vector<PrefixTree::RowTarget> rows;
    tree_->append_completion(seq_idx, tokens, &pairs, &rows);
    c10::DeviceGuard guard(t_options_.device());
    // one launch: every candidate's copy of the tail, and row i of k/v as the new token of
    // sequence seq_idx + i
    std::vector<int32_t> flat, slot_row;
    for (const auto& [src, dst] : pairs) {
        flat.push_back(src);
        flat.push_back(dst);
    }
    for (const auto& r : rows) {
        slot_row.push_back(r.slot);
        slot_row.push_back(r.row);
    }
    check(ca_copy_chunks_put_rows(ctx_, flat.data(), static_cast<int>(pairs.size()), k.data_ptr(), v.data_ptr(), n,
                                  slot_row.data(), stream()));
    ca_ctx_invalidate(ctx_);  // sequence lengths changed under the device tables
    return seq_idx;
}

torch::Tensor Attention::key(const Chunk* chunk) {
    const int64_t chunk_elems = int64_t(chunk_size_) * n_heads_ * d_head_;
    return key_storage_.narrow(0, chunk_elems * chunk->slot(), chunk_elems).view({ n_heads_, chunk_size_, d_head_ });
}

torch::Tensor Attention::value(const Chunk* chunk) {
    const int64_t chunk_elems = int64_t(chunk_size_) * n_heads_ * d_head_;
    return value_storage_.narrow(0, chunk_elems * chunk->slot(), chunk_elems).view({ n_heads_, chunk_size_, d_head_ });
}

void Attention::print(Chunk* root, int level) {
    if (root == nullptr) root = tree_->root();
    std::cout << std::string(size_t(level) * 4, ' ') << root->to_string(true) << std::endl;
    for (Chunk* child : root->children) print(child, level + 1);
}

void rotary_embedding(torch::Tensor& positions, torch::Tensor& query, torch::Tensor& key, int head_size,
                      torch::Tensor& cos_sin_cache, bool is_neox) {
    TORCH_CHECK(query.is_cuda() && key.is_cuda() && cos_sin_cache.is_cuda() && positions.is_cuda(),
                "rotary_embedding: tensors must be on the GPU");
    TORCH_CHECK(query.scalar_type() == torch::kFloat16 && key.scalar_type() == torch::kFloat16 &&
                  cos_sin_cache.scalar_type() == torch::kFloat16,
                "rotary_embedding: float16 only");
    TORCH_CHECK(positions.scalar_type() == torch::kInt64 && positions.is_contiguous(),
                "rotary_embedding: positions must be contiguous int64");
    TORCH_CHECK(cos_sin_cache.dim() == 2 && cos_sin_cache.is_contiguous(), "rotary_embedding: cos_sin_cache must be [max_position, rot_dim]");
    TORCH_CHECK(query.dim() >= 2 && key.dim() >= 2 && query.stride(-1) == 1 && key.stride(-1) == 1,
                "rotary_embedding: rows must be contiguous");
    const int64_t n_tokens = query.numel() / query.size(-1);
    TORCH_CHECK(positions.numel() == n_tokens && key.numel() / key.size(-1) == n_tokens,
                "rotary_embedding: positions, query and key disagree on the number of tokens");
    TORCH_CHECK(query.size(-1) % head_size == 0 && key.size(-1) % head_size == 0,
                "rotary_embedding: row width is not a multiple of head_size");
    // as in the reference, tokens are query.stride(-2) elements apart (leading dims contiguous)
    c10::DeviceGuard guard(query.device());
    void* st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(query.device().index()).stream();
    const int rc = ca_rotary_embedding(positions.data_ptr<int64_t>(), query.data_ptr(), key.data_ptr(),
                                       cos_sin_cache.data_ptr(), n_tokens,
                                       static_cast<int>(query.size(-1) / head_size),
                                       static_cast<int>(key.size(-1) / head_size), head_size,
                                       static_cast<int>(cos_sin_cache.size(1)),
                                       static_cast<int>(cos_sin_cache.size(0)), query.stride(-2),
                                       key.stride(-2), is_neox ? 1 : 0, st);
    if (rc != 0) throw std::runtime_error(ca_last_error());
}

namespace {
void check_norm_tensor(const torch::Tensor& t, int64_t hidden, const char* what) {
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kFloat16 && t.is_contiguous(), what,
                ": contiguous float16 tensors on the GPU only");
    TORCH_CHECK(t.dim() >= 1 && t.size(-1) == hidden, what, ": rows must be as wide as the weight");
}
}  // namespace

void rms_norm(torch::Tensor& out, torch::Tensor& input, torch::Tensor& weight, float epsilon) {
    const int64_t hidden = weight.numel();
    check_norm_tensor(weight, hidden, "rms_norm");
    check_norm_tensor(input, hidden, "rms_norm");
    check_norm_tensor(out, hidden, "rms_norm");
    TORCH_CHECK(out.sizes() == input.sizes(), "rms_norm: out and input differ in shape");
    c10::DeviceGuard guard(input.device());
    void* st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(input.device().index()).stream();
    if (ca_rms_norm(out.data_ptr(), input.data_ptr(), weight.data_ptr(), epsilon, input.numel() / hidden,
                    static_cast<int>(hidden), st) != 0) {
        throw std::runtime_error(ca_last_error());
    }
}

void fused_add_rms_norm(torch::Tensor& input, torch::Tensor& residual, torch::Tensor& weight, float epsilon) {
    const int64_t hidden = weight.numel();
    check_norm_tensor(weight, hidden, "fused_add_rms_norm");
    check_norm_tensor(input, hidden, "fused_add_rms_norm");
    check_norm_tensor(residual, hidden, "fused_add_rms_norm");
    TORCH_CHECK(residual.sizes() == input.sizes(), "fused_add_rms_norm: input and residual differ in shape");
    c10::DeviceGuard guard(input.device());
    void* st = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(input.device().index()).stream();
    if (ca_fused_add_rms_norm(input.data_ptr(), residual.data_ptr(), weight.data_ptr(), epsilon,
                              input.numel() / hidden, static_cast<int>(hidden), st) != 0) {
        throw std::runtime_error(ca_last_error());
    }
}

}  // namespace GPT
