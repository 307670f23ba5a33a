// KVCachePool<T> on paged storage (see include/infer_kv/kvcache.hpp).
#include "infer_kv/kvcache.hpp"

#include <hip/hip_bfloat16.h>
#include <hip/hip_runtime_api.h>

#include <iostream>
#include <stdexcept>

namespace infer {

template <typename T>
KVCachePool<T>::KVCachePool(const KVCachePoolConfig& config, T* storage, void* stream)
    : config_(config), storage_(storage), stream_(stream),
      pool_(static_cast<int32_t>(config.num_blocks), static_cast<int32_t>(config.block_size)) {
    if (!storage) throw std::invalid_argument("KVCachePool: storage is null");
    if (config.head_size == 0 || config.num_heads == 0 || config.num_layers == 0)
        throw std::invalid_argument("KVCachePool: empty geometry");
}

template <typename T>
KVCachePool<T>::KVCachePool(const KVCachePoolConfig& config, ihipStream_t* stream)
    : config_(config), storage_(nullptr), owns_storage_(true), stream_(stream),
      pool_(static_cast<int32_t>(config.num_blocks), static_cast<int32_t>(config.block_size)) {
    if (config.head_size == 0 || config.num_heads == 0 || config.num_layers == 0)
        throw std::invalid_argument("KVCachePool: empty geometry");
    void* p = nullptr;
    const size_t bytes = storage_elements(config) * sizeof(T);
    const hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess || p == nullptr) {
        (void)hipGetLastError();
        throw std::runtime_error("KVCachePool: cannot allocate " + std::to_string(bytes) + " bytes of device memory: " +
                                 hipGetErrorString(e));
    }
    storage_ = static_cast<T*>(p);
}

template <typename T>
KVCachePool<T>::~KVCachePool() {
    if (owns_storage_ && storage_) (void)hipFree(storage_);
}

template <typename T>
size_t KVCachePool<T>::bytes_per_block() const {
    return (config_.use_mla ? 1 : 2) * config_.num_layers * config_.block_size * config_.num_heads * config_.head_size * sizeof(T);
}

template <typename T>
void KVCachePool<T>::grow_locked(Seq& s, size_t new_length) {
    const size_t need = (new_length + config_.block_size - 1) / config_.block_size;
    if (need > s.blocks.size() && need - s.blocks.size() > static_cast<size_t>(pool_.num_free()))
        throw std::runtime_error("KV cache pool exhausted: need " + std::to_string(need - s.blocks.size()) + " more blocks");
    while (s.blocks.size() < need) s.blocks.push_back(pool_.acquire_block());
    s.current_length = new_length;
    if (new_length > max_len_) max_len_ = new_length;
}

template <typename T>
void KVCachePool<T>::shrink_locked(Seq& s, size_t keep_tokens) {
    const size_t keep = (keep_tokens + config_.block_size - 1) / config_.block_size;
    while (s.blocks.size() > keep) {
        pool_.release_block(s.blocks.back());
        s.blocks.pop_back();
    }
}

template <typename T>
PagedCacheView<T> KVCachePool<T>::view_locked(size_t sequence_id, size_t layer_idx, bool value) {
    auto it = seqs_.find(sequence_id);
    if (it == seqs_.end()) throw std::runtime_error("Sequence ID not found: " + std::to_string(sequence_id));
    if (layer_idx >= config_.num_layers)
        throw std::runtime_error("Layer index out of bounds or cache not initialized: " + std::to_string(layer_idx));
    const size_t per_layer = config_.num_blocks * config_.block_size * config_.num_heads * config_.head_size;
    const size_t which = (value && !config_.use_mla) ? 1 : 0;
    PagedCacheView<T> v;
    v.base = storage_ + (which * config_.num_layers + layer_idx) * per_layer;
    v.block_table = it->second.blocks.data();
    v.num_blocks_used = it->second.blocks.size();
    v.length = it->second.current_length;
    v.block_size = config_.block_size;
    v.num_heads = config_.num_heads;
    v.head_size = config_.head_size;
    v.token_stride = config_.num_heads * config_.head_size;
    v.block_stride = config_.block_size * v.token_stride;
    return v;
}

template <typename T>
PagedCacheView<T> KVCachePool<T>::get_key_cache(size_t sequence_id, size_t layer_idx) {
    std::lock_guard<std::mutex> g(mu_);
    return view_locked(sequence_id, layer_idx, false);
}

template <typename T>
PagedCacheView<T> KVCachePool<T>::get_value_cache(size_t sequence_id, size_t layer_idx) {
    std::lock_guard<std::mutex> g(mu_);
    return view_locked(sequence_id, layer_idx, true);
}

template <typename T>
void KVCachePool<T>::extend_sequence(size_t sequence_id, size_t new_length) {
    std::lock_guard<std::mutex> g(mu_);
    const bool fresh = seqs_.find(sequence_id) == seqs_.end();
    Seq& s = seqs_[sequence_id];   // an unknown sequence is created, as in the reference
    if (new_length <= s.blocks.size() * config_.block_size) {
        s.current_length = new_length;
        if (new_length > max_len_) max_len_ = new_length;
        return;
    }
    try {
        grow_locked(s, new_length);
    } catch (...) {
        if (fresh) seqs_.erase(sequence_id);   // a failed creation leaves nothing behind
        throw;
    }
}

template <typename T>
void KVCachePool<T>::prefetch_sequence(size_t sequence_id, size_t initial_length) {
    std::lock_guard<std::mutex> g(mu_);
    const bool fresh = seqs_.find(sequence_id) == seqs_.end();
    Seq& s = seqs_[sequence_id];
    if (initial_length <= s.blocks.size() * config_.block_size) {
        if (initial_length > s.current_length) s.current_length = initial_length;
        if (initial_length > max_len_) max_len_ = initial_length;
        return;
    }
    try {
        grow_locked(s, initial_length);
    } catch (...) {
        if (fresh) seqs_.erase(sequence_id);
        throw;
    }
}

template <typename T>
void KVCachePool<T>::free_sequence(size_t sequence_id) {
    std::lock_guard<std::mutex> g(mu_);
    auto it = seqs_.find(sequence_id);
    if (it == seqs_.end()) return;
    shrink_locked(it->second, 0);
    seqs_.erase(it);
}

template <typename T>
void KVCachePool<T>::optimize_memory() {
    std::lock_guard<std::mutex> g(mu_);
    // the reference's rule (src/kvcache.cc:215-239): when more than 1.5x the live length is held
    // and the slack exceeds one block, keep 1.2x the live length
    for (auto& kv : seqs_) {
        Seq& s = kv.second;
        const size_t allocated = s.blocks.size() * config_.block_size;
        if (allocated > s.current_length * 1.5 && allocated - s.current_length > config_.block_size)
            shrink_locked(s, static_cast<size_t>(s.current_length * 1.2));
    }
}

template <typename T>
KVCachePoolStats KVCachePool<T>::stats() const {
    std::lock_guard<std::mutex> g(mu_);
    KVCachePoolStats st{0, seqs_.size(), max_len_};
    for (const auto& kv : seqs_) st.total_allocated += kv.second.blocks.size() * bytes_per_block();
    return st;
}

template <typename T>
size_t KVCachePool<T>::allocated_length(size_t sequence_id) const {
    std::lock_guard<std::mutex> g(mu_);
    auto it = seqs_.find(sequence_id);
    if (it == seqs_.end()) throw std::runtime_error("Sequence ID not found: " + std::to_string(sequence_id));
    return it->second.blocks.size() * config_.block_size;
}

template <typename T>
void KVCachePool<T>::print_memory_stats() const {
    const KVCachePoolStats st = stats();
    size_t total_len = 0;
    {
        std::lock_guard<std::mutex> g(mu_);
        for (const auto& kv : seqs_) total_len += kv.second.current_length;
    }
    std::cout << "KV Cache Pool Memory Stats:" << std::endl;
    std::cout << "  Total Allocated Memory: " << (st.total_allocated / (1024 * 1024)) << " MB" << std::endl;
    std::cout << "  Active Sequences: " << st.active_sequences << std::endl;
    std::cout << "  Max Sequence Length: " << st.max_sequence_len << std::endl;
    std::cout << "  Free Blocks: " << pool_.num_free() << " / " << pool_.num_blocks() << std::endl;
    if (st.active_sequences > 0)
        std::cout << "  Average Sequence Length: " << static_cast<double>(total_len) / st.active_sequences << " tokens" << std::endl;
}

template class KVCachePool<hip_bfloat16>;   // the reference instantiates bf16 only (src/kvcache.cc:305)
template class KVCachePool<uint16_t>;       // raw bf16 bit patterns, handy on the host

}  // namespace infer
