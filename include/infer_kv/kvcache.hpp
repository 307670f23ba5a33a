// KVCachePool<T>: the C++ cache-pool API of the reference (include/kvcache.hpp:12-97,
// src/kvcache.cc:7-305) on paged storage.
//
// The reference class keeps one contiguous [len, heads, head_size] tensor per sequence and layer
// and re-allocates + copies when a sequence grows; it was never compiled (its .cc is in no build
// glob and does not type-check against its header).  This class keeps the public surface -
// KVCachePoolConfig, get_key_cache / get_value_cache (MLA: value aliases key), extend_sequence,
// free_sequence, prefetch_sequence, print_memory_stats, optimize_memory, std::runtime_error for an
// unknown sequence or layer - but a sequence is a list of fixed-size blocks of one pool
// [K|V][layer][block][token][head][head_size], so growing never copies, and what the getters return
// is a view (layer base pointer + block table) that the paged kernels consume directly.
// Locking is done once at the public boundary (the reference re-locks a non-recursive mutex when
// extend_sequence and prefetch_sequence call each other: src/kvcache.cc:74-79, 144-149).
#pragma once
#include <cstddef>
#include <cstdint>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "infer_kv/block_pool.hpp"

struct ihipStream_t;   // hipStream_t is a pointer to it (hip/hip_runtime_api.h); named here so that host code
                       // that only manages a pool does not need the HIP headers

namespace infer {

struct KVCachePoolConfig {
    size_t block_size;   // tokens per block
    size_t head_size;
    size_t num_heads;    // KV heads
    size_t num_layers;
    bool use_mla;        // one shared cache for K and V
    size_t num_blocks;   // capacity of the pool (not in the reference, which allocates per sequence)

    KVCachePoolConfig(size_t blk_size = 512, size_t h_size = 128, size_t n_heads = 32, size_t n_layers = 32,
                      bool mla = false, size_t n_blocks = 1024)
        : block_size(blk_size), head_size(h_size), num_heads(n_heads), num_layers(n_layers), use_mla(mla),
          num_blocks(n_blocks) {}
};

// What get_key_cache / get_value_cache hand out: the layer's cache and the sequence's blocks in it.
// The paged kernels take it as it is; a caller that wants the reference's dense [len, heads, head_size]
// tensor gets it with one infer_kv_gather_bf16 call on the view (block table copied to the device).
template <typename T>
struct PagedCacheView {
    T* base;                      // [num_blocks, block_size, num_heads, head_size] of this layer
    const int32_t* block_table;   // host pointer, `num_blocks_used` entries, valid until the sequence changes
    size_t num_blocks_used;
    size_t length;                // tokens
    size_t block_size, num_heads, head_size;
    size_t block_stride, token_stride;   // in elements
};

struct KVCachePoolStats {
    size_t total_allocated;    // bytes held by live sequences (all layers, K and V)
    size_t active_sequences;
    size_t max_sequence_len;
};

template <typename T>
class KVCachePool {
public:
    // The reference's constructor (include/kvcache.hpp:35, cudaStream_t there): the pool allocates its
    // own device storage for config.num_blocks blocks (hipMalloc, freed by the destructor) and throws
    // std::runtime_error when the device cannot provide it.
    explicit KVCachePool(const KVCachePoolConfig& config, ihipStream_t* stream = nullptr);
    // Borrows `storage` (device or host memory of storage_elements() elements): the form an engine
    // uses that owns the cache as one tensor sized from free memory.  `stream` is kept for interface
    // compatibility; nothing here launches work.
    KVCachePool(const KVCachePoolConfig& config, T* storage, void* stream = nullptr);
    ~KVCachePool();
    KVCachePool(const KVCachePool&) = delete;
    KVCachePool& operator=(const KVCachePool&) = delete;

    static size_t storage_elements(const KVCachePoolConfig& c) {
        return (c.use_mla ? 1 : 2) * c.num_layers * c.num_blocks * c.block_size * c.num_heads * c.head_size;
    }

    PagedCacheView<T> get_key_cache(size_t sequence_id, size_t layer_idx);
    PagedCacheView<T> get_value_cache(size_t sequence_id, size_t layer_idx);
    void extend_sequence(size_t sequence_id, size_t new_length);
    void free_sequence(size_t sequence_id);
    void prefetch_sequence(size_t sequence_id, size_t initial_length);
    void print_memory_stats() const;
    void optimize_memory();

    KVCachePoolStats stats() const;
    size_t free_blocks() const { return static_cast<size_t>(pool_.num_free()); }
    size_t allocated_length(size_t sequence_id) const;

private:
    struct Seq {
        std::vector<int32_t> blocks;
        size_t current_length = 0;
    };
    void grow_locked(Seq& s, size_t new_length);
    void shrink_locked(Seq& s, size_t keep_tokens);
    PagedCacheView<T> view_locked(size_t sequence_id, size_t layer_idx, bool value);
    size_t bytes_per_block() const;

    KVCachePoolConfig config_;
    T* storage_;
    bool owns_storage_ = false;
    void* stream_;
    BlockPool pool_;
    std::unordered_map<size_t, Seq> seqs_;
    size_t max_len_ = 0;
    mutable std::mutex mu_;
};

}  // namespace infer
