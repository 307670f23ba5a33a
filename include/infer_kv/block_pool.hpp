// Host-side block pool of the paged KV cache: which cache block belongs to which sequence,
// reference counts, and a prefix cache keyed by a chained 64-bit hash of each full block.
//
// Semantics follow the allocator the reference engine actually runs, the Python BlockManager
// (infer/engine/block_mannager.py:26-133): blocks are handed out from the FRONT of a FIFO of
// free ids and returned to its BACK; a full block is registered under
// xxh64(prefix_hash_le8 || token_ids as little-endian int64) (block_mannager.py:54-60); a
// sequence being allocated re-uses registered blocks for as long as its leading full blocks hit
// (hash found AND stored token ids equal), and after the first miss every later block is fresh
// (block_mannager.py:79-103).  A block whose reference count fell to zero keeps its hash and can
// be revived from the free list by a later hit (block_mannager.py:95-99).
//
// Pure host code, no GPU dependency; thread-safe through one internal mutex (the reference's
// C++ pool guards its state the same way: include/kvcache.hpp:93).
#pragma once
#include <cstddef>
#include <cstdint>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace infer {

// XXH64 of `len` bytes with the given seed (public algorithm of the xxHash project).
uint64_t xxh64(const void* data, size_t len, uint64_t seed = 0);

class BlockPool {
public:
    static constexpr int64_t kNoHash = -1;   // "this block has no hash" (partial block), as in the reference

    BlockPool(int32_t num_blocks, int32_t block_size);

    int32_t num_blocks() const { return num_blocks_; }
    int32_t block_size() const { return block_size_; }
    int32_t num_free() const;
    int32_t num_used() const;

    // compute_hash (block_mannager.py:54-60).  `prefix` participates unless it is kNoHash.
    static uint64_t compute_hash(const int64_t* token_ids, size_t n, int64_t prefix_or_minus1, uint64_t prefix_hash);

    // can_allocate (block_mannager.py:76-77): enough free blocks for ceil(n / block_size).
    bool can_allocate(int64_t num_tokens) const;

    // allocate (block_mannager.py:79-103).  `table` must be empty; it receives one block id per
    // block of the sequence.  Returns the number of tokens whose KV is already cached.
    // Throws std::logic_error where the reference asserts.
    int64_t allocate(const int64_t* token_ids, int64_t num_tokens, std::vector<int32_t>& table);

    // deallocate (block_mannager.py:105-112): drops the references in reverse order and clears `table`.
    void deallocate(std::vector<int32_t>& table);

    // can_append (block_mannager.py:114-115): a new block is needed iff len % block_size == 1.
    bool can_append(int64_t seq_len) const;

    // may_append (block_mannager.py:117-133), called after the sequence grew to `seq_len` tokens:
    // opens a new block when the new token is the first of a block, seals (hashes and registers)
    // the last block when the new token filled it.
    void may_append(const int64_t* token_ids, int64_t seq_len, std::vector<int32_t>& table);
    // Same, for callers that keep only the tail of a long sequence at hand: `last_block_tokens` are the
    // block_size tokens of the block that seq_len just filled (read only when seq_len % block_size == 0).
    void may_append_block(const int64_t* last_block_tokens, int64_t seq_len, std::vector<int32_t>& table);

    // Raw allocation without token ids (no prefix sharing), for callers that only know lengths:
    // takes the block at the front of the free FIFO / drops one reference.
    int32_t acquire_block();
    void release_block(int32_t block_id);

    // introspection for tests and statistics
    int32_t ref_count(int32_t block_id) const;
    bool has_hash(int32_t block_id) const;
    uint64_t block_hash(int32_t block_id) const;
    std::vector<int32_t> free_ids() const;      // in FIFO order

private:
    struct Block {
        int32_t ref_count = 0;
        bool hashed = false;
        uint64_t hash = 0;
        std::vector<int64_t> token_ids;
        int32_t prev = -1, next = -1;   // links of the free FIFO
        bool free = true;
    };
    void push_free_back(int32_t id);
    void unlink_free(int32_t id);
    void take(int32_t id);      // _allocate_block
    void release(int32_t id);   // _deallocate_block

    int32_t num_blocks_, block_size_;
    std::vector<Block> blocks_;
    std::unordered_map<uint64_t, int32_t> hash_to_block_;
    int32_t free_head_ = -1, free_tail_ = -1, free_count_ = 0;
    mutable std::mutex mu_;
};

}  // namespace infer
