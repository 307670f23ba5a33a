// Host-side block pool (see include/infer_kv/block_pool.hpp) and its C ABI.
#include "infer_kv/block_pool.hpp"

#include <cstring>
#include <stdexcept>
#include <string>

#include "infer_kv.h"

namespace infer {

// ------------------------------------------------------------------ XXH64
namespace {
constexpr uint64_t P1 = 11400714785074694791ULL;
constexpr uint64_t P2 = 14029467366897019727ULL;
constexpr uint64_t P3 = 1609587929392839161ULL;
constexpr uint64_t P4 = 9650029242287828579ULL;
constexpr uint64_t P5 = 2870177450012600261ULL;

inline uint64_t rotl(uint64_t x, int r) { return (x << r) | (x >> (64 - r)); }
inline uint64_t rd64(const uint8_t* p) { uint64_t v; std::memcpy(&v, p, 8); return v; }   // little-endian host
inline uint32_t rd32(const uint8_t* p) { uint32_t v; std::memcpy(&v, p, 4); return v; }
inline uint64_t round1(uint64_t acc, uint64_t in) { return rotl(acc + in * P2, 31) * P1; }
inline uint64_t merge(uint64_t h, uint64_t v) { return (h ^ round1(0, v)) * P1 + P4; }
}  // namespace

uint64_t xxh64(const void* data, size_t len, uint64_t seed) {
    const uint8_t* p = static_cast<const uint8_t*>(data);
    const uint8_t* const end = p + len;
    uint64_t h;
    if (len >= 32) {
        uint64_t v1 = seed + P1 + P2, v2 = seed + P2, v3 = seed, v4 = seed - P1;
        const uint8_t* const limit = end - 32;
        do {
            v1 = round1(v1, rd64(p));
            v2 = round1(v2, rd64(p + 8));
            v3 = round1(v3, rd64(p + 16));
            v4 = round1(v4, rd64(p + 24));
            p += 32;
        } while (p <= limit);
        h = rotl(v1, 1) + rotl(v2, 7) + rotl(v3, 12) + rotl(v4, 18);
        h = merge(h, v1);
        h = merge(h, v2);
        h = merge(h, v3);
        h = merge(h, v4);
    } else {
        h = seed + P5;
    }
    h += static_cast<uint64_t>(len);
    while (p + 8 <= end) {
        h ^= round1(0, rd64(p));
        h = rotl(h, 27) * P1 + P4;
        p += 8;
    }
    if (p + 4 <= end) {
        h ^= static_cast<uint64_t>(rd32(p)) * P1;
        h = rotl(h, 23) * P2 + P3;
        p += 4;
    }
    while (p < end) {
        h ^= static_cast<uint64_t>(*p) * P5;
        h = rotl(h, 11) * P1;
        ++p;
    }
    h ^= h >> 33;
    h *= P2;
    h ^= h >> 29;
    h *= P3;
    h ^= h >> 32;
    return h;
}

// ------------------------------------------------------------------ BlockPool

BlockPool::BlockPool(int32_t num_blocks, int32_t block_size) : num_blocks_(num_blocks), block_size_(block_size) {
    if (num_blocks <= 0 || block_size <= 0) throw std::invalid_argument("BlockPool: num_blocks and block_size must be positive");
    blocks_.resize(num_blocks);
    for (int32_t i = 0; i < num_blocks; ++i) {
        blocks_[i].free = false;
        push_free_back(i);
    }
}

void BlockPool::push_free_back(int32_t id) {
    Block& b = blocks_[id];
    b.prev = free_tail_;
    b.next = -1;
    if (free_tail_ >= 0) blocks_[free_tail_].next = id; else free_head_ = id;
    free_tail_ = id;
    b.free = true;
    ++free_count_;
}

void BlockPool::unlink_free(int32_t id) {
    Block& b = blocks_[id];
    if (b.prev >= 0) blocks_[b.prev].next = b.next; else free_head_ = b.next;
    if (b.next >= 0) blocks_[b.next].prev = b.prev; else free_tail_ = b.prev;
    b.prev = b.next = -1;
    b.free = false;
    --free_count_;
}

void BlockPool::take(int32_t id) {
    Block& b = blocks_[id];
    if (b.ref_count != 0 || !b.free) throw std::logic_error("BlockPool: block " + std::to_string(id) + " is not free");
    b.ref_count = 1;
    b.hashed = false;
    b.hash = 0;
    b.token_ids.clear();
    unlink_free(id);
}

void BlockPool::release(int32_t id) {
    Block& b = blocks_[id];
    if (b.ref_count != 0 || b.free) throw std::logic_error("BlockPool: block " + std::to_string(id) + " is still referenced");
    push_free_back(id);
}

int32_t BlockPool::num_free() const { std::lock_guard<std::mutex> g(mu_); return free_count_; }
int32_t BlockPool::num_used() const { std::lock_guard<std::mutex> g(mu_); return num_blocks_ - free_count_; }

uint64_t BlockPool::compute_hash(const int64_t* token_ids, size_t n, int64_t prefix_or_minus1, uint64_t prefix_hash) {
    // Stream = [8 bytes of the previous block's hash, little endian] ++ token ids as int64 LE.
    std::vector<uint8_t> buf;
    buf.reserve(8 + n * 8);
    if (prefix_or_minus1 != kNoHash) {
        uint8_t le[8];
        for (int i = 0; i < 8; ++i) le[i] = static_cast<uint8_t>(prefix_hash >> (8 * i));
        buf.insert(buf.end(), le, le + 8);
    }
    const uint8_t* t = reinterpret_cast<const uint8_t*>(token_ids);
    buf.insert(buf.end(), t, t + n * 8);
    return xxh64(buf.data(), buf.size(), 0);
}

bool BlockPool::can_allocate(int64_t num_tokens) const {
    std::lock_guard<std::mutex> g(mu_);
    const int64_t need = (num_tokens + block_size_ - 1) / block_size_;
    return free_count_ >= need;
}

int64_t BlockPool::allocate(const int64_t* token_ids, int64_t num_tokens, std::vector<int32_t>& table) {
    std::lock_guard<std::mutex> g(mu_);
    if (!table.empty()) throw std::logic_error("BlockPool::allocate: sequence already holds blocks");
    const int64_t nblocks = (num_tokens + block_size_ - 1) / block_size_;
    int64_t cached_tokens = 0;
    bool have_hash = false;   // hash of the previous block exists (h != -1 in the reference)
    uint64_t h = 0;
    bool miss = false;
    for (int64_t i = 0; i < nblocks; ++i) {
        const int64_t* blk_tokens = token_ids + i * block_size_;
        const int64_t n = (i + 1) * block_size_ <= num_tokens ? block_size_ : num_tokens - i * block_size_;
        const bool full = n == block_size_;
        if (full) {
            h = compute_hash(blk_tokens, static_cast<size_t>(n), have_hash ? 0 : kNoHash, h);
            have_hash = true;
        } else {
            have_hash = false;
        }
        int32_t id = -1;
        if (have_hash) {
            auto it = hash_to_block_.find(h);
            if (it != hash_to_block_.end()) id = it->second;
        }
        if (id == -1) {
            miss = true;
        } else {
            const std::vector<int64_t>& have = blocks_[id].token_ids;
            if (static_cast<int64_t>(have.size()) != n || std::memcmp(have.data(), blk_tokens, n * 8) != 0) miss = true;
        }
        if (miss) {
            if (free_head_ < 0) throw std::logic_error("BlockPool::allocate: out of blocks");
            id = free_head_;
            take(id);
        } else {
            cached_tokens += block_size_;
            if (!blocks_[id].free) ++blocks_[id].ref_count;
            else take(id);
        }
        if (have_hash) {
            blocks_[id].hashed = true;
            blocks_[id].hash = h;
            blocks_[id].token_ids.assign(blk_tokens, blk_tokens + n);
            hash_to_block_[h] = id;
        }
        table.push_back(id);
    }
    return cached_tokens;
}

void BlockPool::deallocate(std::vector<int32_t>& table) {
    std::lock_guard<std::mutex> g(mu_);
    for (auto it = table.rbegin(); it != table.rend(); ++it) {
        const int32_t id = *it;
        if (id < 0 || id >= num_blocks_) throw std::logic_error("BlockPool::deallocate: bad block id");
        Block& b = blocks_[id];
        if (b.ref_count <= 0) throw std::logic_error("BlockPool::deallocate: block not referenced");
        if (--b.ref_count == 0) release(id);
    }
    table.clear();
}

bool BlockPool::can_append(int64_t seq_len) const {
    std::lock_guard<std::mutex> g(mu_);
    return free_count_ >= (seq_len % block_size_ == 1 ? 1 : 0);
}

void BlockPool::may_append(const int64_t* token_ids, int64_t seq_len, std::vector<int32_t>& table) {
    const int64_t full = seq_len / block_size_;
    const bool seals = seq_len > 0 && seq_len % block_size_ == 0;
    may_append_block(seals ? token_ids + (full - 1) * block_size_ : nullptr, seq_len, table);
}

void BlockPool::may_append_block(const int64_t* blk_tokens, int64_t seq_len, std::vector<int32_t>& table) {
    std::lock_guard<std::mutex> g(mu_);
    if (table.empty()) throw std::logic_error("BlockPool::may_append: sequence holds no blocks");
    Block& last = blocks_[table.back()];
    const int64_t r = seq_len % block_size_;
    if (r == 1) {
        if (!last.hashed) throw std::logic_error("BlockPool::may_append: previous block was not sealed");
        if (free_head_ < 0) throw std::logic_error("BlockPool::may_append: out of blocks");
        const int32_t id = free_head_;
        take(id);
        table.push_back(id);
    } else if (r == 0) {
        if (last.hashed) throw std::logic_error("BlockPool::may_append: block sealed twice");
        if (!blk_tokens) throw std::logic_error("BlockPool::may_append: tokens of the block to seal are missing");
        const bool has_prev = table.size() > 1;
        const Block* prev = has_prev ? &blocks_[table[table.size() - 2]] : nullptr;
        // the reference passes the previous block's hash, or -1 when there is none (or it is unsealed)
        const bool prefix = has_prev && prev->hashed;
        const uint64_t h = compute_hash(blk_tokens, static_cast<size_t>(block_size_), prefix ? 0 : kNoHash,
                                        prefix ? prev->hash : 0);
        last.hashed = true;
        last.hash = h;
        last.token_ids.assign(blk_tokens, blk_tokens + block_size_);
        hash_to_block_[h] = table.back();
    } else {
        if (last.hashed) throw std::logic_error("BlockPool::may_append: appending into a sealed block");
    }
}

int32_t BlockPool::acquire_block() {
    std::lock_guard<std::mutex> g(mu_);
    if (free_head_ < 0) throw std::logic_error("BlockPool::acquire_block: out of blocks");
    const int32_t id = free_head_;
    take(id);
    return id;
}

void BlockPool::release_block(int32_t id) {
    std::lock_guard<std::mutex> g(mu_);
    if (id < 0 || id >= num_blocks_ || blocks_[id].ref_count <= 0) throw std::logic_error("BlockPool::release_block: block not held");
    if (--blocks_[id].ref_count == 0) release(id);
}

int32_t BlockPool::ref_count(int32_t id) const { std::lock_guard<std::mutex> g(mu_); return blocks_.at(id).ref_count; }
bool BlockPool::has_hash(int32_t id) const { std::lock_guard<std::mutex> g(mu_); return blocks_.at(id).hashed; }
uint64_t BlockPool::block_hash(int32_t id) const { std::lock_guard<std::mutex> g(mu_); return blocks_.at(id).hash; }

std::vector<int32_t> BlockPool::free_ids() const {
    std::lock_guard<std::mutex> g(mu_);
    std::vector<int32_t> out;
    for (int32_t i = free_head_; i >= 0; i = blocks_[i].next) out.push_back(i);
    return out;
}

}  // namespace infer

// ------------------------------------------------------------------ C ABI

struct infer_pool {
    infer::BlockPool pool;
    infer_pool(int32_t n, int32_t bs) : pool(n, bs) {}
};

namespace {
thread_local std::string g_last_error;
template <class F>
int64_t guarded(F&& f) {
    try {
        return f();
    } catch (const std::exception& e) {
        g_last_error = e.what();
        return INFER_KV_ESTATE;
    }
}
}  // namespace

extern "C" {

infer_pool* infer_pool_create(int32_t num_blocks, int32_t block_size) {
    try {
        return new infer_pool(num_blocks, block_size);
    } catch (const std::exception& e) {
        g_last_error = e.what();
        return nullptr;
    }
}

void infer_pool_destroy(infer_pool* p) { delete p; }

const char* infer_pool_last_error(void) { return g_last_error.c_str(); }

int32_t infer_pool_num_free(const infer_pool* p) { return p ? p->pool.num_free() : INFER_KV_EINVAL; }
int32_t infer_pool_num_used(const infer_pool* p) { return p ? p->pool.num_used() : INFER_KV_EINVAL; }

int infer_pool_can_allocate(const infer_pool* p, int64_t num_tokens) {
    if (!p || num_tokens < 0) return INFER_KV_EINVAL;
    return p->pool.can_allocate(num_tokens) ? 1 : 0;
}

int64_t infer_pool_allocate(infer_pool* p, const int64_t* token_ids, int64_t num_tokens, int32_t* table_out,
                            int64_t table_capacity) {
    if (!p || !token_ids || !table_out || num_tokens <= 0) return INFER_KV_EINVAL;
    const int64_t need = (num_tokens + p->pool.block_size() - 1) / p->pool.block_size();
    if (table_capacity < need) return INFER_KV_EINVAL;
    return guarded([&]() -> int64_t {
        std::vector<int32_t> table;
        const int64_t cached = p->pool.allocate(token_ids, num_tokens, table);
        for (size_t i = 0; i < table.size(); ++i) table_out[i] = table[i];
        return cached;
    });
}

int infer_pool_deallocate(infer_pool* p, const int32_t* table, int64_t num_blocks) {
    if (!p || (!table && num_blocks > 0) || num_blocks < 0) return INFER_KV_EINVAL;
    return (int)guarded([&]() -> int64_t {
        std::vector<int32_t> t(table, table + num_blocks);
        p->pool.deallocate(t);
        return 0;
    });
}

int infer_pool_can_append(const infer_pool* p, int64_t seq_len) {
    if (!p || seq_len < 0) return INFER_KV_EINVAL;
    return p->pool.can_append(seq_len) ? 1 : 0;
}

int64_t infer_pool_may_append(infer_pool* p, const int64_t* token_ids, int64_t seq_len, int32_t* table,
                              int64_t num_blocks, int64_t table_capacity) {
    if (!p || !token_ids || !table || seq_len <= 0 || num_blocks <= 0 || table_capacity < num_blocks) return INFER_KV_EINVAL;
    if (seq_len % p->pool.block_size() == 1 && table_capacity < num_blocks + 1) return INFER_KV_EINVAL;
    return guarded([&]() -> int64_t {
        std::vector<int32_t> t(table, table + num_blocks);
        p->pool.may_append(token_ids, seq_len, t);
        for (size_t i = 0; i < t.size(); ++i) table[i] = t[i];
        return static_cast<int64_t>(t.size());
    });
}

int64_t infer_pool_may_append_block(infer_pool* p, const int64_t* last_block_tokens, int64_t seq_len, int32_t* table,
                                    int64_t num_blocks, int64_t table_capacity) {
    if (!p || !table || seq_len <= 0 || num_blocks <= 0 || table_capacity < num_blocks) return INFER_KV_EINVAL;
    const int64_t r = seq_len % p->pool.block_size();
    if (r == 1 && table_capacity < num_blocks + 1) return INFER_KV_EINVAL;
    if (r == 0 && !last_block_tokens) return INFER_KV_EINVAL;
    return guarded([&]() -> int64_t {
        std::vector<int32_t> t(table, table + num_blocks);
        p->pool.may_append_block(last_block_tokens, seq_len, t);
        for (size_t i = 0; i < t.size(); ++i) table[i] = t[i];
        return static_cast<int64_t>(t.size());
    });
}

uint64_t infer_pool_hash(const int64_t* token_ids, int64_t n, int has_prefix, uint64_t prefix_hash) {
    if (!token_ids || n < 0) return 0;
    return infer::BlockPool::compute_hash(token_ids, (size_t)n, has_prefix ? 0 : infer::BlockPool::kNoHash, prefix_hash);
}

uint64_t infer_xxh64(const void* data, size_t len, uint64_t seed) { return infer::xxh64(data, len, seed); }

int32_t infer_pool_ref_count(const infer_pool* p, int32_t block_id) {
    if (!p || block_id < 0 || block_id >= p->pool.num_blocks()) return INFER_KV_EINVAL;
    return p->pool.ref_count(block_id);
}

int infer_pool_block_hash(const infer_pool* p, int32_t block_id, uint64_t* hash_out) {
    if (!p || block_id < 0 || block_id >= p->pool.num_blocks()) return INFER_KV_EINVAL;
    if (!p->pool.has_hash(block_id)) return 0;
    if (hash_out) *hash_out = p->pool.block_hash(block_id);
    return 1;
}

int64_t infer_pool_free_ids(const infer_pool* p, int32_t* out, int64_t capacity) {
    if (!p || (!out && capacity > 0)) return INFER_KV_EINVAL;
    const std::vector<int32_t> ids = p->pool.free_ids();
    for (size_t i = 0; i < ids.size() && (int64_t)i < capacity; ++i) out[i] = ids[i];
    return static_cast<int64_t>(ids.size());
}

}  // extern "C"
