// Host-only test of infer::KVCachePool<T> (include/infer_kv/kvcache.hpp); built and run by
// tests/test_kvcache_pool_cpp.py.  Exits non-zero on the first failed check.
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <vector>

#include "infer_kv/kvcache.hpp"

#define CHECK(c) do { if (!(c)) { std::fprintf(stderr, "CHECK failed line %d: %s\n", __LINE__, #c); return 1; } } while (0)

int main() {
    using Pool = infer::KVCachePool<uint16_t>;
    infer::KVCachePoolConfig cfg(/*block_size=*/16, /*head_size=*/8, /*num_heads=*/2, /*num_layers=*/3, /*mla=*/false, /*num_blocks=*/10);
    std::vector<uint16_t> storage(Pool::storage_elements(cfg), 0);
    Pool pool(cfg, storage.data());
    CHECK(Pool::storage_elements(cfg) == 2u * 3 * 10 * 16 * 2 * 8);

    pool.prefetch_sequence(7, 20);                        // 2 blocks
    CHECK(pool.free_blocks() == 8 && pool.allocated_length(7) == 32);
    auto k = pool.get_key_cache(7, 1);
    auto v = pool.get_value_cache(7, 1);
    CHECK(k.length == 20 && k.num_blocks_used == 2 && k.block_table[0] == 0 && k.block_table[1] == 1);
    CHECK(k.token_stride == 16 && k.block_stride == 256);
    CHECK(k.base == storage.data() + (0 * 3 + 1) * (10 * 16 * 2 * 8));
    CHECK(v.base == storage.data() + (1 * 3 + 1) * (10 * 16 * 2 * 8));   // value cache is the second half

    pool.extend_sequence(7, 30);                          // fits: no new block
    CHECK(pool.free_blocks() == 8 && pool.get_key_cache(7, 0).length == 30);
    pool.extend_sequence(7, 33);                          // grows by one block, nothing is copied or moved
    CHECK(pool.free_blocks() == 7 && pool.get_key_cache(7, 0).block_table[2] == 2);
    pool.extend_sequence(9, 5);                           // unknown sequence is created
    CHECK(pool.free_blocks() == 6 && pool.stats().active_sequences == 2 && pool.stats().max_sequence_len == 33);
    CHECK(pool.stats().total_allocated == 4u * (2 * 3 * 16 * 2 * 8 * sizeof(uint16_t)));

    bool threw = false;
    try { pool.get_key_cache(123, 0); } catch (const std::runtime_error&) { threw = true; }
    CHECK(threw);
    threw = false;
    try { pool.get_value_cache(7, 3); } catch (const std::runtime_error&) { threw = true; }
    CHECK(threw);
    threw = false;
    try { pool.prefetch_sequence(11, 16 * 7); } catch (const std::runtime_error&) { threw = true; }   // 7 > 6 free
    CHECK(threw);

    // optimize_memory: shrink when more than 1.5x the live length is held and the slack exceeds a block
    pool.prefetch_sequence(20, 16 * 5);                   // 5 blocks
    pool.extend_sequence(20, 10);                         // live length drops to 10, 80 tokens still held
    CHECK(pool.allocated_length(20) == 80);
    pool.optimize_memory();                               // keeps ceil(12 / 16) = 1 block
    CHECK(pool.allocated_length(20) == 16 && pool.free_blocks() == 5);
    CHECK(pool.allocated_length(7) == 48);                // 48 <= 1.5 * 33: untouched

    pool.free_sequence(7);
    pool.free_sequence(7);                                // freeing twice is a no-op, as in the reference
    CHECK(pool.free_blocks() == 8 && pool.stats().active_sequences == 2);
    pool.print_memory_stats();

    infer::KVCachePoolConfig mla(16, 8, 2, 3, true, 4);
    std::vector<uint16_t> st2(Pool::storage_elements(mla), 0);
    Pool p2(mla, st2.data());
    p2.prefetch_sequence(1, 1);
    CHECK(p2.get_value_cache(1, 2).base == p2.get_key_cache(1, 2).base);   // MLA: value aliases key
    std::puts("ok");
    return 0;
}
