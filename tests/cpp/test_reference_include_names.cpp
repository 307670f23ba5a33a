// A translation unit written the way a user of the reference writes it: the reference's include names
// (include/operator.hpp, opregistry.hpp, opfactory.hpp, unifiedOp.hpp, kvcache.hpp) and the
// reference's KVCachePool constructor (config, stream) - include/kvcache.hpp:35.  It must compile
// against this tree unchanged; run, it exercises the host side (registry lookups, the owning pool).
#include "kvcache.hpp"
#include "operator.hpp"
#include "opfactory.hpp"
#include "opregistry.hpp"
#include "unifiedOp.hpp"

#include <hip/hip_bfloat16.h>
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <stdexcept>

#define REQUIRE(c) do { if (!(c)) { std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #c); return 1; } } while (0)

int main() {
    using T = hip_bfloat16;
    // operator API: nothing registered yet -> nullptr, as in the reference (opregistry.hpp:25-40)
    auto& reg = infer::OperatorRegistry::getInstance();
    REQUIRE((reg.getOperator<T, infer::KVAppendOperator>(infer::OperatorType::KV_APPEND, "KV_APPEND") == nullptr));
    infer::OperatorFactory::registerOperators<T>();
    auto app = infer::OperatorFactory::getKVAppendOperator<T>();
    auto att = infer::OperatorFactory::getPagedAttentionOperator<T>();
    REQUIRE(app && att);
    REQUIRE(app->type() == infer::OperatorType::KV_APPEND && app->name() == "KV_APPEND");
    REQUIRE(att->type() == infer::OperatorType::PAGED_ATTENTION);
    infer::Operator* base = app.get();       // really an Operator
    REQUIRE(base->name() == "KV_APPEND");
    bool threw = false;
    try {
        infer::OperatorFactory::registerOperators<float>();   // the macro instantiates bf16 only
    } catch (const std::runtime_error&) {
        threw = true;
    }
    REQUIRE(threw);
    infer::UnifiedOp<T> unified;
    (void)unified;

    // cache pool with the reference's constructor: the pool owns its storage
    hipStream_t stream = nullptr;
    infer::KVCachePoolConfig cfg(/*blk_size=*/256, /*h_size=*/128, /*n_heads=*/8, /*n_layers=*/2, /*mla=*/false);
    cfg.num_blocks = 8;
    int devices = 0;
    const bool have_gpu = hipGetDeviceCount(&devices) == hipSuccess && devices > 0;
    try {
        infer::KVCachePool<T> pool(cfg, stream);
        REQUIRE(have_gpu);
        pool.prefetch_sequence(7, 300);
        auto k = pool.get_key_cache(7, 1);
        auto v = pool.get_value_cache(7, 1);
        REQUIRE(k.base != nullptr && v.base != nullptr && k.base != v.base);
        REQUIRE(k.num_blocks_used == 2 && k.block_size == 256 && k.num_heads == 8 && k.head_size == 128);
        REQUIRE(hipMemset(k.base, 0, 16) == hipSuccess);        // device memory the pool allocated
        threw = false;
        try {
            pool.get_key_cache(8, 0);
        } catch (const std::runtime_error&) {                 // unknown sequence: src/kvcache.cc:38-41
            threw = true;
        }
        REQUIRE(threw);
        pool.free_sequence(7);
        REQUIRE(pool.free_blocks() == 8);
    } catch (const std::runtime_error& e) {
        REQUIRE(!have_gpu);                                     // without a device the allocation must throw, nothing else
        std::printf("no device: %s\n", e.what());
    }
    std::printf("ok\n");
    return 0;
}
