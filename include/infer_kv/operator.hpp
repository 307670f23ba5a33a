// Operator registry for the KV-cache path, interface-compatible with the reference's C++ operator
// API: OperatorType / Operator (include/operator.hpp:16-46), OperatorRegistry and
// REGISTER_OPERATOR (include/opregistry.hpp:9-71), OperatorFactory (include/opfactory.hpp:16-76).
//
// In the reference that API is vestigial: Operator::forward(vector<Tensor>) is pure virtual and no
// subclass overrides it.  Here the two operators of this path really do: KVAppendOperator and
// PagedAttentionOperator run the HIP kernels of libinfer_kv.so through its C ABI.  The element
// type parameter is the HIP bf16 type (the reference instantiates its macro for __nv_bfloat16).
#pragma once
#include <memory>
#include <stdexcept>
#include <string>
#include <typeinfo>
#include <unordered_map>
#include <vector>

#include <hip/hip_bfloat16.h>
#include <torch/extension.h>

namespace infer {

enum class OperatorType {
    MATMUL,
    RELU,
    SOFTMAX,
    SILU,
    FLASHATTENTION,
    ADD_RMS_NORM,
    MUL,
    ADD,
    ROPE,
    EMBEDDING,
    // the two operators of the paged KV-cache path (not in the reference's enum)
    KV_APPEND,
    PAGED_ATTENTION,
};

enum class DataType { FLOAT32, FLOAT16, BFLOAT16 };

class Operator {
public:
    virtual ~Operator() = default;
    virtual std::vector<torch::Tensor> forward(const std::vector<torch::Tensor>& inputs) = 0;
    virtual OperatorType type() const = 0;
    virtual std::string name() const = 0;
};

class OperatorRegistry {
public:
    static OperatorRegistry& getInstance() {
        static OperatorRegistry instance;
        return instance;
    }
    OperatorRegistry(const OperatorRegistry&) = delete;
    OperatorRegistry& operator=(const OperatorRegistry&) = delete;

    void registerOperator(OperatorType type, const std::string& name, std::shared_ptr<Operator> op) {
        registry_[typeid(*op).name()][static_cast<int>(type)][name] = std::move(op);
    }

    // Returns nullptr when nothing is registered under (class, type, name), as the reference does.
    template <typename T, template <typename> class OpClass>
    std::shared_ptr<OpClass<T>> getOperator(OperatorType type, const std::string& name) {
        auto by_class = registry_.find(typeid(OpClass<T>).name());
        if (by_class == registry_.end()) return nullptr;
        auto by_type = by_class->second.find(static_cast<int>(type));
        if (by_type == by_class->second.end()) return nullptr;
        auto by_name = by_type->second.find(name);
        if (by_name == by_type->second.end()) return nullptr;
        return std::dynamic_pointer_cast<OpClass<T>>(by_name->second);
    }

    std::vector<std::string> listRegisteredOperators() const {
        std::vector<std::string> out;
        for (const auto& c : registry_)
            for (const auto& t : c.second)
                for (const auto& n : t.second) out.push_back(n.first);
        return out;
    }

private:
    OperatorRegistry() = default;
    std::unordered_map<std::string, std::unordered_map<int, std::unordered_map<std::string, std::shared_ptr<Operator>>>> registry_;
};

// forward({key, value, k_cache, v_cache, slot_mapping}) -> {}   (infer/ops/attention.py:38-45)
template <typename T>
class KVAppendOperator : public Operator {
public:
    std::vector<torch::Tensor> forward(const std::vector<torch::Tensor>& inputs) override;
    OperatorType type() const override { return OperatorType::KV_APPEND; }
    std::string name() const override { return "KV_APPEND"; }
};

// forward({q[B,Hq,D], k_cache, v_cache, block_table, context_lens}) -> {out[B,Hq,D]}
// (flash_attn_with_kvcache at infer/ops/attention.py:118-120).  The softmax scale is a member
// (defaults to head_dim^-0.5 when <= 0).
template <typename T>
class PagedAttentionOperator : public Operator {
public:
    explicit PagedAttentionOperator(double scale = 0.0) : scale_(scale) {}
    std::vector<torch::Tensor> forward(const std::vector<torch::Tensor>& inputs) override;
    OperatorType type() const override { return OperatorType::PAGED_ATTENTION; }
    std::string name() const override { return "PAGED_ATTENTION"; }
    void set_scale(double s) { scale_ = s; }

private:
    double scale_;
};

#define REGISTER_OPERATOR(type, name, classname, data_type)                                           \
    do {                                                                                              \
        if constexpr (std::is_same_v<data_type, hip_bfloat16>) {                                      \
            static bool _registered_##classname##_##name = []() {                                     \
                infer::OperatorRegistry::getInstance().registerOperator(                              \
                    type, #name, std::make_shared<classname<hip_bfloat16>>());                        \
                return true;                                                                          \
            }();                                                                                      \
            (void)_registered_##classname##_##name;                                                   \
        } else {                                                                                      \
            throw std::runtime_error("Unsupported data type for operator registration");             \
        }                                                                                             \
    } while (0)

class OperatorFactory {
public:
    template <typename T>
    static void registerOperators() {
        REGISTER_OPERATOR(OperatorType::KV_APPEND, KV_APPEND, KVAppendOperator, T);
        REGISTER_OPERATOR(OperatorType::PAGED_ATTENTION, PAGED_ATTENTION, PagedAttentionOperator, T);
    }
    template <typename T>
    static std::shared_ptr<KVAppendOperator<T>> getKVAppendOperator() {
        return OperatorRegistry::getInstance().getOperator<T, KVAppendOperator>(OperatorType::KV_APPEND, "KV_APPEND");
    }
    template <typename T>
    static std::shared_ptr<PagedAttentionOperator<T>> getPagedAttentionOperator() {
        return OperatorRegistry::getInstance().getOperator<T, PagedAttentionOperator>(OperatorType::PAGED_ATTENTION,
                                                                                      "PAGED_ATTENTION");
    }
};

// Facade in the style of the reference's UnifiedOp (include/unifiedOp.hpp:6-99): registers on
// construction, throws std::runtime_error("... operator not found") when a lookup fails.
template <typename T>
class UnifiedOp {
public:
    UnifiedOp() { OperatorFactory::registerOperators<T>(); }
    void store_kvcache(const torch::Tensor& key, const torch::Tensor& value, torch::Tensor& k_cache,
                       torch::Tensor& v_cache, const torch::Tensor& slot_mapping) {
        auto op = OperatorFactory::getKVAppendOperator<T>();
        if (!op) throw std::runtime_error("KVAppend operator not found");
        op->forward({key, value, k_cache, v_cache, slot_mapping});
    }
    torch::Tensor paged_attention(const torch::Tensor& q, const torch::Tensor& k_cache, const torch::Tensor& v_cache,
                                  const torch::Tensor& block_table, const torch::Tensor& context_lens, double scale) {
        auto op = OperatorFactory::getPagedAttentionOperator<T>();
        if (!op) throw std::runtime_error("PagedAttention operator not found");
        op->set_scale(scale);
        return op->forward({q, k_cache, v_cache, block_table, context_lens})[0];
    }
};

}  // namespace infer
