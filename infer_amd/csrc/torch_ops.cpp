// torch.ops._C.* registration of the KV-cache path and the operator-registry classes, over the C
// ABI of libinfer_kv.so.  Follows the schema convention of the reference's src/bindings.cpp:4-37:
// out-parameters marked `Tensor!`, every op returns (), implementations registered for the CUDA
// dispatch key (which is the key HIP tensors carry on PyTorch-ROCm).
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <mutex>
#include <unordered_map>

#include "infer_kv.h"
#include "infer_kv/operator.hpp"

namespace {

// PyTorch-ROCm presents HIP devices under the "cuda" device type, so the guard and stream
// accessors are the ones that carry that mapping.
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;
void* current_stream() { return static_cast<void*>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()); }

void check_rc(int rc, const char* what) { TORCH_CHECK(rc == 0, what, " failed: ", infer_kv_strerror(rc), " (code ", rc, ")"); }

void check_bf16_cuda(const at::Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor: the HIP kernels are the only implementation");
    TORCH_CHECK(t.scalar_type() == at::kBFloat16, name, " must be bfloat16");
}

// Split-KV workspace, one per (device, head shape), grown on demand and then reused so that
// steady-state steps and graph replays do not allocate.  A workspace that a larger batch outgrows
// stays alive for the life of the process: a HIP graph captured at the smaller batch still points
// at it, and its replays must keep writing to memory nobody else owns.  The buffer is shared by all
// calls for the shape, so those calls must be ordered on one stream (the partial results of one call
// are live until its merge kernel has run): a call that arrives on another stream while the last one is
// still busy is refused; callers that decode the same shape on several streams at once call
// infer_paged_decode_bf16 with a workspace per stream instead.
at::Tensor decode_workspace(const at::Tensor& like, int64_t batch, int64_t hq, int64_t hkv, int64_t d) {
    static std::mutex mu;
    static std::unordered_map<std::string, std::pair<int64_t, at::Tensor>> cache;
    static std::unordered_map<std::string, hipStream_t> last_stream;
    static std::vector<at::Tensor> retired;
    std::lock_guard<std::mutex> g(mu);
    const std::string key = std::to_string(like.get_device()) + ":" + std::to_string(hq) + ":" + std::to_string(hkv) + ":" + std::to_string(d);
    auto& slot = cache[key];
    if (!slot.second.defined() || slot.first < batch) {
        const int64_t cap = std::max<int64_t>(batch, slot.second.defined() ? 2 * slot.first : 64);
        const size_t bytes = infer_paged_decode_workspace_bytes(cap, hq, hkv, d);
        TORCH_CHECK(bytes > 0, "paged decode: unsupported shape (Hq=", hq, ", Hkv=", hkv, ", D=", d, ")");
        if (slot.second.defined()) retired.push_back(slot.second);
        slot = {cap, at::empty({static_cast<int64_t>(bytes)}, like.options().dtype(at::kByte))};
    }
    // a call on another stream while the last one still has work pending would overwrite partial results
    // in use: refused (checked on a change of stream only; streams under capture are not queried)
    const hipStream_t cur = static_cast<hipStream_t>(current_stream());
    auto it = last_stream.find(key);
    if (it != last_stream.end() && it->second != cur) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        const bool capturing = hipStreamIsCapturing(cur, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone;
        const bool busy = !capturing && hipStreamQuery(it->second) == hipErrorNotReady;
        (void)hipGetLastError();
        TORCH_CHECK(!busy, "paged decode: the shared workspace is still in use on another stream; order the calls on one "
                           "stream, or call infer_paged_decode_bf16 with a workspace per stream");
    }
    last_stream[key] = cur;
    return slot.second;
}

void store_kvcache(const at::Tensor& key, const at::Tensor& value, at::Tensor& k_cache, at::Tensor& v_cache,
                   const at::Tensor& slot_mapping) {
    check_bf16_cuda(key, "key"); check_bf16_cuda(value, "value");
    check_bf16_cuda(k_cache, "k_cache"); check_bf16_cuda(v_cache, "v_cache");
    TORCH_CHECK(key.dim() == 3 && value.sizes() == key.sizes(), "key/value must be [N, Hkv, D]");
    const int64_t n = key.size(0), d = key.size(1) * key.size(2);
    // the asserts of infer/ops/attention.py:41-44
    TORCH_CHECK(key.stride(2) == 1 && value.stride(2) == 1 && key.stride(1) == key.size(2) && value.stride(1) == key.size(2),
                "key/value rows must be contiguous");
    TORCH_CHECK(k_cache.stride(1) == d && v_cache.stride(1) == d, "cache token stride must be Hkv*D");
    TORCH_CHECK(slot_mapping.is_cuda() && slot_mapping.scalar_type() == at::kInt && slot_mapping.numel() == n &&
                slot_mapping.is_contiguous(), "slot_mapping must be a contiguous int32 GPU tensor of N entries");
    if (n == 0) return;
    DeviceGuard guard(key.device());
    check_rc(infer_kv_append_bf16(key.data_ptr(), key.stride(0), value.data_ptr(), value.stride(0), k_cache.data_ptr(),
                                  v_cache.data_ptr(), slot_mapping.data_ptr<int>(), n, d,
                                  k_cache.size(0) * k_cache.size(1), current_stream()),
             "store_kvcache");
}

void paged_attn_decode(const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache,
                       const at::Tensor& block_table, const at::Tensor& context_lens, double scale, at::Tensor& out) {
    check_bf16_cuda(q, "q"); check_bf16_cuda(k_cache, "k_cache"); check_bf16_cuda(v_cache, "v_cache"); check_bf16_cuda(out, "out");
    TORCH_CHECK(q.dim() == 3 && out.sizes() == q.sizes(), "q/out must be [B, Hq, D]");
    TORCH_CHECK(k_cache.dim() == 4 && k_cache.sizes() == v_cache.sizes() && k_cache.strides() == v_cache.strides(),
                "caches must be [nblk, bs, Hkv, D] with equal strides");
    const int64_t b = q.size(0), hq = q.size(1), d = q.size(2), hkv = k_cache.size(2);
    TORCH_CHECK(q.stride(2) == 1 && q.stride(1) == d && out.stride(2) == 1 && out.stride(1) == d, "q/out heads must be contiguous");
    TORCH_CHECK(k_cache.size(3) == d && k_cache.stride(3) == 1 && k_cache.stride(2) == d, "cache heads must be contiguous");
    TORCH_CHECK(block_table.is_cuda() && block_table.scalar_type() == at::kInt && block_table.dim() == 2 && block_table.size(0) == b && block_table.size(1) >= 1 && block_table.stride(1) == 1,
                "block_table must be int32 [B, MB] with MB >= 1");
    TORCH_CHECK(context_lens.is_cuda() && context_lens.scalar_type() == at::kInt && context_lens.numel() == b && context_lens.is_contiguous(),
                "context_lens must be int32 [B]");
    if (b == 0) return;
    DeviceGuard guard(q.device());
    at::Tensor ws = decode_workspace(q, b, hq, hkv, d);
    check_rc(infer_paged_decode_bf16(q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), k_cache.stride(0),
                                     k_cache.stride(1), out.data_ptr(), out.stride(0), block_table.data_ptr<int>(),
                                     block_table.stride(0), block_table.size(1), context_lens.data_ptr<int>(), b, hq, hkv, d,
                                     k_cache.size(1), k_cache.size(0), static_cast<float>(scale), /*split_workgroups=*/0,
                                     ws.data_ptr(), ws.numel(), current_stream()),
             "paged_attn_decode");
}

// Signature the reference's stub src/operators/flashattn/flashattn_decode.cu:11-12 intended
// (Q, K, V, is_causal, block_table, O), plus the context lengths it left out.
void flash_attn_decode(const at::Tensor& Q, const at::Tensor& K, const at::Tensor& V, bool /*is_causal*/,
                       const at::Tensor& block_table, const at::Tensor& context_lens, at::Tensor& O) {
    paged_attn_decode(Q, K, V, block_table, context_lens, 1.0 / std::sqrt(static_cast<double>(Q.size(-1))), O);
}

void paged_attn_prefill(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& cu_seqlens_q,
                        const at::Tensor& cu_seqlens_k, int64_t max_seqlen_q, const c10::optional<at::Tensor>& block_table,
                        double scale, bool causal, at::Tensor& out) {
    check_bf16_cuda(q, "q"); check_bf16_cuda(k, "k"); check_bf16_cuda(v, "v"); check_bf16_cuda(out, "out");
    TORCH_CHECK(q.dim() == 3 && out.sizes() == q.sizes() && q.stride(2) == 1 && q.stride(1) == q.size(2) &&
                out.stride(2) == 1 && out.stride(1) == q.size(2), "q/out must be [T, Hq, D] with contiguous heads");
    TORCH_CHECK(cu_seqlens_q.is_cuda() && cu_seqlens_q.scalar_type() == at::kInt && cu_seqlens_q.is_contiguous() &&
                cu_seqlens_k.is_cuda() && cu_seqlens_k.scalar_type() == at::kInt && cu_seqlens_k.is_contiguous() &&
                cu_seqlens_k.numel() == cu_seqlens_q.numel(), "cu_seqlens must be contiguous int32 GPU tensors of equal size");
    const int64_t nseq = cu_seqlens_q.numel() - 1, hq = q.size(1), d = q.size(2);
    if (q.size(0) == 0 || nseq <= 0) return;
    DeviceGuard guard(q.device());
    int rc;
    if (block_table.has_value()) {
        const at::Tensor& bt = *block_table;
        TORCH_CHECK(k.dim() == 4 && k.sizes() == v.sizes() && k.strides() == v.strides() && k.size(3) == d &&
                    k.stride(3) == 1 && k.stride(2) == d, "paged k/v must be [nblk, bs, Hkv, D]");
        TORCH_CHECK(bt.is_cuda() && bt.scalar_type() == at::kInt && bt.size(0) == nseq && bt.stride(1) == 1, "block_table must be int32 [nseq, MB]");
        rc = infer_paged_prefill_bf16(q.data_ptr(), q.stride(0), k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1),
                                      k.size(0) * k.size(1), out.data_ptr(), out.stride(0), cu_seqlens_q.data_ptr<int>(),
                                      cu_seqlens_k.data_ptr<int>(), bt.data_ptr<int>(), bt.stride(0), bt.size(1), nseq, max_seqlen_q, hq,
                                      k.size(2), d, k.size(1), k.size(0), static_cast<float>(scale), causal, current_stream());
    } else {
        TORCH_CHECK(k.dim() == 3 && k.sizes() == v.sizes() && k.strides() == v.strides() && k.size(2) == d &&
                    k.stride(2) == 1 && k.stride(1) == d, "packed k/v must be [T, Hkv, D]");
        rc = infer_paged_prefill_bf16(q.data_ptr(), q.stride(0), k.data_ptr(), v.data_ptr(), 0, k.stride(0), k.size(0),
                                      out.data_ptr(), out.stride(0), cu_seqlens_q.data_ptr<int>(), cu_seqlens_k.data_ptr<int>(),
                                      nullptr, 0, 0, nseq, max_seqlen_q, hq, k.size(1), d, 0, 0, static_cast<float>(scale),
                                      causal, current_stream());
    }
    check_rc(rc, "paged_attn_prefill");
}

// Goes through the registry facade, to show that the operator classes are live.
void registry_store_kvcache(const at::Tensor& key, const at::Tensor& value, at::Tensor& k_cache, at::Tensor& v_cache,
                            const at::Tensor& slot_mapping) {
    static infer::UnifiedOp<hip_bfloat16> ops;
    ops.store_kvcache(key, value, k_cache, v_cache, slot_mapping);
}

void registry_paged_attn_decode(const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache,
                                const at::Tensor& block_table, const at::Tensor& context_lens, double scale, at::Tensor& out) {
    static infer::UnifiedOp<hip_bfloat16> ops;
    out.copy_(ops.paged_attention(q, k_cache, v_cache, block_table, context_lens, scale));
}

}  // namespace

namespace infer {

template <typename T>
std::vector<torch::Tensor> KVAppendOperator<T>::forward(const std::vector<torch::Tensor>& in) {
    TORCH_CHECK(in.size() == 5, "KV_APPEND takes {key, value, k_cache, v_cache, slot_mapping}");
    torch::Tensor kc = in[2], vc = in[3];
    ::store_kvcache(in[0], in[1], kc, vc, in[4]);
    return {};
}

template <typename T>
std::vector<torch::Tensor> PagedAttentionOperator<T>::forward(const std::vector<torch::Tensor>& in) {
    TORCH_CHECK(in.size() == 5, "PAGED_ATTENTION takes {q, k_cache, v_cache, block_table, context_lens}");
    torch::Tensor out = torch::empty_like(in[0]);
    const double scale = scale_ > 0.0 ? scale_ : 1.0 / std::sqrt(static_cast<double>(in[0].size(-1)));
    ::paged_attn_decode(in[0], in[1], in[2], in[3], in[4], scale, out);
    return {out};
}

template class KVAppendOperator<hip_bfloat16>;
template class PagedAttentionOperator<hip_bfloat16>;

}  // namespace infer

TORCH_LIBRARY_FRAGMENT(_C, m) {
    m.def("store_kvcache(Tensor key, Tensor value, Tensor! k_cache, Tensor! v_cache, Tensor slot_mapping) -> ()");
    m.def("paged_attn_decode(Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_table, Tensor context_lens, "
          "float scale, Tensor! out) -> ()");
    m.def("flash_attn_decode(Tensor Q, Tensor K, Tensor V, bool is_causal, Tensor block_table, Tensor context_lens, "
          "Tensor! O) -> ()");
    m.def("paged_attn_prefill(Tensor q, Tensor k, Tensor v, Tensor cu_seqlens_q, Tensor cu_seqlens_k, int max_seqlen_q, "
          "Tensor? block_table, float scale, bool causal, Tensor! out) -> ()");
    m.def("registry_store_kvcache(Tensor key, Tensor value, Tensor! k_cache, Tensor! v_cache, Tensor slot_mapping) -> ()");
    m.def("registry_paged_attn_decode(Tensor q, Tensor k_cache, Tensor v_cache, Tensor block_table, Tensor context_lens, "
          "float scale, Tensor! out) -> ()");
}

TORCH_LIBRARY_IMPL(_C, CUDA, m) {
    m.impl("store_kvcache", &store_kvcache);
    m.impl("paged_attn_decode", &paged_attn_decode);
    m.impl("flash_attn_decode", &flash_attn_decode);
    m.impl("paged_attn_prefill", &paged_attn_prefill);
    m.impl("registry_store_kvcache", &registry_store_kvcache);
    m.impl("registry_paged_attn_decode", &registry_paged_attn_decode);
}
