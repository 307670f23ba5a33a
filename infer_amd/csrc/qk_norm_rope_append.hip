// Fused per-head RMSNorm(Q, K) + neox RoPE(Q, K) + KV append for gfx950 (MI355X).
//
// Fuses what the reference does in four launches in front of attention
// (infer/models/Qwen3.py:113-131): q_norm and k_norm (RMSNorm.rms_forward, infer/ops/norm.py:63-73),
// the in-place rotary embedding (rotary_embedding_kernel, src/operators/rope/rope.cu:43-133, neox
// style), and store_kvcache (infer/ops/attention.py:16-45).  Q is normalised and rotated in place;
// K is normalised, rotated and written straight into the paged K cache at its slot (and, if asked,
// back in place, which the prefill path without a cached prefix needs); the V row is copied to the
// V cache.  K is read once and never re-read; one launch instead of four.
//
// Arithmetic follows the reference step by step so that results match it to rounding: float32 mean
// of squares and x * rsqrt(var + eps), rounded to bf16; times the bf16 weight, rounded to bf16;
// o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin with each product and the sum rounded to bf16.
//
// One workgroup of 256 threads per token.  A group of 16 lanes owns one head at a time (8 elements
// = 16 bytes per lane); the sum of squares is reduced with four lane shuffles, the rotation partner
// (element i <-> i + 64) is lane p ^ 8 of the same group.  Memory bound (every byte read and
// written once).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/infer_kv.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kD = 128;

struct FusedArgs {
    uint16_t* q; int64_t q_stride0;
    uint16_t* k; int64_t k_stride0;
    const uint16_t* v; int64_t v_stride0;
    const int64_t* positions;
    const uint16_t* q_weight;
    const uint16_t* k_weight;
    const uint16_t* cos_sin;     // [max_position, 128]: cos(64) | sin(64)
    int64_t max_position;
    uint16_t* k_cache;
    uint16_t* v_cache;
    const int32_t* slots;
    int64_t num_slots;
    int hq, hkv;
    float eps;
    int write_k_inplace;
};

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
// round-to-nearest-even to bf16, result kept as float
__device__ __forceinline__ float rb(float x) { return (float)(__bf16)x; }
__device__ __forceinline__ uint32_t pack(float lo, float hi) {
    const __bf16 a = (__bf16)lo, b = (__bf16)hi;
    return (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
}
__device__ __forceinline__ void unpack8(u32x4 r, float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { x[2 * i] = bf16_lo(r[i]); x[2 * i + 1] = bf16_hi(r[i]); }
}

__global__ void __launch_bounds__(256) qk_norm_rope_append_kernel(FusedArgs a) {
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const int p = tid & 15;          // 16-byte chunk of the head owned by this lane
    const int grp = tid >> 4;        // 16 groups of 16 lanes
    const int64_t slot = __builtin_amdgcn_readfirstlane(a.slots[row]);
    const bool store = slot >= 0 && slot < a.num_slots;
    int64_t pos = a.positions[row];
    pos = pos < 0 ? 0 : (pos >= a.max_position ? a.max_position - 1 : pos);

    // cos / sin of this lane's rotation index i = 8 (p % 8) + e
    float cs[8], sn[8];
    {
        const uint16_t* c = a.cos_sin + pos * kD + 8 * (p & 7);
        unpack8(*reinterpret_cast<const u32x4*>(c), cs);
        unpack8(*reinterpret_cast<const u32x4*>(c + 64), sn);
    }
    const int dkv = a.hkv * kD;

    for (int head = grp; head < a.hq + a.hkv; head += 16) {
        const bool is_q = head < a.hq;
        uint16_t* src = is_q ? a.q + row * a.q_stride0 + (int64_t)head * kD
                             : a.k + row * a.k_stride0 + (int64_t)(head - a.hq) * kD;
        const uint16_t* wptr = is_q ? a.q_weight : a.k_weight;
        float x[8], w[8];
        unpack8(*reinterpret_cast<const u32x4*>(src + 8 * p), x);
        unpack8(*reinterpret_cast<const u32x4*>(wptr + 8 * p), w);
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
#pragma unroll
        for (int m = 1; m < 16; m <<= 1) ss += __shfl_xor(ss, m);
        const float r = 1.0f / sqrtf(ss * (1.0f / kD) + a.eps);
        float z[8], zp[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) z[e] = rb(rb(x[e] * r) * w[e]);
#pragma unroll
        for (int e = 0; e < 8; ++e) zp[e] = __shfl_xor(z[e], 8);     // partner element i +- 64
        float o[8];
        if (p < 8) {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = rb(z[e] * cs[e]) - rb(zp[e] * sn[e]);     // x1*cos - x2*sin
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = rb(z[e] * cs[e]) + rb(zp[e] * sn[e]);     // x2*cos + x1*sin
        }
        u32x4 out;
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = pack(o[2 * i], o[2 * i + 1]);
        if (is_q) {
            *reinterpret_cast<u32x4*>(src + 8 * p) = out;
        } else {
            if (a.write_k_inplace) *reinterpret_cast<u32x4*>(src + 8 * p) = out;
            if (store) *reinterpret_cast<u32x4*>(a.k_cache + slot * dkv + (int64_t)(head - a.hq) * kD + 8 * p) = out;
        }
    }
    if (store) {
        const u32x4* vs = reinterpret_cast<const u32x4*>(a.v + row * a.v_stride0);
        u32x4* vd = reinterpret_cast<u32x4*>(a.v_cache + slot * dkv);
        for (int c = tid; c < dkv / 8; c += 256) vd[c] = vs[c];
    }
}

}  // namespace

extern "C" int infer_kv_qk_norm_rope_append_bf16(void* q, int64_t q_stride0, void* k, int64_t k_stride0, const void* v,
                                                 int64_t v_stride0, const int64_t* positions, const void* q_norm_weight,
                                                 const void* k_norm_weight, float eps, const void* cos_sin_cache,
                                                 int64_t max_position, void* k_cache, void* v_cache,
                                                 const int32_t* slot_mapping, int64_t n_rows, int64_t num_q_heads,
                                                 int64_t num_kv_heads, int64_t head_dim, int64_t num_slots,
                                                 int write_k_inplace, void* stream) {
    if (n_rows == 0) return INFER_KV_OK;
    if (!q || !k || !v || !positions || !q_norm_weight || !k_norm_weight || !cos_sin_cache || !k_cache || !v_cache ||
        !slot_mapping)
        return INFER_KV_EINVAL;
    if (n_rows < 0 || n_rows > 0x7fffffffLL || num_q_heads <= 0 || num_kv_heads <= 0 || max_position <= 0 || num_slots <= 0)
        return INFER_KV_EINVAL;
    if (head_dim != kD) return INFER_KV_EUNSUPPORTED;
    if (q_stride0 < num_q_heads * kD || k_stride0 < num_kv_heads * kD || v_stride0 < num_kv_heads * kD) return INFER_KV_EINVAL;
    if ((q_stride0 | k_stride0 | v_stride0) & 7) return INFER_KV_EALIGN;
    if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)q_norm_weight | (uintptr_t)k_norm_weight |
         (uintptr_t)cos_sin_cache | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15)
        return INFER_KV_EALIGN;
    FusedArgs a;
    a.q = (uint16_t*)q; a.q_stride0 = q_stride0;
    a.k = (uint16_t*)k; a.k_stride0 = k_stride0;
    a.v = (const uint16_t*)v; a.v_stride0 = v_stride0;
    a.positions = positions;
    a.q_weight = (const uint16_t*)q_norm_weight;
    a.k_weight = (const uint16_t*)k_norm_weight;
    a.cos_sin = (const uint16_t*)cos_sin_cache;
    a.max_position = max_position;
    a.k_cache = (uint16_t*)k_cache;
    a.v_cache = (uint16_t*)v_cache;
    a.slots = slot_mapping;
    a.num_slots = num_slots;
    a.hq = (int)num_q_heads;
    a.hkv = (int)num_kv_heads;
    a.eps = eps;
    a.write_k_inplace = write_k_inplace ? 1 : 0;
    hipLaunchKernelGGL(qk_norm_rope_append_kernel, dim3((unsigned)n_rows), dim3(256), 0, (hipStream_t)stream, a);
    return (int)hipGetLastError();
}
