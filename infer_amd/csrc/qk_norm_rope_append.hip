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
// = 16 bytes per lane); the sum of squares is reduced with four rotations inside the 16-lane row and the
// rotation partner (element i <-> i + 64) is the lane 8 places further on in the row, both as DPP
// operands of the consuming instruction (no LDS traffic).  Every byte is read and written once; at
// prefill sizes the kernel is bound by the vector pipe as much as by HBM (about 26 vector instructions
// per element: four bf16 roundings each), so the instruction count is kept down: roundings in pairs,
// the sign of the rotation folded into the sine, weights unpacked once.
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

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
// two floats rounded to nearest-even bf16 and packed (one v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}
// rounds a pair to bf16 and hands it back as floats: three instructions for two roundings
__device__ __forceinline__ void rb2(float& a, float& b) {
    const uint32_t w = pack(a, b);
    a = bf16_lo(w);
    b = bf16_hi(w);
}
__device__ __forceinline__ void unpack8(u32x4 r, float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { x[2 * i] = bf16_lo(r[i]); x[2 * i + 1] = bf16_hi(r[i]); }
}
// value of the lane `ROT` places further on in its row of 16 lanes (a rotation inside the row): stays on the
// vector pipe, and the compiler folds it into the instruction that consumes it
template <int ROT>
__device__ __forceinline__ float row_ror(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + ROT, 0xf, 0xf, false));
}

// Heads are handed out to the 16 groups of 16 lanes in passes of kPass heads per group: all rows of a
// pass (and, in the first pass, the V row, the slot, the position and the norm weights) are requested
// before anything is computed, so a token costs two memory round trips (position -> cos/sin) instead
// of one per head.
constexpr int kPass = 3;

__global__ void __launch_bounds__(256) qk_norm_rope_append_kernel(FusedArgs a) {
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const int p = tid & 15;          // 16-byte chunk of the head owned by this lane
    const int grp = tid >> 4;        // 16 groups of 16 lanes
    const int heads = a.hq + a.hkv;
    const int dkv = a.hkv * kD;
    const int64_t slot = __builtin_amdgcn_readfirstlane(a.slots[row]);
    const bool store = slot >= 0 && slot < a.num_slots;
    int64_t pos = a.positions[row];

    auto head_ptr = [&](int head) -> uint16_t* {
        return head < a.hq ? a.q + row * a.q_stride0 + (int64_t)head * kD + 8 * p
                           : a.k + row * a.k_stride0 + (int64_t)(head - a.hq) * kD + 8 * p;
    };
    u32x4 xin[kPass];
#pragma unroll
    for (int i = 0; i < kPass; ++i)
        if (grp + 16 * i < heads) xin[i] = *reinterpret_cast<const u32x4*>(head_ptr(grp + 16 * i));
    // the V row: 16-byte chunks tid, tid + 256, ... (one per lane of the first half of the workgroup at 8 x 128)
    const u32x4* vs = reinterpret_cast<const u32x4*>(a.v + row * a.v_stride0);
    u32x4 vin = {0u, 0u, 0u, 0u};
    const int vchunks = dkv / 8;
    if (tid < vchunks) vin = __builtin_nontemporal_load(vs + tid);      // before the slot is known: a padding row costs a wasted read
    float wq[8], wk[8];
    unpack8(*reinterpret_cast<const u32x4*>(a.q_weight + 8 * p), wq);
    unpack8(*reinterpret_cast<const u32x4*>(a.k_weight + 8 * p), wk);

    // cos / sin of this lane's rotation index i = 8 (p % 8) + e; the sine carries the sign of the lane's half:
    // o1 = x1 cos - x2 sin (lanes 0..7), o2 = x2 cos + x1 sin (lanes 8..15); rounding is symmetric, so
    // round(x * -sin) = -round(x * sin)
    pos = pos < 0 ? 0 : (pos >= a.max_position ? a.max_position - 1 : pos);
    float cs[8], sn[8];
    {
        const uint16_t* c = a.cos_sin + pos * kD + 8 * (p & 7);
        unpack8(*reinterpret_cast<const u32x4*>(c), cs);
        unpack8(*reinterpret_cast<const u32x4*>(c + 64), sn);
        if (p < 8) {
#pragma unroll
            for (int e = 0; e < 8; ++e) sn[e] = -sn[e];
        }
    }

    auto finish = [&](u32x4 raw, int head) {
        const bool is_q = head < a.hq;
        float x[8];
        unpack8(raw, x);
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
        ss += row_ror<8>(ss);
        ss += row_ror<4>(ss);
        ss += row_ror<2>(ss);
        ss += row_ror<1>(ss);
        const float r = 1.0f / sqrtf(ss * (1.0f / kD) + a.eps);
        float z[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) z[e] = x[e] * r;
#pragma unroll
        for (int e = 0; e < 8; e += 2) rb2(z[e], z[e + 1]);
#pragma unroll
        for (int e = 0; e < 8; ++e) z[e] *= is_q ? wq[e] : wk[e];
#pragma unroll
        for (int e = 0; e < 8; e += 2) rb2(z[e], z[e + 1]);
        float c1[8], c2[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            c1[e] = z[e] * cs[e];
            c2[e] = row_ror<8>(z[e]) * sn[e];     // partner element i +- 64 lives 8 lanes further on in the row
        }
#pragma unroll
        for (int e = 0; e < 8; e += 2) { rb2(c1[e], c1[e + 1]); rb2(c2[e], c2[e + 1]); }
        u32x4 out;
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = pack(c1[2 * i] + c2[2 * i], c1[2 * i + 1] + c2[2 * i + 1]);
        uint16_t* dst = head_ptr(head);
        if (is_q) {
            *reinterpret_cast<u32x4*>(dst) = out;
        } else {
            if (a.write_k_inplace) *reinterpret_cast<u32x4*>(dst) = out;
            if (store)
                __builtin_nontemporal_store(out, reinterpret_cast<u32x4*>(a.k_cache + slot * dkv + (int64_t)(head - a.hq) * kD + 8 * p));
        }
    };

#pragma unroll
    for (int i = 0; i < kPass; ++i)
        if (grp + 16 * i < heads) finish(xin[i], grp + 16 * i);
    if (store) {
        u32x4* vd = reinterpret_cast<u32x4*>(a.v_cache + slot * dkv);
        if (tid < vchunks) __builtin_nontemporal_store(vin, vd + tid);
        for (int c = tid + 256; c < vchunks; c += 256) __builtin_nontemporal_store(__builtin_nontemporal_load(vs + c), vd + c);
    }
    // more than 16 * kPass heads: further passes, each again with its loads first
    for (int h0 = 16 * kPass; h0 < heads; h0 += 16 * kPass) {
#pragma unroll
        for (int i = 0; i < kPass; ++i)
            if (h0 + grp + 16 * i < heads) xin[i] = *reinterpret_cast<const u32x4*>(head_ptr(h0 + grp + 16 * i));
#pragma unroll
        for (int i = 0; i < kPass; ++i)
            if (h0 + grp + 16 * i < heads) finish(xin[i], h0 + grp + 16 * i);
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
