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
// operands or moves (no LDS traffic).  Every byte is read and written once.  With four bf16 roundings
// per element the vector pipe was as loaded as HBM, so the instruction count is kept down (the kernel
// now runs at the rate of a copy with this mix of reads and in-place writes).  Rounded values stay PACKED (two bf16 per register, one
// v_cvt_pk_bf16_f32 per pair) and the next product reads them with v_dot2_f32_bf16 against a factor
// pair whose other half is zero: a.lo * b.lo + a.hi * 0 + 0 is the exact float32 product of two bf16
// values, so "unpack, then multiply" is one instruction instead of two, and the last addition of the
// rotation is the same instruction on the pair (x1 cos, x2 sin) against (1, 1).  The sign of the
// rotation is folded into the sine, the factor pairs are masked once per token, and the reciprocal
// square root is the hardware's (1 ulp; after the rounding to bf16 that follows, one element in tens of
// thousands differs from a correctly rounded one by a bf16 ulp).  About 15 vector instructions per
// element (25 with every value unpacked to float32 after each rounding).
// Two corners differ from an element-by-element evaluation and are outside what the reference's own
// tests pin: a NaN or infinity in one element of a pair reaches its neighbour (0 * inf), and a result
// that is zero may carry the other sign.
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
// value of the lane `ROT` places further on in its row of 16 lanes (a rotation inside the row): stays on the
// vector pipe
template <int ROT>
__device__ __forceinline__ float row_ror(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + ROT, 0xf, 0xf, false));
}

// v_dot2_f32_bf16 d, a, b, c:  d = a.lo * b.lo + a.hi * b.hi + c  in float32 (a, b pairs of bf16).
// The compiler only selects the accumulating two-operand form of this instruction, which costs a move
// per product that starts from zero, so the three-operand form is written out - in blocks, because the
// instruction has no interlock on this part: a register it wrote may be read, by anything but the
// accumulator input of another dot2, only three issue slots later, and the compiler does not insert
// wait states for instructions it cannot see.  Inside the blocks below every consumer sits at least
// three instructions behind its producer, with s_nop where nothing useful is left to fill the gap.

// sum of the squares of the eight elements of four pairs
__device__ __forceinline__ float sum_squares(u32x4 x) {
    float r;
    __asm__("v_dot2_f32_bf16 %0, %1, %1, 0\n\t"
            "v_dot2_f32_bf16 %0, %2, %2, %0\n\t"
            "v_dot2_f32_bf16 %0, %3, %3, %0\n\t"
            "v_dot2_f32_bf16 %0, %4, %4, %0\n\t"
            "s_nop 2"
            : "=&v"(r) : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]));
    return r;
}

// A factor pair split for dot2: lo[i] = (value 2 i, 0), hi[i] = (0, value 2 i + 1).
struct Factors {
    uint32_t lo[4], hi[4];
    __device__ __forceinline__ void set(u32x4 packed) {
#pragma unroll
        for (int i = 0; i < 4; ++i) { lo[i] = packed[i] & 0x0000ffffu; hi[i] = packed[i] & 0xffff0000u; }
    }
};

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
    Factors wq, wk;
    wq.set(*reinterpret_cast<const u32x4*>(a.q_weight + 8 * p));
    wk.set(*reinterpret_cast<const u32x4*>(a.k_weight + 8 * p));

    // cos / sin of this lane's rotation index i = 8 (p % 8) + e; the sine carries the sign of the lane's half:
    // o1 = x1 cos - x2 sin (lanes 0..7), o2 = x2 cos + x1 sin (lanes 8..15); rounding is symmetric, so
    // round(x * -sin) = -round(x * sin)
    pos = pos < 0 ? 0 : (pos >= a.max_position ? a.max_position - 1 : pos);
    Factors cs, sn;
    {
        const uint16_t* c = a.cos_sin + pos * kD + 8 * (p & 7);
        cs.set(*reinterpret_cast<const u32x4*>(c));
        u32x4 s4 = *reinterpret_cast<const u32x4*>(c + 64);
        if (p < 8) s4 ^= u32x4{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
        sn.set(s4);
    }
    const float inv_d = 1.0f / kD;

    auto finish = [&](u32x4 raw, int head, const Factors& w) {
        const bool is_q = head < a.hq;
        // mean of squares: the pairs squared and summed as they are, then over the 16 lanes of the head
        float ss = sum_squares(raw);
        ss += row_ror<8>(ss);
        ss += row_ror<4>(ss);
        ss += row_ror<2>(ss);
        ss += row_ror<1>(ss);
        const float r = __builtin_amdgcn_rsqf(__builtin_fmaf(ss, inv_d, a.eps));
        uint32_t z[4];
        // x * rsqrt(var + eps), rounded
#pragma unroll
        for (int i = 0; i < 4; ++i) z[i] = pack(bf16_lo(raw[i]) * r, bf16_hi(raw[i]) * r);
        // times the weight, rounded: z[i] = pack(z[i].lo * w[2 i], z[i].hi * w[2 i + 1])
        {
            uint32_t t0, t1, t2, t3, t4, t5, t6, t7;
            // (volatile: the blocks of a head keep their order, which the DPP reads of the next block count on:
            // a register written by the vector pipe may be read through DPP two issue slots later)
            __asm__ volatile("v_dot2_f32_bf16 %4, %0, %12, 0\n\t"
                    "v_dot2_f32_bf16 %5, %0, %16, 0\n\t"
                    "v_dot2_f32_bf16 %6, %1, %13, 0\n\t"
                    "v_dot2_f32_bf16 %7, %1, %17, 0\n\t"
                    "v_dot2_f32_bf16 %8, %2, %14, 0\n\t"
                    "v_dot2_f32_bf16 %9, %2, %18, 0\n\t"
                    "v_dot2_f32_bf16 %10, %3, %15, 0\n\t"
                    "v_dot2_f32_bf16 %11, %3, %19, 0\n\t"
                    "v_cvt_pk_bf16_f32 %0, %4, %5\n\t"
                    "v_cvt_pk_bf16_f32 %1, %6, %7\n\t"
                    "v_cvt_pk_bf16_f32 %2, %8, %9\n\t"
                    "v_cvt_pk_bf16_f32 %3, %10, %11"
                    : "+v"(z[0]), "+v"(z[1]), "+v"(z[2]), "+v"(z[3]), "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3),
                      "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7)
                    : "v"(w.lo[0]), "v"(w.lo[1]), "v"(w.lo[2]), "v"(w.lo[3]), "v"(w.hi[0]), "v"(w.hi[1]), "v"(w.hi[2]),
                      "v"(w.hi[3]));
        }
        // rotation of two pairs at a time: the partner element i +- 64 lives 8 lanes further on in the
        // row (DPP move of the pair); x cos and partner sin are rounded as a pair, their sum is that
        // pair against (1, 1), and two sums are rounded into one output pair
        uint32_t o[4];
        const uint32_t ones = 0x3f803f80u;
        auto rotate2 = [&](int i, uint32_t& o0, uint32_t& o1) {
            uint32_t p0, p1, t0, t1, t2, t3, t4, t5, t6, t7;
            __asm__ volatile("v_mov_b32_dpp %2, %12 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %3, %13 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                    "v_dot2_f32_bf16 %4, %12, %14, 0\n\t"
                    "v_dot2_f32_bf16 %5, %2, %16, 0\n\t"
                    "v_dot2_f32_bf16 %6, %12, %15, 0\n\t"
                    "v_dot2_f32_bf16 %7, %2, %17, 0\n\t"
                    "v_dot2_f32_bf16 %8, %13, %18, 0\n\t"
                    "v_dot2_f32_bf16 %9, %3, %20, 0\n\t"
                    "v_dot2_f32_bf16 %10, %13, %19, 0\n\t"
                    "v_dot2_f32_bf16 %11, %3, %21, 0\n\t"
                    "v_cvt_pk_bf16_f32 %4, %4, %5\n\t"
                    "v_cvt_pk_bf16_f32 %6, %6, %7\n\t"
                    "v_cvt_pk_bf16_f32 %8, %8, %9\n\t"
                    "v_cvt_pk_bf16_f32 %10, %10, %11\n\t"
                    "v_dot2_f32_bf16 %5, %4, %22, 0\n\t"
                    "v_dot2_f32_bf16 %7, %6, %22, 0\n\t"
                    "v_dot2_f32_bf16 %9, %8, %22, 0\n\t"
                    "v_dot2_f32_bf16 %11, %10, %22, 0\n\t"
                    "s_nop 1\n\t"
                    "v_cvt_pk_bf16_f32 %0, %5, %7\n\t"
                    "v_cvt_pk_bf16_f32 %1, %9, %11"
                    : "=&v"(o0), "=&v"(o1), "=&v"(p0), "=&v"(p1), "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4),
                      "=&v"(t5), "=&v"(t6), "=&v"(t7)
                    : "v"(z[i]), "v"(z[i + 1]), "v"(cs.lo[i]), "v"(cs.hi[i]), "v"(sn.lo[i]), "v"(sn.hi[i]), "v"(cs.lo[i + 1]),
                      "v"(cs.hi[i + 1]), "v"(sn.lo[i + 1]), "v"(sn.hi[i + 1]), "s"(ones));
        };
        rotate2(0, o[0], o[1]);
        rotate2(2, o[2], o[3]);
        const u32x4 out = {o[0], o[1], o[2], o[3]};
        uint16_t* dst = head_ptr(head);
        if (is_q) {
            *reinterpret_cast<u32x4*>(dst) = out;    // not streamed: the attention kernel behind it reads these rows from cache
        } else {
            if (a.write_k_inplace) *reinterpret_cast<u32x4*>(dst) = out;
            if (store)
                __builtin_nontemporal_store(out, reinterpret_cast<u32x4*>(a.k_cache + slot * dkv + (int64_t)(head - a.hq) * kD + 8 * p));
        }
    };
    // The four heads of a wavefront are consecutive: all query heads or all key heads unless the number of
    // query heads is not a multiple of four.  The weights are chosen per wavefront where that is so.
    auto finish_head = [&](u32x4 raw, int head) {
        const bool is_q = head < a.hq;
        if (__all(is_q)) finish(raw, head, wq);
        else if (__all(!is_q)) finish(raw, head, wk);
        else {
            Factors w;
#pragma unroll
            for (int i = 0; i < 4; ++i) { w.lo[i] = is_q ? wq.lo[i] : wk.lo[i]; w.hi[i] = is_q ? wq.hi[i] : wk.hi[i]; }
            finish(raw, head, w);
        }
    };

#pragma unroll
    for (int i = 0; i < kPass; ++i)
        if (grp + 16 * i < heads) finish_head(xin[i], grp + 16 * i);
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
            if (h0 + grp + 16 * i < heads) finish_head(xin[i], h0 + grp + 16 * i);
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
