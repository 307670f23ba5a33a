// Paged decode attention for gfx950 (MI355X): block_table-gathered GQA attention of one query
// token per sequence, flash-decoding style (split KV + merge), bf16 in / fp32 accumulate.
//
// Replaces flash_attn_with_kvcache(...) at infer/ops/attention.py:118-120 of the reference
// (the reference's own decode kernel, src/operators/flashattn/flashattn_decode.cu, is an empty
// stub).  The merge rule for partial (max, sum) pairs is the same algebra as the reference's
// softmax reduction (src/operators/softmax/softmax.cu:5-16).
//
// Work decomposition
//   A "step" is 32 consecutive tokens of one sequence (never straddles a cache block because
//   block_size % 32 == 0).  All steps of all sequences are laid end to end and cut into at
//   most gridDim.x spans of equal length (to within one step); workgroup x streams span x for up to 8 KV heads, one wavefront per
//   KV head, so a workgroup reads whole 2 KiB token rows while each wavefront runs its own
//   private pipeline (no workgroup barrier anywhere).  A span may cover the tail of one
//   sequence and the head of the next: each (sequence, span) piece is a "segment" and leaves a
//   partial result (parked in LDS, stored once the wavefront has issued its last load); the merge
//   kernel folds the segments of a sequence together.
//
// Per step and wavefront (KV head h, G = Hq/Hkv query heads):
//   S^T[token, head] = K[token, :] . Q^T        2 tiles x 4 v_mfma_f32_16x16x32_bf16
//   online softmax in the MFMA accumulator layout (lane = head, 8 tokens per lane)
//   O^T[d, head]    += V^T[d, token] . P^T      8 v_mfma_f32_16x16x32_bf16
//   K fragments are loaded straight from global memory in MFMA operand layout (16 B per lane);
//   V rows are loaded coalesced (256 B per token), staged in a wave-private LDS tile and read
//   back transposed.  The accumulator layout of S^T is exactly the B-operand layout of the
//   second product, so P never moves between lanes.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "decode_layout.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef short i16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) i16x4 lds_i16x4;

constexpr int kD = 128;            // head_dim
constexpr int kStep = 32;          // tokens per step
constexpr int kLdsRow = 288;       // bytes per staged V row: 256 + 32 so 4 consecutive rows hit disjoint banks
constexpr int kLdsWave = kStep * kLdsRow;

struct DecodeArgs {
    const uint16_t* q;
    int64_t q_stride0;
    const uint16_t* k;
    const uint16_t* v;
    int64_t blk_stride;
    int64_t tok_stride;
    const int32_t* bt;
    int64_t bt_stride0;
    const int32_t* ctx; // nullptr: every sequence has uniform_len tokens
    int uniform_len;
    int max_ctx;        // lengths are clamped to what the block table can address (table_cols * block_size)
    int batch;
    int group;          // query heads per KV head
    int num_kv_heads;
    int block_size;
    int num_blocks;
    float scale_log2;   // softmax scale * log2(e)
    int32_t* header;
    int32_t* seg_first;
    int32_t* seg_last;
    unsigned char* rec; // [slots] partial-result records (layout: decode_record_bytes)
    int rec_stride;
    int slots_per_head; // records per KV head in the workspace (layout constant, >= gridDim.x + batch)
    uint16_t* out;      // uniform kernel only: it writes the result itself
    int64_t out_stride0;
};

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 x) { return __builtin_bit_cast(bf16x8, x); }

__device__ __forceinline__ u32x4 load16(const uint16_t* p) {
    return *reinterpret_cast<const u32x4*>(p);
}
// V rows are read once per launch, 256 contiguous bytes per token and instruction: with the streaming
// hint the split kernel takes 103.4 instead of 112.9 us on 64 sequences of 512-4096 tokens.  K fragments
// (64 bytes per token and instruction, each cache line touched by two instructions) gain nothing from
// the hint, and with it the merge kernel that follows runs slower (split + merge 106.4 against 105.6 us
// there, 175 against 170.5 us on 8 sequences of 32,768), so K is loaded plainly.
__device__ __forceinline__ u32x4 load16_stream(const uint16_t* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}

__device__ __forceinline__ int steps_of(int len) { return len > 0 ? (len + kStep - 1) / kStep : 0; }

// Context length of sequence i as the kernels use it: a length the block table row cannot address is
// cut to the row's capacity, so a corrupt length cannot make the table gather run past the row.
__device__ __forceinline__ int ctx_len(const DecodeArgs& a, int i) {
    const int len = a.ctx ? a.ctx[i] : a.uniform_len;
    return len < a.max_ctx ? len : a.max_ctx;
}

// Inclusive prefix sum over the 64 lanes on the vector pipe (data-parallel primitives): shifts by 1,
// 2, 4 and 8 inside each row of 16 lanes, then the last lane of row 0 (2) is added to row 1 (3) and the
// last lane of the lower half to the upper half.  Six instructions, where shuffles would be six round
// trips through LDS in front of the first load of the kernel.
__device__ __forceinline__ int wave_inclusive_scan(int x, int) {
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false);   // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false);   // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false);   // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false);   // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false);   // row_bcast:15 into rows 1 and 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false);   // row_bcast:31 into rows 2 and 3
    return x;
}

__device__ __forceinline__ int wave_sum(int x) { return __builtin_amdgcn_readlane(wave_inclusive_scan(x, 0), 63); }

// max over lanes l and l ^ 16 (l ^ 32) in every lane.  v_permlane16_swap exchanges the odd 16-lane rows
// of its first operand with the even rows of its second: fed the same value twice it returns
// (rows 0 0 2 2, rows 1 1 3 3), whose maximum is the reduction; v_permlane32_swap does the same with
// the two halves of the wavefront.  Both stay on the vector pipe, where a shuffle would go through LDS.
__device__ __forceinline__ float max_xor16(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return fmaxf(__builtin_bit_cast(float, r[0]), __builtin_bit_cast(float, r[1]));
}
__device__ __forceinline__ float max_xor32(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__builtin_bit_cast(float, r[0]), __builtin_bit_cast(float, r[1]));
}

// Keeps the compiler from moving LDS traffic across this point.  The LDS queue of one
// wavefront is processed in order, so within a wavefront a compiler barrier is all the
// write -> read -> write sequence on the private tile needs.
__device__ __forceinline__ void lds_order() { __asm__ volatile("" ::: "memory"); }

// ---------------------------------------------------------------------------------------------
// Span plan.  A wavefront first lists the segments (pieces of sequences) of its span in a small
// wave-private LDS table and gathers the block ids of all of them into ONE vector register
// (lane i = i-th block touched by the span, "block ordinal" i).  After that the streaming loop
// needs no memory access for addressing: crossing a block or a sequence boundary is a register
// read, so loads for the next sequence are in flight long before the current one is finished.
constexpr int kPlanInts = 8;        // ints per segment record
constexpr int kMaxSegs = 32;        // segments per batch (a span with more is run in several batches)
constexpr int kPlanBytes = kMaxSegs * kPlanInts * 4;
// Partial results of finished segments wait in LDS until the wavefront has issued its last load:
// a global store in the middle of the stream would make the outstanding-load counter unordered
// (loads and stores share it) and force a full drain of the prefetch pipeline.
constexpr int kDeferBytes = 8448;   // 4 segments at group size 4, 2 at 8, 1 at 16
constexpr int kLdsPerWave = kLdsWave + kPlanBytes + kDeferBytes;

struct SegRec {      // one record of the plan, all wave-uniform
    int b;           // sequence
    int len;         // its context length
    int s_lo, s_hi;  // steps of the sequence covered by this span
    int ord0;        // block ordinal of the first step's block
    int in0;         // step index of s_lo inside its block
    int blk0;        // index of that block in the sequence's table row
};

__device__ __forceinline__ SegRec read_rec(const int* plan, int seg) {
    const int* p = plan + seg * kPlanInts;
    SegRec r;
    r.b = __builtin_amdgcn_readfirstlane(p[0]);
    r.len = __builtin_amdgcn_readfirstlane(p[1]);
    r.s_lo = __builtin_amdgcn_readfirstlane(p[2]);
    r.s_hi = __builtin_amdgcn_readfirstlane(p[3]);
    r.ord0 = __builtin_amdgcn_readfirstlane(p[4]);
    r.in0 = __builtin_amdgcn_readfirstlane(p[5]);
    r.blk0 = __builtin_amdgcn_readfirstlane(p[6]);
    return r;
}

// Walks the steps of a batch of segments in order.  Used three times: by the K loads (two steps
// ahead), the V loads (one step ahead) and the arithmetic.
struct StepCursor {
    int seg, nseg;
    int s, s_hi;     // current step of the current segment, end of the segment
    int in, ord;     // step inside its block, block ordinal
    int b, blk0, ord0;
    __device__ __forceinline__ void enter(const int* plan, int seg_) {
        seg = seg_;
        if (seg < nseg) {
            const SegRec r = read_rec(plan, seg);
            s = r.s_lo; s_hi = r.s_hi; in = r.in0; ord = r.ord0; b = r.b; blk0 = r.blk0; ord0 = r.ord0;
        }
    }
    __device__ __forceinline__ bool live() const { return seg < nseg; }
    __device__ __forceinline__ void advance(const int* plan, int steps_per_blk) {
        ++s;
        if (++in == steps_per_blk) { in = 0; ++ord; }
        if (s == s_hi) enter(plan, seg + 1);
    }
};

// Runs one batch of segments for KV head h.
//
// Software pipeline (loads return in issue order, so the waits are exact counts): K fragments are
// double-buffered in registers, V rows single-buffered; while step i is being reduced, K(i+1),
// then K(i+2) and V(i+1) are in flight, across sequence boundaries.  Loads past the end of the
// batch are redirected to one dummy 16-byte location instead of being skipped, which keeps the
// number of outstanding loads at every wait independent of control flow.
template <bool kKeep = false>
__device__ __forceinline__ void run_batch(const DecodeArgs& a, unsigned char* lds, const int* plan, int nseg,
                                          int total_steps, int tblv_loaded, int h, int w, int lane) {
    // The block ids were gathered by vector loads.  Hand them to the loop as a plain register value:
    // otherwise every later read of this register is treated as "may still be in flight" and gets a
    // wait that also drains the K/V loads issued since, which defeats the pipeline.
    int tblv;
    __asm__ volatile("v_mov_b32 %0, %1" : "=v"(tblv) : "v"(tblv_loaded));
    const int g = lane >> 4;   // lane group: the k-slice of MFMA operands, the row-quad of results
    const int n = lane & 15;   // operand row / result column
    const int G = a.group;
    const int steps_per_blk = a.block_size / kStep;

    auto block_id = [&](const StepCursor& c) -> int {
        int blk;
        if (c.ord < 64) blk = __builtin_amdgcn_readlane(tblv, c.ord);
        else   // a single segment longer than 64 blocks (it is alone in its batch)
            blk = __builtin_amdgcn_readfirstlane(a.bt[(int64_t)c.b * a.bt_stride0 + c.blk0 + (c.ord - c.ord0)]);
        return blk < 0 ? 0 : (blk >= a.num_blocks ? a.num_blocks - 1 : blk);
    };

    // Q as the B operand of S^T = K Q^T: lane (g, n) holds Q[head n][32 j + 8 g .. +8].
    auto load_q = [&](int b, u32x4 (&dst)[4]) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        const uint16_t* qp = a.q + (int64_t)b * a.q_stride0 + (int64_t)(h * G + (n < G ? n : 0)) * kD + 8 * g;
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[j] = n < G ? load16(qp + 32 * j) : z;
    };

    StepCursor ccur, kcur, vcur;
    ccur.nseg = kcur.nseg = vcur.nseg = nseg;
    ccur.enter(plan, 0);
    kcur = ccur;
    vcur = ccur;
    SegRec cseg = read_rec(plan, 0);

    u32x4 qreg[4], qnext[4];
    load_q(cseg.b, qreg);
    if (nseg > 1) load_q(__builtin_amdgcn_readfirstlane(plan[kPlanInts]), qnext);
    else {
#pragma unroll
        for (int j = 0; j < 4; ++j) qnext[j] = u32x4{0u, 0u, 0u, 0u};
    }

    f32x4 acc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY;
    float l_run = 0.f;

    // Row r of K tile t holds token 8 (r / 4) + 4 t + r % 4 of the step, so that result element
    // (tile t, quad element e) of lane group g is token 8 g + (4 t + e): lane group g ends up with
    // the 8 consecutive tokens 8 g .. 8 g + 7, which is also how the transposing LDS read hands out V.
    const uint32_t k_lane = (uint32_t)((8 * (n >> 2) + (n & 3)) * a.tok_stride + 8 * g);
    const uint32_t v_lane = (uint32_t)(g * a.tok_stride + 8 * n);
    const uint32_t tile_off = (uint32_t)(4 * a.tok_stride);
    const uint32_t quad_off = (uint32_t)(4 * a.tok_stride);
    const uint16_t* dummy = a.q;   // 256 readable bytes that stay in cache

    u32x4 kbuf[2][2][4];
    u32x4 vreg[8];

    auto issue_k = [&](auto PC) {
        constexpr int P = decltype(PC)::value;
        const uint16_t* kb = dummy;
        uint32_t lane_off = 0, t_off = 0;
        if (kcur.live()) {
            kb = a.k + ((int64_t)block_id(kcur) * a.blk_stride + (int64_t)(kcur.in * kStep) * a.tok_stride + (int64_t)h * kD);
            lane_off = k_lane;
            t_off = tile_off;
            kcur.advance(plan, steps_per_blk);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) kbuf[P][t][j] = load16(kb + (t * t_off + lane_off) + 32 * j);
    };
    auto issue_v = [&]() {
        const uint16_t* vb = dummy;
        uint32_t lane_off = 0, q_off = 0;
        if (vcur.live()) {
            vb = a.v + ((int64_t)block_id(vcur) * a.blk_stride + (int64_t)(vcur.in * kStep) * a.tok_stride + (int64_t)h * kD);
            lane_off = v_lane;
            q_off = quad_off;
            vcur.advance(plan, steps_per_blk);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) vreg[i] = load16_stream(vb + (i * q_off + lane_off));
    };

    // Partial results: parked in LDS (lane-private layout, valid lanes only), written out by drain().
    unsigned char* defer = lds + kLdsWave + kPlanBytes;
    const int slot_bytes = a.rec_stride;            // 4G lanes x 8 x 16 B accumulators + G x 8 B (max, sum), padded
    const int defer_cap = kDeferBytes / slot_bytes; // >= 1 for G <= 16
    int ndef = 0, first_def = 0;                    // parked segments are first_def .. first_def + ndef - 1
    const int vlane = g * G + n;                    // index among the 4G lanes that hold real heads

    auto drain = [&]() {
        for (int k = 0; k < ndef; ++k) {
            const int b = __builtin_amdgcn_readfirstlane(plan[(first_def + k) * kPlanInts]);
            const int64_t slot = (int64_t)h * a.slots_per_head + w + b;
            // the record leaves as it was parked: all 64 lanes, 16 B each, one contiguous run
            const unsigned char* src = defer + k * slot_bytes;
            unsigned char* dst = a.rec + slot * slot_bytes;
            for (int off = lane * 16; off < slot_bytes; off += 1024)
                *reinterpret_cast<u32x4*>(dst + off) = *reinterpret_cast<const u32x4*>(src + off);
        }
        first_def += ndef;
        ndef = 0;
    };

    // Parks the partial result of the segment just finished and resets the accumulators.
    auto flush = [&]() {
        float l_tot = l_run + __shfl_xor(l_run, 16);
        l_tot += __shfl_xor(l_tot, 32);
        if (ndef == defer_cap) {          // only when one span covers many short sequences
            lds_order();
            drain();
            __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): leave no store in flight behind
        }
        unsigned char* dst = defer + ndef * slot_bytes;
        lds_order();
        if (n < G) {
#pragma unroll
            for (int t = 0; t < 8; ++t) *reinterpret_cast<f32x4*>(dst + (vlane * 8 + t) * 16) = acc[t];
            if (g == 0) *reinterpret_cast<float2*>(dst + 512 * G + n * 8) = make_float2(m_run, l_tot);
        }
        lds_order();
        ++ndef;
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        m_run = -INFINITY;
        l_run = 0.f;
    };

    auto step = [&](auto PC) {
        constexpr int P = decltype(PC)::value;
        // ---- S^T = K Q^T
        f32x4 sc[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            sc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                sc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kbuf[P][t][j]), as_bf16x8(qreg[j]), sc[t], 0, 0, 0);
        }
        issue_k(PC);   // refill this K buffer with the step after next

        // ---- online softmax, base 2
        const int len = cseg.len;
        const int tok0 = ccur.s * kStep;
        const bool tail = tok0 + kStep > len;
        float sv[8];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) sv[4 * t + e] = sc[t][e] * a.scale_log2;
        if (tail) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (tok0 + 8 * g + i >= len) sv[i] = -INFINITY;
        }
        float mx = sv[0];
#pragma unroll
        for (int i = 1; i < 8; ++i) mx = fmaxf(mx, sv[i]);
        mx = max_xor32(max_xor16(mx));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
        float pv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            pv[i] = __builtin_amdgcn_exp2f(sv[i] - m_new);
            psum += pv[i];
        }
        l_run = l_run * alpha + psum;
        bf16x8 pb;
#pragma unroll
        for (int i = 0; i < 8; ++i) pb[i] = (__bf16)pv[i];

        // ---- stage V (rows past the end of the sequence are zeroed: their P is 0 and 0 * NaN must not leak)
        if (tail) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (tok0 + 4 * i + g >= len) vreg[i] = u32x4{0u, 0u, 0u, 0u};
        }
        lds_order();
#pragma unroll
        for (int i = 0; i < 8; ++i)
            *reinterpret_cast<u32x4*>(lds + (4 * i + g) * kLdsRow + n * 16) = vreg[i];
        lds_order();
        issue_v();     // V of the next step

        if (__any(alpha != 1.f)) {
#pragma unroll
            for (int t = 0; t < 8; ++t) acc[t] *= alpha;
        }
        // ---- O^T += V^T P^T : A operand element i of lane (g, n) is V[token 8 g + i][16 t + n].
        // ds_read_b64_tr_b16: in each group of 16 lanes, lane i points at 4 consecutive elements of
        // row i / 4 (column quad i % 4) and lane l receives column l of those four rows.
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const unsigned char* src = lds + (8 * g + (n >> 2)) * kLdsRow + (16 * t + 4 * (n & 3)) * 2;
            const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(src));
            const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(src + 4 * kLdsRow));
            const i16x8 vt = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vt), pb, acc[t], 0, 0, 0);
        }
        lds_order();

        // ---- next step; at a sequence boundary leave the partial result and switch Q
        const int seg_before = ccur.seg;
        ccur.advance(plan, steps_per_blk);
        if (ccur.seg != seg_before) {
            flush();
            if (ccur.live()) {
                cseg = read_rec(plan, ccur.seg);
#pragma unroll
                for (int j = 0; j < 4; ++j) qreg[j] = qnext[j];
                if (ccur.seg + 1 < nseg)
                    load_q(__builtin_amdgcn_readfirstlane(plan[(ccur.seg + 1) * kPlanInts]), qnext);
            }
        }
    };

    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    issue_k(P0{});
    issue_v();
    issue_k(P1{});
    int i = 0;
    for (; i + 1 < total_steps; i += 2) {
        step(P0{});
        step(P1{});
    }
    if (i < total_steps) step(P0{});
    lds_order();
    if (!kKeep) drain();   // kKeep: a single segment whose partial result stays parked in LDS for the caller
}

// Uniform batch: every sequence has the same number of tokens, known on the host.  A workgroup is
// 8 wavefronts = (8 / parts) KV heads of ONE sequence x `parts` pieces of its steps.  The pieces of a
// head are folded through LDS and the workgroup writes the bf16 result itself: no span plan (the
// block ids are the only load in front of the first K row), no partial result in memory, no merge
// launch.  The price is that a workgroup reads (8 / parts) x 256 B of every token row instead of
// the whole 2 KiB row.
__global__ void __launch_bounds__(512) paged_decode_uniform_kernel(DecodeArgs a, int parts) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_all[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int heads_per_wg = 8 / parts;
    const int wg_per_seq = a.num_kv_heads / heads_per_wg;
    const int b = blockIdx.x / wg_per_seq;
    const int h = (blockIdx.x % wg_per_seq) * heads_per_wg + wave / parts;   // consecutive wavefronts: the pieces of one head
    const int part = wave % parts;
    unsigned char* lds = lds_all + wave * kLdsPerWave;
    int* plan = reinterpret_cast<int*>(lds + kLdsWave);
    unsigned char* defer = lds + kLdsWave + kPlanBytes;
    const int steps_per_blk = a.block_size / kStep;
    const int G = a.group;
    const int g = lane >> 4, n = lane & 15;
    const int len = a.uniform_len < a.max_ctx ? a.uniform_len : a.max_ctx;
    const int nsteps = steps_of(len), share = (nsteps + parts - 1) / parts;
    const int s_lo = part * share, s_hi = s_lo + share < nsteps ? s_lo + share : nsteps;
    if (s_lo < s_hi) {
        const int blk0 = s_lo / steps_per_blk;
        const int nblk = (s_hi - 1) / steps_per_blk - blk0 + 1;
        if (lane == 0) {
            plan[0] = b; plan[1] = len; plan[2] = s_lo; plan[3] = s_hi; plan[4] = 0;
            plan[5] = s_lo - blk0 * steps_per_blk; plan[6] = blk0;
        }
        int tblv = 0;   // lane i = i-th block of this piece (a piece of more than 64 blocks looks the rest up)
        if (lane < nblk) tblv = a.bt[(int64_t)b * a.bt_stride0 + blk0 + lane];
        lds_order();
        run_batch<true>(a, lds, plan, 1, s_hi - s_lo, tblv, h, 0, lane);
    } else if (g == 0 && n < G) {
        // fewer steps than pieces: an empty piece parks an empty (max, sum)
        *reinterpret_cast<float2*>(defer + 512 * G + n * 8) = make_float2(-INFINITY, 0.f);
    }
    __syncthreads();
    if (part != 0 || n >= G) return;
    // piece 0 of every head folds the records of its `parts` pieces (the next wavefronts' LDS areas);
    // lane (g, n) holds head n, columns 16 t + 4 g .. + 3 of accumulator tile t
    const int vlane = g * G + n;
    float m = -INFINITY;
    for (int p = 0; p < parts; ++p)
        m = fmaxf(m, reinterpret_cast<const float2*>(defer + p * kLdsPerWave + 512 * G + n * 8)->x);
    float den = 0.f;
    f32x4 num[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) num[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int p = 0; p < parts; ++p) {
        const unsigned char* r = defer + p * kLdsPerWave;
        const float2 ml = *reinterpret_cast<const float2*>(r + 512 * G + n * 8);
        if (ml.y > 0.f) {
            const float f = __builtin_amdgcn_exp2f(ml.x - m);
            den += ml.y * f;
#pragma unroll
            for (int t = 0; t < 8; ++t) num[t] += *reinterpret_cast<const f32x4*>(r + (vlane * 8 + t) * 16) * f;
        }
    }
    const float inv = den > 0.f ? 1.f / den : 0.f;
    uint16_t* op = a.out + (int64_t)b * a.out_stride0 + (int64_t)(h * G + n) * kD + 4 * g;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        union { __bf16 hv[4]; u32x2 u; } r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r.hv[e] = (__bf16)(num[t][e] * inv);
        *reinterpret_cast<u32x2*>(op + 16 * t) = r.u;
    }
}

__global__ void __launch_bounds__(512) paged_decode_split_kernel(DecodeArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_all[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int waves = blockDim.x >> 6;
    const int h = __builtin_amdgcn_readfirstlane(blockIdx.y * waves + wave);
    const int w = blockIdx.x;
    const int W = gridDim.x;
    unsigned char* lds = lds_all + wave * kLdsPerWave;
    int* plan = reinterpret_cast<int*>(lds + kLdsWave);
    const int steps_per_blk = a.block_size / kStep;

    // total number of steps (the first 64 lengths stay in registers for the second pass)
    const int len0 = lane < a.batch ? ctx_len(a, lane) : 0;
    int total = wave_sum(steps_of(len0));
    for (int c = 64; c < a.batch; c += 64) {
        const int i = c + lane;
        total += wave_sum(i < a.batch ? steps_of(ctx_len(a, i)) : 0);
    }
    total = __builtin_amdgcn_readfirstlane(total);   // wave-uniform: keep the plan in scalar registers

    // Equal shares: the first `rem` workgroups take one step more.  With fewer steps than workgroups
    // every step gets a workgroup of its own: on tiny problems a longer span would only serialise
    // memory latency (measured: one sequence of 512 tokens 14.7 -> 6.7 us).
    //
    // A launch takes as long as its longest span (a sweep over forced span counts on 4907 steps:
    // 102-103 us at 20 steps per workgroup, 104-105 at 22, 108 at 23-24, 113 at 26), so the longest
    // span is made as short as the grid allows, ceil(total / W) steps, and then the fewest workgroups
    // that reach it are used: the shares are as even as whole steps permit (4907 steps, 256
    // workgroups: 246 spans of 19 or 20 steps instead of 42 of 20 and 214 of 19); the workgroups beyond
    // the span count leave at once.
    int spans = W;
    if (total > W) {
        const int longest = (total + W - 1) / W;
        spans = (total + longest - 1) / longest;
    }
    if (w == 0 && h == 0 && lane == 0) {
        a.header[0] = spans;
        a.header[1] = total;
    }
    if (w >= spans) return;
    const int q = total / spans, rem = total - q * spans;
    const int lo = w * q + (w < rem ? w : rem);
    const int hi = lo + q + (w < rem ? 1 : 0);
    if (lo >= hi) return;

    int nseg = 0, nord = 0, nsteps = 0, tblv = 0;
    int running = 0;
    for (int c = 0; c < a.batch; c += 64) {
        const int i = c + lane;
        const int len = c == 0 ? len0 : (i < a.batch ? ctx_len(a, i) : 0);
        const int cnt = steps_of(len);
        const int incl = wave_inclusive_scan(cnt, lane);
        const int start = running + incl - cnt;
        const int end = start + cnt;
        unsigned long long hits = __ballot(cnt > 0 && start < hi && end > lo);
        while (hits) {
            const int bit = __builtin_ctzll(hits);
            hits &= hits - 1;
            const int st = __builtin_amdgcn_readlane(start, bit);
            const int en = __builtin_amdgcn_readlane(end, bit);
            const int ln = __builtin_amdgcn_readlane(len, bit);
            const int s_lo = (st > lo ? st : lo) - st;
            const int s_hi = (en < hi ? en : hi) - st;
            const int b = c + bit;
            if (h == 0 && lane == 0) {
                if (s_lo == 0) a.seg_first[b] = w;
                if (s_hi == en - st) a.seg_last[b] = w;
            }
            const int blk0 = s_lo / steps_per_blk;
            const int nblk = (s_hi - 1) / steps_per_blk - blk0 + 1;
            if (nseg == kMaxSegs || (nseg > 0 && nord + nblk > 64)) {
                lds_order();
                run_batch(a, lds, plan, nseg, nsteps, tblv, h, w, lane);
                lds_order();
                nseg = nord = nsteps = 0;
                tblv = 0;
            }
            if (lane == 0) {
                int* p = plan + nseg * kPlanInts;
                p[0] = b; p[1] = ln; p[2] = s_lo; p[3] = s_hi; p[4] = nord; p[5] = s_lo - blk0 * steps_per_blk; p[6] = blk0;
            }
            {   // gather this segment's block ids into lanes [nord, nord + nblk)
                const int k = lane - nord;
                if (k >= 0 && k < nblk && lane < 64) tblv = a.bt[(int64_t)b * a.bt_stride0 + blk0 + k];
            }
            ++nseg;
            nord += nblk;
            nsteps += s_hi - s_lo;
        }
        running += __builtin_amdgcn_readlane(incl, 63);
        if (running >= hi) break;
    }
    if (nseg > 0) {
        lds_order();
        run_batch(a, lds, plan, nseg, nsteps, tblv, h, w, lane);
    }
}

struct MergeArgs {
    uint16_t* out;
    int64_t out_stride0;
    const int32_t* ctx;     // nullptr: every sequence has uniform_len tokens
    int uniform_len;
    int group;
    int slots_per_head;     // records per KV head in the workspace, as in the split launch
    const int32_t* seg_first;
    const int32_t* seg_last;
    const unsigned char* rec;
    int rec_stride;
    int batch;
};

// grid (batch, Hq), 256 threads = 8 segment lanes x 32 column quads.  Thread (j, c) folds segments
// j, j + 8, ... of its (sequence, query head) for output columns 4c .. 4c+3 with the running
// (max, sum) rule; the eight lanes are then folded through LDS.  All loads of a thread are
// independent, so a sequence cut into many segments costs about one memory round trip.
__global__ void __launch_bounds__(256) paged_decode_merge_kernel(MergeArgs a) {
    __shared__ float red[8][32][6];
    const int b = blockIdx.x;
    const int head = blockIdx.y;
    const int G = a.group;
    const int h = head / G, n = head - h * G;
    const int j = threadIdx.x >> 5, c4 = threadIdx.x & 31;
    uint16_t* op = a.out + (int64_t)b * a.out_stride0 + (int64_t)head * kD + 4 * c4;
    if ((a.ctx ? a.ctx[b] : a.uniform_len) <= 0) {
        if (j == 0) *reinterpret_cast<u32x2*>(op) = u32x2{0u, 0u};
        return;
    }
    const int w0 = a.seg_first[b], w1 = a.seg_last[b];
    const int64_t slot0 = (int64_t)h * a.slots_per_head + b;
    float m = -INFINITY, den = 0.f;
    f32x4 num = {0.f, 0.f, 0.f, 0.f};
    for (int wb = w0 + j; wb <= w1; wb += 32) {
        float2 mlv[4];
        f32x4 pov[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int wu = wb + 8 * u <= w1 ? wb + 8 * u : wb;
            // columns 4 c4 .. 4 c4 + 3 = accumulator tile t = c4 / 4 of lane group g = c4 % 4
            const unsigned char* rec = a.rec + (slot0 + wu) * a.rec_stride;
            mlv[u] = *reinterpret_cast<const float2*>(rec + 512 * G + n * 8);
            pov[u] = *reinterpret_cast<const f32x4*>(rec + (((c4 & 3) * G + n) * 8 + (c4 >> 2)) * 16);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (wb + 8 * u > w1) break;
            const float m_new = fmaxf(m, mlv[u].x);
            const float f_old = __builtin_amdgcn_exp2f(m - m_new);
            const float f_new = __builtin_amdgcn_exp2f(mlv[u].x - m_new);
            den = den * f_old + mlv[u].y * f_new;
            num = num * f_old + pov[u] * f_new;
            m = m_new;
        }
    }
    red[j][c4][0] = m; red[j][c4][1] = den;
    red[j][c4][2] = num[0]; red[j][c4][3] = num[1]; red[j][c4][4] = num[2]; red[j][c4][5] = num[3];
    __syncthreads();
    if (j == 0) {
        float mx = m;
#pragma unroll
        for (int k = 1; k < 8; ++k) mx = fmaxf(mx, red[k][c4][0]);
        float d_tot = 0.f;
        f32x4 n_tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float mk = red[k][c4][0];
            const float f = mk == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mk - mx);
            d_tot += red[k][c4][1] * f;
            n_tot += f32x4{red[k][c4][2], red[k][c4][3], red[k][c4][4], red[k][c4][5]} * f;
        }
        const float inv = d_tot > 0.f ? 1.f / d_tot : 0.f;
        union { __bf16 hv[4]; u32x2 u; } r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r.hv[e] = (__bf16)(n_tot[e] * inv);
        *reinterpret_cast<u32x2*>(op) = r.u;
    }
}

constexpr int kMaxDevices = 64;

int current_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
    return dev;
}

// Compute units of the current device (cached per device; a benign race writes the same value).
int device_cu_count() {
    static int cus[kMaxDevices] = {0};
    const int dev = current_device();
    if (cus[dev] == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) return 256;
        cus[dev] = v;
    }
    return cus[dev];
}

struct Launch {
    int waves;      // wavefronts (KV heads) per workgroup
    int grid_y;
    int W;          // workgroups along the KV-split axis
};

// split_workgroups: 0 = two wavefronts per SIMD over the whole chip, else the caller's count.
int plan_launch(int64_t hkv, int64_t split_workgroups, Launch* out) {
    if (hkv <= 0 || split_workgroups < 0) return INFER_KV_EINVAL;
    int waves;
    if (hkv <= 8) waves = (int)hkv;
    else if (hkv % 8 == 0) waves = 8;
    else return INFER_KV_EUNSUPPORTED;
    int64_t W = split_workgroups;
    if (W == 0) {
        W = device_cu_count() * 8 / hkv;
        if (W < 1) W = 1;
    }
    if (W > INFER_KV_MAX_SPLIT_WG) W = INFER_KV_MAX_SPLIT_WG;
    out->waves = waves;
    out->grid_y = (int)(hkv / waves);
    out->W = (int)W;
    return INFER_KV_OK;
}

int check_shape(int64_t batch, int64_t hq, int64_t hkv, int64_t d, int64_t bs, int64_t nblk, int64_t table_cols) {
    if (batch <= 0 || hq <= 0 || hkv <= 0 || nblk <= 0 || bs <= 0 || table_cols <= 0) return INFER_KV_EINVAL;
    if (batch > (1 << 20)) return INFER_KV_EINVAL;
    if (d != kD) return INFER_KV_EUNSUPPORTED;
    if (hq % hkv != 0 || hq / hkv > 16) return INFER_KV_EUNSUPPORTED;
    if (bs % kStep != 0) return INFER_KV_EUNSUPPORTED;
    // the step count of the whole batch is summed in 32 bits
    const int64_t max_ctx = table_cols * bs;
    if (bs > (1 << 24) || table_cols > (1 << 24) || batch * ((max_ctx + kStep - 1) / kStep) > 0x7fffffffLL)
        return INFER_KV_EINVAL;
    return INFER_KV_OK;
}

struct DecodeCall {
    const void* q; int64_t q_stride0;
    const void* k_cache; const void* v_cache;
    int64_t cache_block_stride, cache_token_stride;
    const int32_t* block_table; int64_t bt_stride0, table_cols;
    const int32_t* context_lens;   // nullptr: every sequence has uniform_len tokens
    int64_t batch, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks;
    float scale;
    int64_t uniform_len = 0;
};

// Checks every argument of the split phase and fills in the launch shape.
int check_split(const DecodeCall& c, int64_t split_workgroups, const void* workspace, Launch* L) {
    if (!c.q || !c.k_cache || !c.v_cache || !c.block_table || !workspace) return INFER_KV_EINVAL;
    int rc = check_shape(c.batch, c.num_q_heads, c.num_kv_heads, c.head_dim, c.block_size, c.num_blocks, c.table_cols);
    if (rc) return rc;
    // 16-byte vector loads: every row start must be 16-byte aligned.
    if (((uintptr_t)c.q | (uintptr_t)c.k_cache | (uintptr_t)c.v_cache | (uintptr_t)workspace) & 15) return INFER_KV_EALIGN;
    if ((c.q_stride0 | c.cache_block_stride | c.cache_token_stride) & 7) return INFER_KV_EALIGN;
    if (c.cache_token_stride < c.num_kv_heads * kD || c.cache_block_stride < c.block_size * c.cache_token_stride)
        return INFER_KV_EINVAL;
    if (c.batch > 1 && c.bt_stride0 < c.table_cols) return INFER_KV_EINVAL;
    // lane offsets inside one step are kept in 32 bits
    if (32 * c.cache_token_stride >= (int64_t)1 << 31) return INFER_KV_EINVAL;
    return plan_launch(c.num_kv_heads, split_workgroups, L);
}

int check_out(const void* out, int64_t out_stride0, int64_t num_q_heads) {
    if (!out || out_stride0 < num_q_heads * kD) return INFER_KV_EINVAL;
    // 8-byte stores of four outputs
    if (((uintptr_t)out & 7) || (out_stride0 & 3)) return INFER_KV_EALIGN;
    return INFER_KV_OK;
}

// Enqueues the split kernel; `base` is device memory laid out as `ws` (arguments already checked).
int launch_split(const DecodeCall& c, const Launch& L, const DecodeWorkspace& ws, void* base_v, hipStream_t stream) {
    DecodeArgs a;
    a.q = (const uint16_t*)c.q;
    a.q_stride0 = c.q_stride0;
    a.k = (const uint16_t*)c.k_cache;
    a.v = (const uint16_t*)c.v_cache;
    a.blk_stride = c.cache_block_stride;
    a.tok_stride = c.cache_token_stride;
    a.bt = c.block_table;
    a.bt_stride0 = c.bt_stride0;
    a.ctx = c.context_lens;
    a.uniform_len = c.uniform_len > 0x7fffffffLL ? 0x7fffffff : (c.uniform_len < 0 ? 0 : (int)c.uniform_len);
    a.out = nullptr;
    a.out_stride0 = 0;
    const int64_t max_ctx = c.table_cols * c.block_size;
    a.max_ctx = max_ctx > 0x7fffffffLL ? 0x7fffffff : (int)max_ctx;
    a.batch = (int)c.batch;
    a.group = (int)(c.num_q_heads / c.num_kv_heads);
    a.num_kv_heads = (int)c.num_kv_heads;
    a.block_size = (int)c.block_size;
    a.num_blocks = (int)c.num_blocks;
    a.scale_log2 = c.scale * 1.4426950408889634f;
    char* base = (char*)base_v;
    a.header = (int32_t*)(base + ws.header_off);
    a.seg_first = (int32_t*)(base + ws.seg_first_off);
    a.seg_last = (int32_t*)(base + ws.seg_last_off);
    a.rec = (unsigned char*)base + ws.rec_off;
    a.rec_stride = (int)ws.rec_stride;
    a.slots_per_head = (int)ws.slots_per_head;

    const size_t lds_bytes = (size_t)L.waves * kLdsPerWave;
    static bool attr_set[kMaxDevices] = {false};   // the attribute is per device
    const int dev = current_device();
    if (!attr_set[dev]) {
        hipError_t e = hipFuncSetAttribute((const void*)paged_decode_split_kernel,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 8 * kLdsPerWave);
        if (e != hipSuccess) return (int)e;
        attr_set[dev] = true;
    }
    dim3 grid(L.W, L.grid_y, 1), block(64 * L.waves, 1, 1);
    hipLaunchKernelGGL(paged_decode_split_kernel, grid, block, lds_bytes, stream, a);
    return (int)hipGetLastError();
}

// Pieces per KV head for the uniform kernel, or 0 when the span kernel serves the shape better.  The
// uniform kernel holds one 8-wavefront workgroup per compute unit (its LDS), so it is used when
// batch x KV heads x pieces / 8 workgroups fill the chip in one round with even pieces.
int uniform_parts(const DecodeCall& c) {
    if (c.uniform_len <= 0 || c.num_kv_heads > (1 << 16)) return 0;
    const int64_t cus = device_cu_count();
    const int64_t len = c.uniform_len < c.table_cols * c.block_size ? c.uniform_len : c.table_cols * c.block_size;
    const int64_t steps = (len + kStep - 1) / kStep;
    for (int parts = 8; parts >= 1; parts >>= 1) {
        const int heads_per_wg = 8 / parts;
        if (c.num_kv_heads % heads_per_wg != 0) continue;
        const int64_t wgs = c.batch * (c.num_kv_heads / heads_per_wg);
        if (wgs > cus) continue;
        if (wgs * 5 < cus * 4) return 0;                        // the largest fit leaves a fifth of the chip idle
        const int64_t share = (steps + parts - 1) / parts;
        return steps * 20 >= share * parts * 17 ? parts : 0;    // pieces at least 85 % even
    }
    return 0;
}

int launch_uniform(const DecodeCall& c, void* out, int64_t out_stride0, int parts, hipStream_t stream) {
    DecodeArgs a{};
    a.q = (const uint16_t*)c.q;
    a.q_stride0 = c.q_stride0;
    a.k = (const uint16_t*)c.k_cache;
    a.v = (const uint16_t*)c.v_cache;
    a.blk_stride = c.cache_block_stride;
    a.tok_stride = c.cache_token_stride;
    a.bt = c.block_table;
    a.bt_stride0 = c.bt_stride0;
    a.ctx = nullptr;
    a.uniform_len = c.uniform_len > 0x7fffffffLL ? 0x7fffffff : (int)c.uniform_len;
    const int64_t max_ctx = c.table_cols * c.block_size;
    a.max_ctx = max_ctx > 0x7fffffffLL ? 0x7fffffff : (int)max_ctx;
    a.batch = (int)c.batch;
    a.group = (int)(c.num_q_heads / c.num_kv_heads);
    a.num_kv_heads = (int)c.num_kv_heads;
    a.block_size = (int)c.block_size;
    a.num_blocks = (int)c.num_blocks;
    a.scale_log2 = c.scale * 1.4426950408889634f;
    a.rec_stride = (int)decode_record_bytes(a.group);   // layout of a parked partial result
    a.out = (uint16_t*)out;
    a.out_stride0 = out_stride0;
    static bool attr_set[kMaxDevices] = {false};   // the attribute is per device
    const int dev = current_device();
    if (!attr_set[dev]) {
        hipError_t e = hipFuncSetAttribute((const void*)paged_decode_uniform_kernel,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 8 * kLdsPerWave);
        if (e != hipSuccess) return (int)e;
        attr_set[dev] = true;
    }
    const unsigned wgs = (unsigned)(c.batch * (c.num_kv_heads / (8 / parts)));
    hipLaunchKernelGGL(paged_decode_uniform_kernel, dim3(wgs, 1, 1), dim3(512, 1, 1), 8 * kLdsPerWave, stream, a, parts);
    return (int)hipGetLastError();
}

int launch_merge(void* out, int64_t out_stride0, const int32_t* context_lens, int64_t uniform_len, int64_t batch,
                 int64_t num_q_heads, int64_t num_kv_heads, const DecodeWorkspace& ws, const void* base_v,
                 hipStream_t stream) {
    const char* base = (const char*)base_v;
    MergeArgs m;
    m.out = (uint16_t*)out;
    m.out_stride0 = out_stride0;
    m.ctx = context_lens;
    m.uniform_len = uniform_len > 0 ? 1 : 0;   // only its sign matters here
    m.group = (int)(num_q_heads / num_kv_heads);
    m.slots_per_head = (int)ws.slots_per_head;
    m.seg_first = (const int32_t*)(base + ws.seg_first_off);
    m.seg_last = (const int32_t*)(base + ws.seg_last_off);
    m.rec = (const unsigned char*)base + ws.rec_off;
    m.rec_stride = (int)ws.rec_stride;
    m.batch = (int)batch;
    dim3 grid((unsigned)batch, (unsigned)num_q_heads, 1), block(256, 1, 1);
    hipLaunchKernelGGL(paged_decode_merge_kernel, grid, block, 0, stream, m);
    return (int)hipGetLastError();
}

}  // namespace

// Scratch of infer_paged_decode_noalloc_bf16: the split-KV partial results of one call.  Every device
// the library runs on holds its own copy of this array, at its own address, until the process ends.
// In host code the array's NAME is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t kNoAllocScratchBytes = INFER_KV_DECODE_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char infer_kv_decode_scratch[kNoAllocScratchBytes];

namespace {

// Device address of the scratch array on the current device, resolved once per device.
int noalloc_scratch(void** out) {
    static void* ptrs[kMaxDevices] = {nullptr};
    static bool known[kMaxDevices] = {false};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return INFER_KV_EUNSUPPORTED;
    if (!__atomic_load_n(&known[dev], __ATOMIC_ACQUIRE)) {      // a race between two first calls resolves the same address twice
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(infer_kv_decode_scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return INFER_KV_EINVAL;
        ptrs[dev] = p;
        __atomic_store_n(&known[dev], true, __ATOMIC_RELEASE);
    }
    *out = ptrs[dev];
    return INFER_KV_OK;
}

}  // namespace

extern "C" {

size_t infer_paged_decode_workspace_bytes(int64_t max_batch, int64_t num_q_heads, int64_t num_kv_heads,
                                          int64_t head_dim) {
    if (max_batch <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim != kD) return 0;
    if (num_q_heads % num_kv_heads != 0) return 0;
    DecodeWorkspace ws = decode_workspace_layout(max_batch, num_q_heads / num_kv_heads, num_kv_heads);
    return ws.total_bytes;
}

int infer_paged_decode_split_bf16(const void* q, int64_t q_stride0, const void* k_cache, const void* v_cache,
                                  int64_t cache_block_stride, int64_t cache_token_stride,
                                  const int32_t* block_table, int64_t bt_stride0, int64_t table_cols,
                                  const int32_t* context_lens, int64_t batch, int64_t num_q_heads,
                                  int64_t num_kv_heads, int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                  float scale, int64_t split_workgroups, void* workspace, size_t workspace_bytes,
                                  void* stream) {
    const DecodeCall c{q, q_stride0, k_cache, v_cache, cache_block_stride, cache_token_stride, block_table, bt_stride0,
                       table_cols, context_lens, batch, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks,
                       scale};
    if (!context_lens) return INFER_KV_EINVAL;
    Launch L;
    int rc = check_split(c, split_workgroups, workspace, &L);
    if (rc) return rc;
    const DecodeWorkspace ws = decode_workspace_layout(batch, num_q_heads / num_kv_heads, num_kv_heads);
    if (ws.total_bytes > workspace_bytes) return INFER_KV_EWORKSPACE;
    return launch_split(c, L, ws, workspace, (hipStream_t)stream);
}

int infer_paged_decode_merge_bf16(void* out, int64_t out_stride0, const int32_t* context_lens, int64_t batch,
                                  int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                                  const void* workspace, size_t workspace_bytes, void* stream) {
    if (!out || !context_lens || !workspace) return INFER_KV_EINVAL;
    if (batch <= 0 || batch > (1 << 20) || num_q_heads <= 0 || num_kv_heads <= 0) return INFER_KV_EINVAL;
    if (head_dim != kD) return INFER_KV_EUNSUPPORTED;
    if (num_q_heads % num_kv_heads != 0 || num_q_heads / num_kv_heads > 16) return INFER_KV_EUNSUPPORTED;
    int rc = check_out(out, out_stride0, num_q_heads);
    if (rc) return rc;
    if ((uintptr_t)workspace & 15) return INFER_KV_EALIGN;   // 16-byte loads of the records
    const DecodeWorkspace ws = decode_workspace_layout(batch, num_q_heads / num_kv_heads, num_kv_heads);
    if (ws.total_bytes > workspace_bytes) return INFER_KV_EWORKSPACE;
    return launch_merge(out, out_stride0, context_lens, 0, batch, num_q_heads, num_kv_heads, ws, workspace,
                        (hipStream_t)stream);
}

int infer_paged_decode_bf16(const void* q, int64_t q_stride0, const void* k_cache, const void* v_cache,
                            int64_t cache_block_stride, int64_t cache_token_stride, void* out,
                            int64_t out_stride0, const int32_t* block_table, int64_t bt_stride0, int64_t table_cols,
                            const int32_t* context_lens, int64_t batch, int64_t num_q_heads,
                            int64_t num_kv_heads, int64_t head_dim, int64_t block_size, int64_t num_blocks,
                            float scale, int64_t split_workgroups, void* workspace, size_t workspace_bytes,
                            void* stream) {
    const DecodeCall c{q, q_stride0, k_cache, v_cache, cache_block_stride, cache_token_stride, block_table, bt_stride0,
                       table_cols, context_lens, batch, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks,
                       scale};
    // everything is checked before the first launch is enqueued
    if (!context_lens) return INFER_KV_EINVAL;
    Launch L;
    int rc = check_split(c, split_workgroups, workspace, &L);
    if (rc) return rc;
    rc = check_out(out, out_stride0, num_q_heads);
    if (rc) return rc;
    const DecodeWorkspace ws = decode_workspace_layout(batch, num_q_heads / num_kv_heads, num_kv_heads);
    if (ws.total_bytes > workspace_bytes) return INFER_KV_EWORKSPACE;
    rc = launch_split(c, L, ws, workspace, (hipStream_t)stream);
    if (rc) return rc;
    return launch_merge(out, out_stride0, context_lens, 0, batch, num_q_heads, num_kv_heads, ws, workspace,
                        (hipStream_t)stream);
}

int infer_paged_decode_uniform_bf16(const void* q, int64_t q_stride0, const void* k_cache, const void* v_cache,
                                    int64_t cache_block_stride, int64_t cache_token_stride, void* out,
                                    int64_t out_stride0, const int32_t* block_table, int64_t bt_stride0,
                                    int64_t table_cols, int64_t context_len, int64_t batch, int64_t num_q_heads,
                                    int64_t num_kv_heads, int64_t head_dim, int64_t block_size, int64_t num_blocks,
                                    float scale, void* workspace, size_t workspace_bytes, void* stream) {
    DecodeCall c{q, q_stride0, k_cache, v_cache, cache_block_stride, cache_token_stride, block_table, bt_stride0,
                 table_cols, nullptr, batch, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, scale};
    c.uniform_len = context_len;
    if (context_len < 0 || context_len > 0x7fffffffLL) return INFER_KV_EINVAL;
    Launch L;
    int rc = check_split(c, /*split_workgroups=*/0, workspace, &L);
    if (rc) return rc;
    rc = check_out(out, out_stride0, num_q_heads);
    if (rc) return rc;
    const DecodeWorkspace ws = decode_workspace_layout(batch, num_q_heads / num_kv_heads, num_kv_heads);
    if (ws.total_bytes > workspace_bytes) return INFER_KV_EWORKSPACE;
    if (const int parts = uniform_parts(c)) return launch_uniform(c, out, out_stride0, parts, (hipStream_t)stream);
    // shapes the uniform kernel does not fill the chip with: equal spans + merge, without a lengths array
    rc = launch_split(c, L, ws, workspace, (hipStream_t)stream);
    if (rc) return rc;
    return launch_merge(out, out_stride0, nullptr, context_len, batch, num_q_heads, num_kv_heads, ws, workspace,
                        (hipStream_t)stream);
}

int infer_paged_decode_noalloc_bf16(const void* q, int64_t q_stride0, const void* k_cache, const void* v_cache,
                                    int64_t cache_block_stride, int64_t cache_token_stride, void* out,
                                    int64_t out_stride0, const int32_t* block_table, int64_t bt_stride0,
                                    int64_t table_cols, const int32_t* context_lens, int64_t batch,
                                    int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                                    int64_t num_blocks, float scale, void* stream) {
    const DecodeCall c{q, q_stride0, k_cache, v_cache, cache_block_stride, cache_token_stride, block_table, bt_stride0,
                       table_cols, context_lens, batch, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks,
                       scale};
    if (!context_lens) return INFER_KV_EINVAL;
    void* scratch = nullptr;
    int rc = noalloc_scratch(&scratch);
    if (rc) return rc;
    Launch L;
    rc = check_split(c, /*split_workgroups=*/0, scratch, &L);
    if (rc) return rc;
    rc = check_out(out, out_stride0, num_q_heads);
    if (rc) return rc;
    // laid out for the split count this call launches, not for the largest one a workspace allows
    const DecodeWorkspace ws = decode_workspace_layout(batch, num_q_heads / num_kv_heads, num_kv_heads, L.W);
    if (ws.total_bytes > kNoAllocScratchBytes) return INFER_KV_EWORKSPACE;
    rc = launch_split(c, L, ws, scratch, (hipStream_t)stream);
    if (rc) return rc;
    return launch_merge(out, out_stride0, context_lens, 0, batch, num_q_heads, num_kv_heads, ws, scratch,
                        (hipStream_t)stream);
}

}  // extern "C"
