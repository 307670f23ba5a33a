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
//   block_size % 32 == 0).  All steps of all sequences are laid end to end and cut into spans of
//   equal length (to within one step), one per wavefront.  A workgroup is 8 wavefronts: `parts`
//   consecutive spans for each of 8 / parts KV heads, every wavefront with a private pipeline (no
//   workgroup barrier while the cache is streamed).  A span may cover the tail of one sequence and
//   the head of the next: each (sequence, span) piece is a "segment" and leaves a partial result
//   parked in LDS.  After ONE barrier the segments of a sequence that lie in the same workgroup are
//   folded through LDS ("chain") and leave one record in the workspace; the merge kernel folds the
//   records of a sequence that reaches into neighbouring workgroups and writes the bf16 result.  When
//   the host knows that every sequence lies inside one workgroup (one length for the whole batch that
//   fits the span grid) the chains are whole sequences: the workgroups write the result themselves
//   and there is no second launch.
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
    unsigned char* rec; // [slots] partial-result records (layout: decode_record_bytes): pieces kFirstPieces and later of a sequence
    unsigned char* rec_first; // [batch][KV head][kFirstPieces] records: the first pieces of every sequence, at places the merge kernel knows in advance
    int rec_stride;
    int slots_per_head; // records per KV head in the workspace (layout constant, >= wg_spans + batch)
    uint16_t* out;      // [batch, Hq, D] result (only when the workgroups write it themselves)
    int64_t out_stride0;
    int parts;          // wavefronts (consecutive spans) per KV head in a workgroup: 1, 2, 4 or 8
    int head_groups;    // workgroups per span position = num_kv_heads / (8 / parts)
    int wg_spans;       // span positions of the launch; the grid is wg_spans * head_groups workgroups
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
    // the halves go through scalars of their own: a bit cast applied to `r[1]` itself reads element 0
    const unsigned lo = r[0], hi = r[1];
    float m;   // written out: fmaxf would first quiet a NaN in each operand, two more instructions
    __asm__("v_max_f32_e32 %0, %1, %2" : "=v"(m) : "v"(lo), "v"(hi));
    return m;
}
__device__ __forceinline__ float max_xor32(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    // the halves go through scalars of their own: a bit cast applied to `r[1]` itself reads element 0
    const unsigned lo = r[0], hi = r[1];
    float m;   // written out: fmaxf would first quiet a NaN in each operand, two more instructions
    __asm__("v_max_f32_e32 %0, %1, %2" : "=v"(m) : "v"(lo), "v"(hi));
    return m;
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
// Partial results wait in LDS until the wavefront has issued its last load: a global store in the
// middle of the stream would make the outstanding-load counter unordered (loads and stores share
// it) and force a full drain of the prefetch pipeline.  The area holds one record (the span's first
// segment when its sequence began in an earlier span or goes on in a later one) and behind it a few
// results of sequences that lie wholly inside the span.
constexpr int kDeferBytes = 8448;
// Per wavefront: what its span left for the fold after the barrier.
//   ints 0..3  first segment {sequence, flags, position of the sequence's first step on the step axis}
//   ints 4..7  last segment (only when it is not also the first), same fields
//   ints 8..15 sequences of the finished results waiting behind the record
constexpr int kExitBytes = 64;
constexpr int kLdsPerWave = kLdsWave + kPlanBytes + kDeferBytes + kExitBytes;
constexpr int kExitValid = 1, kExitLeft = 2, kExitRight = 4;   // flags: entry in use; sequence has earlier / later steps
constexpr int kMaxRing = 8;
constexpr int kFirstPieces = INFER_KV_DECODE_FIRST_PIECES;

struct SegRec {      // one record of the plan, all wave-uniform
    int b;           // sequence
    int len;         // its context length
    int s_lo, s_hi;  // steps of the sequence covered by this span
    int ord0;        // block ordinal of the first step's block
    int in0;         // step index of s_lo inside its block
    int blk0;        // index of that block in the sequence's table row
    int st;          // position of the sequence's first step on the step axis
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
    r.st = __builtin_amdgcn_readfirstlane(p[7]);
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

// A partial result as one wavefront holds it: lane (g, n), n < G, has columns 16 t + 4 g .. + 3 of
// query head n in acc[t] (unnormalised), m = running maximum (log2 domain), l = sum, both per head.
struct Partial {
    f32x4 acc[8];
    float m, l;
};

// (vlane * 8 + t) * 16 is the place of acc[t] in a record, 512 G + 8 n the place of (m, l): the layout
// of decode_record_bytes().  The same code parks a record in LDS and stores it to the workspace.
__device__ __forceinline__ void put_record(unsigned char* dst, const Partial& r, int G, int g, int n) {
    if (n < G) {
        const int vlane = g * G + n;
#pragma unroll
        for (int t = 0; t < 8; ++t) *reinterpret_cast<f32x4*>(dst + (vlane * 8 + t) * 16) = r.acc[t];
        if (g == 0) *reinterpret_cast<float2*>(dst + 512 * G + n * 8) = make_float2(r.m, r.l);
    }
}
__device__ __forceinline__ void get_record(const unsigned char* src, Partial& r, int G, int g, int n) {
    const int nn = n < G ? n : 0;   // lanes without a head read head 0's values and never store
    const int vlane = g * G + nn;
#pragma unroll
    for (int t = 0; t < 8; ++t) r.acc[t] = *reinterpret_cast<const f32x4*>(src + (vlane * 8 + t) * 16);
    const float2 ml = *reinterpret_cast<const float2*>(src + 512 * G + nn * 8);
    r.m = ml.x;
    r.l = ml.y;
}

// into <- into (+) other: the (max, sum) rule of the reference's softmax reduction (softmax.cu:5-16).
__device__ __forceinline__ void fold(Partial& into, const Partial& other) {
    const float mn = fmaxf(into.m, other.m);
    const float f1 = into.m == mn ? 1.f : __builtin_amdgcn_exp2f(into.m - mn);
    const float f2 = other.m == mn ? 1.f : __builtin_amdgcn_exp2f(other.m - mn);
#pragma unroll
    for (int t = 0; t < 8; ++t) into.acc[t] = into.acc[t] * f1 + other.acc[t] * f2;
    into.l = into.l * f1 + other.l * f2;
    into.m = mn;
}

// out[b, h G + n, 16 t + 4 g .. + 3] = acc[t] / l as bf16: four outputs = one 8-byte value per tile.
__device__ __forceinline__ u32x2 pack_out(const f32x4& v, float inv) {
    union { __bf16 hv[4]; u32x2 u; } r;
#pragma unroll
    for (int e = 0; e < 4; ++e) r.hv[e] = (__bf16)(v[e] * inv);
    return r.u;
}
__device__ __forceinline__ void store_out(const DecodeArgs& a, int b, int h, const Partial& r, int G, int g, int n) {
    if (n < G) {
        const float inv = r.l > 0.f ? 1.f / r.l : 0.f;
        uint16_t* op = a.out + (int64_t)b * a.out_stride0 + (int64_t)(h * G + n) * kD + 4 * g;
#pragma unroll
        for (int t = 0; t < 8; ++t) *reinterpret_cast<u32x2*>(op + 16 * t) = pack_out(r.acc[t], inv);
    }
}

// What a wavefront carries from one batch of segments to the next and to the fold after the barrier.
struct WaveTail {
    int flushed;   // segments finished so far
    int nring;     // finished results waiting in LDS
};

// Geometry of one wavefront's place in the launch.
struct WavePlace {
    int h;       // KV head
    int s;       // span position of the workgroup (index of its records in the workspace)
    int lane;
};

// Where the record of (sequence b, KV head h) from the workgroup at span position s goes: the sequence's
// piece number is s minus the span position of its first step; the first kFirstPieces pieces have fixed
// places (the merge kernel requests them before it knows how many there are), later ones the slot
// h * slots_per_head + s + b, unique because consecutive chains advance s or b.
__device__ __forceinline__ unsigned char* record_place(const DecodeArgs& a, int b, int h, int s, int s_first) {
    const int k = s - s_first;
    if (k < kFirstPieces) return a.rec_first + (((int64_t)b * a.num_kv_heads + h) * kFirstPieces + k) * a.rec_stride;
    return a.rec + ((int64_t)h * a.slots_per_head + s + b) * a.rec_stride;
}

// Writes out the finished results parked behind the record.  kRecords: they are records for the merge
// kernel (slot = the workgroup's span position + sequence); otherwise bf16 rows of `out`.
template <bool kRecords>
__device__ __forceinline__ void drain_ring(const DecodeArgs& a, unsigned char* lds, const WavePlace& wp, WaveTail& wt) {
    const int G = a.group, g = wp.lane >> 4, n = wp.lane & 15;
    const unsigned char* ring = lds + kLdsWave + kPlanBytes + a.rec_stride;
    const int* exitT = reinterpret_cast<const int*>(lds + kLdsWave + kPlanBytes + kDeferBytes);
    for (int k = 0; k < wt.nring; ++k) {
        const int b = __builtin_amdgcn_readfirstlane(exitT[8 + k]);
        if (kRecords) {
            // the record leaves as it was parked: all 64 lanes, 16 B each, one contiguous run
            const unsigned char* src = ring + k * a.rec_stride;
            unsigned char* dst = record_place(a, b, wp.h, 0, 0);   // a whole sequence: its only piece
            for (int off = wp.lane * 16; off < a.rec_stride; off += 1024)
                *reinterpret_cast<u32x4*>(dst + off) = *reinterpret_cast<const u32x4*>(src + off);
        } else if (n < G) {
            const unsigned char* src = ring + k * (G * 256) + (g * G + n) * 64;
            uint16_t* op = a.out + (int64_t)b * a.out_stride0 + (int64_t)(wp.h * G + n) * kD + 4 * g;
#pragma unroll
            for (int t = 0; t < 8; ++t) *reinterpret_cast<u32x2*>(op + 16 * t) = *reinterpret_cast<const u32x2*>(src + 8 * t);
        }
    }
    wt.nring = 0;
}

// Runs one batch of segments for KV head h.
//
// Software pipeline (loads return in issue order, so the waits are exact counts): K fragments are
// double-buffered in registers, V rows single-buffered; while step i is being reduced, K(i+1),
// then K(i+2) and V(i+1) are in flight, across sequence boundaries.  Loads past the end of the
// batch are redirected to one dummy 16-byte location instead of being skipped, which keeps the
// number of outstanding loads at every wait independent of control flow.
template <bool kRecords>
__device__ __forceinline__ void run_batch(const DecodeArgs& a, unsigned char* lds, const int* plan, int nseg,
                                          int total_steps, int tblv_loaded, const WavePlace& wp, WaveTail& wt) {
    // The block ids were gathered by vector loads.  Hand them to the loop as a plain register value:
    // otherwise every later read of this register is treated as "may still be in flight" and gets a
    // wait that also drains the K/V loads issued since, which defeats the pipeline.
    int tblv;
    __asm__ volatile("v_mov_b32 %0, %1" : "=v"(tblv) : "v"(tblv_loaded));
    const int lane = wp.lane, h = wp.h;
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

    Partial cur;
#pragma unroll
    for (int t = 0; t < 8; ++t) cur.acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    cur.m = -INFINITY;
    cur.l = 0.f;

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

    unsigned char* defer = lds + kLdsWave + kPlanBytes;
    int* exitT = reinterpret_cast<int*>(defer + kDeferBytes);
    // results of sequences that lie wholly inside the span wait behind the record: as records for the
    // merge kernel (kRecords) or already as the bf16 rows of `out`
    const int ring_entry = kRecords ? a.rec_stride : G * 256;
    const int ring_room = (kDeferBytes - a.rec_stride) / ring_entry;
    const int ring_cap = ring_room < kMaxRing ? ring_room : kMaxRing;   // 0 at group size 16 (and 8 for records)

    // The segment just finished leaves its partial result; the accumulators start over.
    auto flush = [&]() {
        float l_tot = cur.l + __shfl_xor(cur.l, 16);
        l_tot += __shfl_xor(l_tot, 32);
        cur.l = l_tot;
        const bool left = cseg.s_lo > 0;
        const bool right = cseg.s_hi < steps_of(cseg.len);
        const int flags = kExitValid | (left ? kExitLeft : 0) | (right ? kExitRight : 0);
        lds_order();
        if (wt.flushed == 0 && (left || right)) {
            put_record(defer, cur, G, g, n);
            if (lane == 0) { exitT[0] = cseg.b; exitT[1] = flags; exitT[2] = cseg.st; }
        } else if (right) {
            // the span's last segment, and not its first: its steps were the last to use the V tile
            put_record(lds, cur, G, g, n);
            if (lane == 0) { exitT[4] = cseg.b; exitT[5] = flags; exitT[6] = cseg.st; }
        } else {
            if (ring_cap > 0 && wt.nring == ring_cap) {   // only when one span covers many short sequences
                drain_ring<kRecords>(a, lds, wp, wt);
                __builtin_amdgcn_s_waitcnt(0x0F70);        // vmcnt(0): leave no store in flight behind
            }
            if (ring_cap == 0) {
                if (kRecords) put_record(record_place(a, cseg.b, h, 0, 0), cur, G, g, n);
                else store_out(a, cseg.b, h, cur, G, g, n);
                __builtin_amdgcn_s_waitcnt(0x0F70);
            } else {
                unsigned char* dst = defer + a.rec_stride + wt.nring * ring_entry;
                if (kRecords) put_record(dst, cur, G, g, n);
                else if (n < G) {
                    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
#pragma unroll
                    for (int t = 0; t < 8; ++t) *reinterpret_cast<u32x2*>(dst + (g * G + n) * 64 + 8 * t) = pack_out(cur.acc[t], inv);
                }
                if (lane == 0) exitT[8 + wt.nring] = cseg.b;
                ++wt.nring;
            }
        }
        lds_order();
        ++wt.flushed;
#pragma unroll
        for (int t = 0; t < 8; ++t) cur.acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        cur.m = -INFINITY;
        cur.l = 0.f;
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
        const float m_new = fmaxf(cur.m, mx);
        const float alpha = __builtin_amdgcn_exp2f(cur.m - m_new);
        cur.m = m_new;
        float psum = 0.f;
        float pv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            pv[i] = __builtin_amdgcn_exp2f(sv[i] - m_new);
            psum += pv[i];
        }
        cur.l = cur.l * alpha + psum;
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
            for (int t = 0; t < 8; ++t) cur.acc[t] *= alpha;
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
            cur.acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vt), pb, cur.acc[t], 0, 0, 0);
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
}

// kRecords = true: the streaming phase; every chain is left as a record for paged_decode_merge_kernel.
// kRecords = false: the whole op in one launch, for launches in which the host has made sure that no
// sequence reaches across two workgroups (every chain is a whole sequence).
//
// Grid: wg_spans * head_groups workgroups of 8 wavefronts.  Workgroup (s, hg): wavefront
// (hsub, piece) streams span s * parts + piece for KV head hg * (8 / parts) + hsub.
template <bool kRecords>
__global__ void __launch_bounds__(512) paged_decode_kernel(DecodeArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_all[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int parts = a.parts;
    const int hsub = wave / parts, piece = wave - hsub * parts;
    const int s = blockIdx.x / a.head_groups, hg = blockIdx.x - s * a.head_groups;
    WavePlace wp;
    wp.h = hg * (8 / parts) + hsub;
    wp.s = s;
    wp.lane = lane;
    const int h = wp.h;
    const int w = s * parts + piece;        // this wavefront's span
    const int W = a.wg_spans * parts;       // spans of the launch
    unsigned char* lds = lds_all + wave * kLdsPerWave;
    int* plan = reinterpret_cast<int*>(lds + kLdsWave);
    int* exitT = reinterpret_cast<int*>(lds + kLdsWave + kPlanBytes + kDeferBytes);
    const int steps_per_blk = a.block_size / kStep;
    const int G = a.group, g = lane >> 4, n = lane & 15;

    if (lane < kExitBytes / 4) exitT[lane] = 0;

    // Total number of steps (the first 64 lengths stay in registers for the second pass).  On the way,
    // rows without tokens (graph padding) get their zeros: row b from wavefront b / grid of workgroup
    // b % grid (the merge kernel does it when the chains are left as records).
    auto zero_rows = [&](int c, int len, bool in_batch) {
        unsigned long long empty = __ballot(in_batch && len <= 0);
        while (empty) {
            const int b = c + __builtin_ctzll(empty);
            empty &= empty - 1;
            if (b % (int)gridDim.x == (int)blockIdx.x && (b / (int)gridDim.x) % 8 == wave) {
                uint16_t* op = a.out + (int64_t)b * a.out_stride0;
                for (int off = lane * 4; off < a.num_kv_heads * G * kD; off += 256)
                    *reinterpret_cast<u32x2*>(op + off) = u32x2{0u, 0u};
            }
        }
    };
    const int len0 = lane < a.batch ? ctx_len(a, lane) : 0;
    if (!kRecords) zero_rows(0, len0, lane < a.batch);
    int total = wave_sum(steps_of(len0));
    for (int c = 64; c < a.batch; c += 64) {
        const int i = c + lane;
        const int len = i < a.batch ? ctx_len(a, i) : 0;
        if (!kRecords) zero_rows(c, len, i < a.batch);
        total += wave_sum(steps_of(len));
    }
    total = __builtin_amdgcn_readfirstlane(total);   // wave-uniform: keep the plan in scalar registers

    // Equal shares: the first `rem` spans take one step more.  With fewer steps than spans every step
    // gets a wavefront of its own: on tiny problems a longer span would only serialise memory latency.
    //
    // A launch takes as long as its longest span, so the longest span is made as short as the grid
    // allows, ceil(total / W) steps, and then the fewest spans that reach it are used: the shares are
    // as even as whole steps permit; the wavefronts beyond the span count have nothing to stream.
    int spans = W;
    if (total > W) {
        const int longest = (total + W - 1) / W;
        spans = (total + longest - 1) / longest;
    }
    if (blockIdx.x == 0 && wave == 0 && lane == 0) {
        a.header[0] = spans;
        a.header[1] = total;
        a.header[2] = parts;
    }
    if (s * parts >= spans) return;   // the whole workgroup is beyond the span count
    const int q = total / spans, rem = total - q * spans;
    const int lo = w * q + (w < rem ? w : rem);
    const int hi = w < spans ? lo + q + (w < rem ? 1 : 0) : lo;

    WaveTail wt;
    wt.flushed = 0;
    wt.nring = 0;
    if (lo < hi) {
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
                if (kRecords && h == 0 && lane == 0) {
                    if (s_lo == 0) a.seg_first[b] = s;
                    if (s_hi == en - st) a.seg_last[b] = s;
                }
                const int blk0 = s_lo / steps_per_blk;
                const int nblk = (s_hi - 1) / steps_per_blk - blk0 + 1;
                if (nseg == kMaxSegs || (nseg > 0 && nord + nblk > 64)) {
                    lds_order();
                    run_batch<kRecords>(a, lds, plan, nseg, nsteps, tblv, wp, wt);
                    lds_order();
                    nseg = nord = nsteps = 0;
                    tblv = 0;
                }
                if (lane == 0) {
                    int* p = plan + nseg * kPlanInts;
                    p[0] = b; p[1] = ln; p[2] = s_lo; p[3] = s_hi; p[4] = nord; p[5] = s_lo - blk0 * steps_per_blk; p[6] = blk0;
                    p[7] = st;
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
            run_batch<kRecords>(a, lds, plan, nseg, nsteps, tblv, wp, wt);
        }
        lds_order();
        drain_ring<kRecords>(a, lds, wp, wt);
    }

    // ---- the fold: segments of one sequence in consecutive spans of this workgroup form a chain,
    // folded by the wavefront that holds the chain's first segment
    __syncthreads();
    for (int e = 0; e < 2; ++e) {
        const int* et = exitT + 4 * e;
        const int flags = __builtin_amdgcn_readfirstlane(et[1]);
        if (!(flags & kExitValid)) continue;
        const bool left = flags & kExitLeft;
        bool right = flags & kExitRight;
        if (left && piece > 0) continue;   // folded into the chain that began in an earlier wavefront
        const int b = __builtin_amdgcn_readfirstlane(et[0]);
        Partial acc;
        get_record(e == 0 ? lds + kLdsWave + kPlanBytes : lds, acc, G, g, n);
        for (int p2 = piece + 1; right && p2 < parts; ++p2) {
            const unsigned char* ow = lds_all + (hsub * parts + p2) * kLdsPerWave + kLdsWave + kPlanBytes;
            const int f2 = __builtin_amdgcn_readfirstlane(reinterpret_cast<const int*>(ow + kDeferBytes)[1]);
            if (!(f2 & kExitValid)) break;   // cannot happen: the sequence's next step lies in that span
            Partial nx;
            get_record(ow, nx, G, g, n);
            fold(acc, nx);
            right = f2 & kExitRight;
        }
        if (!kRecords && !left && !right) {   // the whole sequence: this workgroup writes the result
            store_out(a, b, h, acc, G, g, n);
            continue;
        }
        // (without records every chain is a whole sequence: the host checked the span grid)
        if (kRecords) {
            // span position of the workgroup that holds the sequence's first step
            const int st = __builtin_amdgcn_readfirstlane(et[2]);
            const int big = rem * (q + 1);
            const int sp = st < big ? st / (q + 1) : rem + (q > 0 ? (st - big) / q : 0);
            put_record(record_place(a, b, h, s, sp / parts), acc, G, g, n);
        }
    }
}

struct MergeArgs {
    uint16_t* out;
    int64_t out_stride0;
    const int32_t* ctx;     // nullptr: every sequence has uniform_len tokens
    int uniform_len;
    int group;
    int num_kv_heads;
    int slots_per_head;     // records per KV head in the workspace, as in the split launch
    const int32_t* seg_first;
    const int32_t* seg_last;
    const unsigned char* rec;
    const unsigned char* rec_first;
    int rec_stride;
    int batch;
};

// Grid (batch, KV heads), 4 wavefronts: the workgroup folds the records of one sequence for the whole
// GQA group of a KV head (they are contiguous in a record).  Wavefront j takes pieces j, j + 4, ... of
// the sequence; lane c the 16-byte vectors c, c + 64, ... of a record (NU of them: 32 G / 64), each
// with the (max, sum) of its head.  The first kFirstPieces pieces sit at places that depend only on
// (sequence, KV head, piece), so they are requested together with the sequence's length and piece
// range, before either is known: one memory round trip for a sequence of up to four pieces.  The four
// wavefronts are then folded through LDS in piece order.
template <int NU>
__global__ void __launch_bounds__(256) paged_decode_merge_kernel(MergeArgs a) {
    static_assert(kFirstPieces == 4, "one wavefront per fixed place");
    extern __shared__ __attribute__((aligned(16))) unsigned char red[];   // [3 wavefronts][NU][64 lanes] f32x4, then as many float2
    f32x4* red_num = reinterpret_cast<f32x4*>(red);
    float2* red_ml = reinterpret_cast<float2*>(red + 3 * NU * 64 * 16);
    const int b = blockIdx.x, h = blockIdx.y;
    const int G = a.group;
    const int j = threadIdx.x >> 6, c = threadIdx.x & 63;
    const int nvec = 32 * G;
    auto load_record = [&](const unsigned char* rec, f32x4 (&v)[NU], float2 (&ml)[NU]) {
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            const int i = c + 64 * u < nvec ? c + 64 * u : 0;
            v[u] = *reinterpret_cast<const f32x4*>(rec + i * 16);
            ml[u] = *reinterpret_cast<const float2*>(rec + 512 * G + ((i >> 3) % G) * 8);
        }
    };
    f32x4 v[NU];
    float2 ml[NU];
    load_record(a.rec_first + (((int64_t)b * a.num_kv_heads + h) * kFirstPieces + j) * a.rec_stride, v, ml);
    const int len = a.ctx ? a.ctx[b] : a.uniform_len;
    const int w0 = a.seg_first[b], w1 = a.seg_last[b];
    auto store_vec = [&](int i, u32x2 bits) {
        const int vlane = i >> 3, t = i & 7;
        uint16_t* op = a.out + (int64_t)b * a.out_stride0 + (int64_t)(h * G + vlane % G) * kD + 16 * t + 4 * (vlane / G);
        *reinterpret_cast<u32x2*>(op) = bits;
    };
    if (len <= 0) {   // no tokens (graph padding): zeros; the piece range of such a row is not written
        if (j == 0) {
#pragma unroll
            for (int u = 0; u < NU; ++u)
                if (c + 64 * u < nvec) store_vec(c + 64 * u, u32x2{0u, 0u});
        }
        return;
    }
    const int pieces = w1 - w0 + 1;
    float m[NU], den[NU];
    f32x4 num[NU];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        const bool have = j < pieces;
        m[u] = have ? ml[u].x : -INFINITY;
        den[u] = have ? ml[u].y : 0.f;
        num[u] = have ? v[u] : f32x4{0.f, 0.f, 0.f, 0.f};
    }
    for (int k = j + 4; k < pieces; k += 4) {   // pieces beyond the fixed places (kFirstPieces == 4 wavefronts)
        load_record(a.rec + ((int64_t)h * a.slots_per_head + (w0 + k) + b) * a.rec_stride, v, ml);
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            const float mn = fmaxf(m[u], ml[u].x);
            const float f_old = m[u] == mn ? 1.f : __builtin_amdgcn_exp2f(m[u] - mn);
            const float f_new = ml[u].x == mn ? 1.f : __builtin_amdgcn_exp2f(ml[u].x - mn);
            den[u] = den[u] * f_old + ml[u].y * f_new;
            num[u] = num[u] * f_old + v[u] * f_new;
            m[u] = mn;
        }
    }
    if (j > 0) {
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            red_num[((j - 1) * NU + u) * 64 + c] = num[u];
            red_ml[((j - 1) * NU + u) * 64 + c] = make_float2(m[u], den[u]);
        }
    }
    __syncthreads();
    if (j > 0) return;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        for (int w = 0; w < 3; ++w) {
            const float2 o = red_ml[(w * NU + u) * 64 + c];
            if (o.y > 0.f) {
                const float mn = fmaxf(m[u], o.x);
                const float f_old = m[u] == mn ? 1.f : __builtin_amdgcn_exp2f(m[u] - mn);
                const float f_new = o.x == mn ? 1.f : __builtin_amdgcn_exp2f(o.x - mn);
                den[u] = den[u] * f_old + o.y * f_new;
                num[u] = num[u] * f_old + red_num[(w * NU + u) * 64 + c] * f_new;
                m[u] = mn;
            }
        }
        if (c + 64 * u < nvec) store_vec(c + 64 * u, pack_out(num[u], den[u] > 0.f ? 1.f / den[u] : 0.f));
    }
}

constexpr int kMaxDevices = 64;

}  // namespace

// Scratch of infer_paged_decode_noalloc_bf16: the split-KV records of one call.  Every
// device the library runs on holds its own copy of this array, at its own address, until the process
// ends.  In host code the array's NAME is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t kNoAllocScratchBytes = INFER_KV_DECODE_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char infer_kv_decode_scratch[kNoAllocScratchBytes];

namespace {

// What the library knows about a device: set once by init_device(), read by every decode call.
struct DeviceState {
    int cus;          // compute units
    void* scratch;    // device address of infer_kv_decode_scratch on this device
    hipStream_t last_scratch_stream;   // stream of the last call that used the scratch array
    bool scratch_used;
};
DeviceState g_dev[kMaxDevices];
bool g_dev_known[kMaxDevices] = {false};

// One-time set-up for the current device: the kernels' LDS limit, the compute-unit count and the
// address of the scratch array.  Two first calls that race do the same work twice and store the same
// values.  A first call that arrives while `stream` is being captured is refused: the set-up calls
// are not stream work and must not run inside a capture.
int init_device(hipStream_t stream, bool have_stream, DeviceState** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return INFER_KV_EUNSUPPORTED;
    if (!__atomic_load_n(&g_dev_known[dev], __ATOMIC_ACQUIRE)) {
        if (have_stream) {
            hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(stream, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
                (void)hipGetLastError();
                return INFER_KV_ENOTINIT;
            }
        }
        DeviceState d;
        d.cus = 0;
        if (hipDeviceGetAttribute(&d.cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || d.cus <= 0) d.cus = 256;
        e = hipFuncSetAttribute((const void*)paged_decode_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 8 * kLdsPerWave);
        if (e != hipSuccess) return (int)e;
        e = hipFuncSetAttribute((const void*)paged_decode_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 8 * kLdsPerWave);
        if (e != hipSuccess) return (int)e;
        d.scratch = nullptr;
        d.last_scratch_stream = nullptr;
        d.scratch_used = false;
        e = hipGetSymbolAddress(&d.scratch, HIP_SYMBOL(infer_kv_decode_scratch));
        if (e != hipSuccess) return (int)e;
        if (d.scratch == nullptr) return INFER_KV_EINVAL;
        g_dev[dev] = d;
        __atomic_store_n(&g_dev_known[dev], true, __ATOMIC_RELEASE);
    }
    if (out) *out = &g_dev[dev];
    return INFER_KV_OK;
}

// Spans per KV head in a workgroup for the streaming phase.  More of them fold more of a sequence in
// LDS (fewer records for the merge kernel); fewer make the workgroup read longer contiguous pieces
// of a token row.  Measured on Qwen3-8B shapes (8 KV heads): 2 is 1-2 % ahead of 1 and of 4 from
// 1,024 to 32,768 tokens per sequence; 8 (one KV head = 256 B of a row per workgroup) streams 3-6 %
// slower on contexts of 2,048 tokens and more.
#ifndef INFER_KV_DECODE_PARTS
#define INFER_KV_DECODE_PARTS 2
#endif

struct Launch {
    int parts;        // wavefronts (consecutive spans) per KV head in a workgroup
    int head_groups;  // workgroups per span position
    int S;            // span positions
};

// split_workgroups: span positions of the launch; 0 = as many as fill the chip with one workgroup per
// compute unit.
int plan_launch(int64_t hkv, int64_t split_workgroups, int cus, int parts, Launch* out) {
    if (hkv <= 0 || hkv > (1 << 16) || split_workgroups < 0) return INFER_KV_EINVAL;
    while (hkv % (8 / parts) != 0) parts *= 2;    // 8 / parts heads per workgroup must divide the heads; parts = 8 always does
    const int64_t head_groups = hkv / (8 / parts);
    int64_t S = split_workgroups;
    if (S == 0) {
        S = cus / head_groups;
        if (S < 1) S = 1;
    }
    if (S > INFER_KV_MAX_SPLIT_WG) S = INFER_KV_MAX_SPLIT_WG;
    out->parts = parts;
    out->head_groups = (int)head_groups;
    out->S = (int)S;
    return INFER_KV_OK;
}

// One length for the whole batch: does every sequence lie inside one workgroup's spans under launch L?
// The same arithmetic as the kernel's span plan, so the answer is exact.
bool sequences_fit_workgroups(int64_t batch, int64_t len, const Launch& L) {
    if (batch > 4096) return false;               // (the check is a loop over the batch)
    const int64_t n = (len + kStep - 1) / kStep;  // steps per sequence
    const int64_t total = batch * n, W = (int64_t)L.S * L.parts;
    if (n == 0) return true;                      // nothing to attend: the kernel writes the zeros
    int64_t spans = W;
    if (total > W) {
        const int64_t longest = (total + W - 1) / W;
        spans = (total + longest - 1) / longest;
    }
    const int64_t q = total / spans, rem = total - q * spans, big = rem * (q + 1);
    auto wg_of = [&](int64_t x) { return (x < big ? x / (q + 1) : rem + (x - big) / q) / L.parts; };
    for (int64_t b = 0; b < batch; ++b)
        if (wg_of(b * n) != wg_of((b + 1) * n - 1)) return false;
    return true;
}

int check_shape(int64_t batch, int64_t hq, int64_t hkv, int64_t d, int64_t bs, int64_t nblk, int64_t table_cols) {
    if (batch <= 0 || hq <= 0 || hkv <= 0 || nblk <= 0 || bs <= 0 || table_cols <= 0) return INFER_KV_EINVAL;
    if (batch > (1 << 20) || hkv > (1 << 16)) return INFER_KV_EINVAL;
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

// Checks every argument of the streaming phase (host only: no device is touched).
int check_split(const DecodeCall& c, int64_t split_workgroups, const void* workspace) {
    if (split_workgroups < 0) return INFER_KV_EINVAL;
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
    return INFER_KV_OK;
}

int check_out(const void* out, int64_t out_stride0, int64_t num_q_heads) {
    if (!out || out_stride0 < num_q_heads * kD) return INFER_KV_EINVAL;
    // 8-byte stores of four outputs
    if (((uintptr_t)out & 7) || (out_stride0 & 3)) return INFER_KV_EALIGN;
    return INFER_KV_OK;
}

// Enqueues the streaming kernel; `base` is device memory laid out as `ws` (arguments already checked).
// kRecords: every chain stays in the workspace as a record (out is not touched).
template <bool kRecords>
int launch_stream(const DecodeCall& c, const Launch& L, const DecodeWorkspace& ws, void* base_v, void* out,
                  int64_t out_stride0, hipStream_t stream) {
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
    a.out = (uint16_t*)out;
    a.out_stride0 = out_stride0;
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
    a.rec_first = (unsigned char*)base + ws.rec_first_off;
    a.rec_stride = (int)ws.rec_stride;
    a.slots_per_head = (int)ws.slots_per_head;
    a.parts = L.parts;
    a.head_groups = L.head_groups;
    a.wg_spans = L.S;
    dim3 grid((unsigned)(L.S * L.head_groups), 1, 1), block(512, 1, 1);
    hipLaunchKernelGGL(paged_decode_kernel<kRecords>, grid, block, 8 * kLdsPerWave, stream, a);
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
    m.num_kv_heads = (int)num_kv_heads;
    m.slots_per_head = (int)ws.slots_per_head;
    m.seg_first = (const int32_t*)(base + ws.seg_first_off);
    m.seg_last = (const int32_t*)(base + ws.seg_last_off);
    m.rec = (const unsigned char*)base + ws.rec_off;
    m.rec_first = (const unsigned char*)base + ws.rec_first_off;
    m.rec_stride = (int)ws.rec_stride;
    m.batch = (int)batch;
    dim3 grid((unsigned)batch, (unsigned)num_kv_heads, 1), block(256, 1, 1);
    const int nu = (32 * m.group + 63) / 64;   // 16-byte vectors of a record per lane
    if (nu <= 1) hipLaunchKernelGGL(paged_decode_merge_kernel<1>, grid, block, 3 * 1 * 64 * 24, stream, m);
    else if (nu <= 2) hipLaunchKernelGGL(paged_decode_merge_kernel<2>, grid, block, 3 * 2 * 64 * 24, stream, m);
    else if (nu <= 4) hipLaunchKernelGGL(paged_decode_merge_kernel<4>, grid, block, 3 * 4 * 64 * 24, stream, m);
    else hipLaunchKernelGGL(paged_decode_merge_kernel<8>, grid, block, 3 * 8 * 64 * 24, stream, m);
    return (int)hipGetLastError();
}

// The decode op on memory laid out as `ws`: the streaming kernel and the merge kernel behind it.
int run_decode(const DecodeCall& c, const Launch& L, const DecodeWorkspace& ws, void* base, void* out,
               int64_t out_stride0, hipStream_t stream) {
    int rc = launch_stream<true>(c, L, ws, base, nullptr, 0, stream);
    if (rc) return rc;
    return launch_merge(out, out_stride0, c.context_lens, c.uniform_len, c.batch, c.num_q_heads, c.num_kv_heads, ws,
                        base, stream);
}

}  // namespace

extern "C" {

int infer_kv_init(void) { return init_device(nullptr, false, nullptr); }

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
    int rc = check_split(c, split_workgroups, workspace);
    if (rc) return rc;
    const DecodeWorkspace ws = decode_workspace_layout(batch, num_q_heads / num_kv_heads, num_kv_heads);
    if (ws.total_bytes > workspace_bytes) return INFER_KV_EWORKSPACE;
    DeviceState* dev = nullptr;
    rc = init_device((hipStream_t)stream, true, &dev);
    if (rc) return rc;
    Launch L;
    rc = plan_launch(num_kv_heads, split_workgroups, dev->cus, INFER_KV_DECODE_PARTS, &L);
    if (rc) return rc;
    return launch_stream<true>(c, L, ws, workspace, nullptr, 0, (hipStream_t)stream);
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
    int rc = check_split(c, split_workgroups, workspace);
    if (rc) return rc;
    rc = check_out(out, out_stride0, num_q_heads);
    if (rc) return rc;
    const DecodeWorkspace ws = decode_workspace_layout(batch, num_q_heads / num_kv_heads, num_kv_heads);
    if (ws.total_bytes > workspace_bytes) return INFER_KV_EWORKSPACE;
    DeviceState* dev = nullptr;
    rc = init_device((hipStream_t)stream, true, &dev);
    if (rc) return rc;
    Launch L;
    rc = plan_launch(num_kv_heads, split_workgroups, dev->cus, INFER_KV_DECODE_PARTS, &L);
    if (rc) return rc;
    return run_decode(c, L, ws, workspace, out, out_stride0, (hipStream_t)stream);
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
    int rc = check_split(c, /*split_workgroups=*/0, workspace);
    if (rc) return rc;
    rc = check_out(out, out_stride0, num_q_heads);
    if (rc) return rc;
    const DecodeWorkspace ws = decode_workspace_layout(batch, num_q_heads / num_kv_heads, num_kv_heads);
    if (ws.total_bytes > workspace_bytes) return INFER_KV_EWORKSPACE;
    DeviceState* dev = nullptr;
    rc = init_device((hipStream_t)stream, true, &dev);
    if (rc) return rc;
    Launch L;
    // four spans per KV head in a workgroup, else eight: when every sequence then lies inside one
    // workgroup, the workgroups write the result themselves and no merge launch follows
    const int64_t len = context_len < table_cols * block_size ? context_len : table_cols * block_size;
    for (int parts = 4; parts <= 8; parts *= 2) {
        rc = plan_launch(num_kv_heads, /*split_workgroups=*/0, dev->cus, parts, &L);
        if (rc) return rc;
        if (sequences_fit_workgroups(batch, len, L))
            return launch_stream<false>(c, L, ws, workspace, out, out_stride0, (hipStream_t)stream);
    }
    rc = plan_launch(num_kv_heads, /*split_workgroups=*/0, dev->cus, INFER_KV_DECODE_PARTS, &L);
    if (rc) return rc;
    return run_decode(c, L, ws, workspace, out, out_stride0, (hipStream_t)stream);
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
    int rc = check_split(c, /*split_workgroups=*/0, /*workspace: the library's own=*/(const void*)16);
    if (rc) return rc;
    rc = check_out(out, out_stride0, num_q_heads);
    if (rc) return rc;
    DeviceState* dev = nullptr;
    rc = init_device((hipStream_t)stream, true, &dev);
    if (rc) return rc;
    void* scratch = dev->scratch;
    // All calls on a device share the scratch array.  A call on another stream than the last one, while
    // that stream still has work pending, would overwrite records in use: refused (a cheap check, not a
    // lock: calls that race on two host threads are still the caller's to order).  Streams under capture
    // are not queried.
    {
        const hipStream_t st = (hipStream_t)stream;
        hipStream_t last = __atomic_load_n(&dev->last_scratch_stream, __ATOMIC_ACQUIRE);
        if (__atomic_load_n(&dev->scratch_used, __ATOMIC_ACQUIRE) && last != st) {
            hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
            const bool capturing = hipStreamIsCapturing(st, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone;
            if (!capturing && hipStreamQuery(last) == hipErrorNotReady) return INFER_KV_EBUSY;
            (void)hipGetLastError();
        }
        __atomic_store_n(&dev->last_scratch_stream, st, __ATOMIC_RELEASE);
        __atomic_store_n(&dev->scratch_used, true, __ATOMIC_RELEASE);
    }
    Launch L;
    rc = plan_launch(num_kv_heads, /*split_workgroups=*/0, dev->cus, INFER_KV_DECODE_PARTS, &L);
    if (rc) return rc;
    // laid out for the span positions this call launches, not for the largest count a workspace allows
    const DecodeWorkspace ws = decode_workspace_layout(batch, num_q_heads / num_kv_heads, num_kv_heads, L.S);
    if (ws.total_bytes > kNoAllocScratchBytes) return INFER_KV_EWORKSPACE;
    return run_decode(c, L, ws, scratch, out, out_stride0, (hipStream_t)stream);
}

}  // extern "C"
