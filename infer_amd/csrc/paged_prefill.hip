// Paged variable-length causal prefill attention for gfx950 (MI355X), bf16 in / fp32 accumulate.
//
// Replaces flash_attn_varlen_func(Q, K, V, cu_seqlens_q/k, max_seqlen_q/k, softmax_scale,
// causal=True, block_table=...) at infer/ops/attention.py:110-116 of the reference.  With a block
// table (a prefix of the sequence is already cached) the keys of sequence b are tokens [0, sk_b)
// of its paged cache; without one K and V are the packed new rows.  The causal mask is aligned to
// the bottom-right corner: key j is visible to query i iff j <= i + (sk - sq).
//
// A wavefront owns 32 consecutive queries (two MFMA column tiles) of one query head and walks the
// visible keys in steps of 32, with the arithmetic of the decode kernel, the MFMA columns now being
// queries instead of the heads of a GQA group:
//   S^T[key, query] = K[key, :] . Q^T       2 row tiles x 4 v_mfma_f32_16x16x32_bf16 per column tile
//   online softmax in the accumulator layout (lane = query, 8 keys per lane)
//   O^T[d, query]  += V^T[d, key] . P^T     8 MFMAs per column tile
// A workgroup is 3 or 4 wavefronts that read the same keys: up to four query heads of one KV head
// (the largest divisor of the group size that is at most 4) times as many consecutive query blocks
// as fit (4 blocks for one head, 2 for two, 1 otherwise).  They share
// every 32-key K tile and V tile through LDS: the tiles are fetched once per workgroup, straight
// from global memory into a ring of three LDS buffers (global_load_dwordx4 ... lds: no registers, no
// LDS store instructions; tile s + 2 is in flight while tile s + 1 has landed and tile s is consumed;
// one barrier per step).  Without staging registers the kernel fits three wavefronts per SIMD.
#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>


#include "../../include/infer_kv.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef short i16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) i16x4 lds_i16x4;

constexpr int kD = 128;
constexpr int kStep = 32;        // keys per step
constexpr int kQTile = 16;       // queries per wavefront
struct PrefillArgs {
    const uint16_t* q;
    int64_t q_stride0;
    const uint16_t* k;
    const uint16_t* v;
    int64_t blk_stride;
    int64_t tok_stride;
    uint16_t* out;
    int64_t out_stride0;
    const int32_t* cu_q;
    const int32_t* cu_k;
    const int32_t* bt;      // nullptr: packed K/V
    int64_t bt_stride0;
    int group;              // query heads per KV head
    int heads_per_wg;       // query heads of the group that one workgroup covers (divides group)
    int qblocks_per_wg;     // consecutive query blocks one workgroup covers
    int block_size;
    int num_blocks;
    int max_sk;             // paged keys: what a block-table row can address (table_cols * block_size)
    int table_cols;         // entries of a block-table row
    float scale_log2;
    int causal;
};

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 x) { return __builtin_bit_cast(bf16x8, x); }
__device__ __forceinline__ u32x4 load16(const uint16_t* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void lds_order() { __asm__ volatile("" ::: "memory"); }

// max over lanes l and l ^ 16 (l ^ 32) in every lane.  v_permlane16_swap exchanges the odd 16-lane rows
// of its first operand with the even rows of its second: fed the same value twice it returns
// (rows 0 0 2 2, rows 1 1 3 3), whose maximum is the reduction; v_permlane32_swap does the same with
// the two halves of the wavefront.  Both run on the vector pipe: a shuffle through LDS
// (ds_bpermute) would put two LDS round trips on the critical path of every softmax.
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

// LDS layout of a tile.  Key k of the step is row  16 ((k >> 2) & 1) + 4 (k >> 3) + (k & 3)  of the
// tile, so that the 16 K rows one ds_read_b128 touches (one MFMA row tile) and the 8 V rows one
// transposing read touches are consecutive rows.  The tiles are written by global_load ... lds, which
// fills 1 KiB (four rows) per wavefront instruction, lane l at byte 16 l; which 16-byte chunk of which
// row a lane fetches is free, and the choice here interleaves the four rows of such a group in pieces
// of 64 B (four chunks; four consecutive lanes still fetch 64 contiguous bytes of global memory):
// chunk c of row r sits at
//     (r / 4) * kGroupB + (c / 4) * 256 + (r % 4) * 64 + (c % 4) * 16 ,   kGroupB = 1 KiB + 32 B.
// The pad follows from how the LDS of this part serves a wavefront (64 banks of 4 B, measured with a
// probe that times one read pattern at a time): a ds_read_b128 is served in four passes of 16 lanes,
// and the lanes of a pass are NOT consecutive - lanes 0-3, 12-15, 20-27 form one pass, 4-11, 16-19,
// 28-31 the next, and likewise in the upper half.  Lane (g, n) of a K read takes chunk g of row n:
// byte (n / 4) * kGroupB + (n % 4) * 64 + g * 16 modulo 256 selects its banks, so a pass holds the
// (n / 4, g) pairs (0,0) (3,0) (1,1) (2,1) or (1,0) (2,0) (0,1) (3,1), and they fall into four different
// 16-byte slots only if (n / 4) * pad / 16 + g is distinct modulo 4 over each set: pad = 32 does that,
// pad = 16 (slots 0 3 2 3) does not and costs 8 instead of 5 cycles per read.  The transposing V reads
// (4 rows x 32 B per 16 lanes) take 3.9 cycles with this pad against 4.4 with 16.  And the address of a
// read is one per-lane register plus a constant for every K step, row tile and column tile, where a
// rotation of the chunks inside a row (the other conflict-free choice for 256-byte rows) needs a
// register and an addition per read.
constexpr int kNQ = 2;
constexpr float kLazy = 8.f;
constexpr int kQBlock = kNQ * kQTile;
constexpr int kGroupB = 1024 + 32;                        // four interleaved rows and the pad
constexpr int kKTileBytes = (kStep / 4) * kGroupB;
constexpr int kVTileBytes = (kStep / 4) * kGroupB;
constexpr int kTileBytes = kKTileBytes + kVTileBytes;     // one K tile + one V tile
constexpr int kRing = 3;                                  // tiles resident in LDS: consumed, landed, in flight
constexpr int kTblLds = 256;                              // block ids of a sequence kept in LDS
__device__ __forceinline__ int tile_row(int k) { return 16 * ((k >> 2) & 1) + 4 * (k >> 3) + (k & 3); }
__device__ __forceinline__ int tile_key(int r) { return (((r >> 2) & 3) << 3) | ((r >> 4) << 2) | (r & 3); }   // inverse of tile_row

// WAVES = heads per workgroup x QB, QB = query blocks per workgroup (a compile-time constant so that the
// common QB == 1 case carries no per-wavefront step guard).
template <int WAVES, int QB>
__global__ void __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(3, 3))) paged_prefill_tile_kernel(PrefillArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_all[];   // [2][K tile | V tile]
    constexpr int kHeads = WAVES / QB;                                 // query heads per workgroup
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, n = lane & 15;
    // Workgroups are dealt to the eight dies (XCDs) round-robin by their linear id, and each die has an L2
    // of its own.  The linear id is therefore remapped so that die k works through the k-th contiguous
    // eighth of the (query block, sequence, KV head) space: the workgroups that read the same keys sit
    // behind one L2 and the K/V tiles of a (sequence, KV head) are fetched from HBM once, not once per die.
    const unsigned wg_total = gridDim.x * gridDim.y * gridDim.z;
    const unsigned wg_linear = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    const unsigned die = wg_linear & 7u, per_die = wg_total >> 3, extra = wg_total & 7u;
    const unsigned wg_id = __builtin_amdgcn_readfirstlane(die * per_die + (die < extra ? die : extra) + (wg_linear >> 3));
    const int block_x = (int)(wg_id % gridDim.x);
    const int b = (int)((wg_id / gridDim.x) % gridDim.y);
    const int block_z = (int)(wg_id / (gridDim.x * gridDim.y));
    const int parts = a.group / kHeads;                    // workgroups that share one KV head
    const int kvh = block_z / parts;
    const int head = kvh * a.group + (block_z % parts) * kHeads + (QB == 1 ? wave : wave % kHeads);
    const int qb = QB == 1 ? 0 : wave / kHeads;            // query block of this wavefront inside the workgroup

    // The first kTblLds block ids of the sequence go to LDS (see below).  Their loads depend on nothing but
    // the sequence index, so they are issued first and travel while the sequence bounds are fetched;
    // entries of the row behind the sequence's own blocks are loaded too and never used.
    constexpr int kTblPer = (kTblLds + 64 * WAVES - 1) / (64 * WAVES);
    const int tbl_cols = a.bt ? (a.table_cols < kTblLds ? a.table_cols : kTblLds) : 0;
    int tbl_reg[kTblPer];
#pragma unroll
    for (int i = 0; i < kTblPer; ++i) {
        const int c = tid + i * 64 * WAVES;
        tbl_reg[i] = c < tbl_cols ? a.bt[(int64_t)b * a.bt_stride0 + c] : 0;
    }
    const int q_beg = a.cu_q[b], q_end = a.cu_q[b + 1];
    const int k_beg = a.cu_k[b], k_end = a.cu_k[b + 1];
    const int sq = q_end - q_beg;
    int sk = k_end - k_beg;
    if (a.bt != nullptr && sk > a.max_sk) sk = a.max_sk;   // a corrupt length cannot run the gather past its table row
    // late query blocks see the most keys: hand them out first so the long workgroups start early
    const int wg_q0 = (int)(gridDim.x - 1 - block_x) * QB * kQBlock;
    if (wg_q0 >= sq) return;
    const int q0 = wg_q0 + qb * kQBlock;
    const bool live = QB == 1 || q0 < sq;   // a trailing wavefront may have no queries: it only helps to fetch
    if (sk <= 0) {
#pragma unroll
        for (int u = 0; u < kNQ; ++u)
            if (live && q0 + 16 * u + n < sq) {
                uint16_t* op = a.out + (int64_t)(q_beg + q0 + 16 * u + n) * a.out_stride0 + (int64_t)head * kD + 4 * g;
                for (int t = 0; t < 8; ++t) *reinterpret_cast<u32x2*>(op + 16 * t) = u32x2{0u, 0u};
            }
        return;
    }
    const int shift = sk - sq;
    int my_q[kNQ], my_limit[kNQ];
#pragma unroll
    for (int u = 0; u < kNQ; ++u) {
        my_q[u] = q0 + 16 * u + n;
        my_limit[u] = a.causal ? (my_q[u] + shift < sk - 1 ? my_q[u] + shift : sk - 1) : sk - 1;
    }
    // lane 0 holds the earliest query of a tile, hence the smallest limit
    int lim_lo[kNQ];
#pragma unroll
    for (int u = 0; u < kNQ; ++u) lim_lo[u] = __builtin_amdgcn_readfirstlane(my_limit[u]);
    // keys the workgroup walks (its last query block sees the most) and keys this wavefront needs
    auto key_end_of = [&](int first_q, int count) {
        const int last = first_q + count - 1 < sq - 1 ? first_q + count - 1 : sq - 1;
        return a.causal ? (last + shift + 1 < sk ? last + shift + 1 : sk) : sk;
    };
    const int nsteps = (key_end_of(wg_q0, QB * kQBlock) + kStep - 1) / kStep;
    const int my_steps = live ? (key_end_of(q0, kQBlock) + kStep - 1) / kStep : 0;

    // The first kTblLds block ids of the sequence are copied to LDS behind the ring (one barrier, before
    // anything is fetched): a lookup in memory, behind a division by the block size, would put some
    // 300 ns of dependent work in front of every tile fetch, and a register copy gets spilled, whose
    // reload is a vector load and so drains the ring.  Tiles are fetched in order, so the block index
    // and the step inside the block are counters.
    const int steps_per_blk = a.block_size / kStep;
    int* lds_tbl = reinterpret_cast<int*>(lds_all + kRing * kTileBytes);
    if (a.bt) {
#pragma unroll
        for (int i = 0; i < kTblPer; ++i) {
            const int c = tid + i * 64 * WAVES;
            if (c < tbl_cols) lds_tbl[c] = tbl_reg[i];
        }
        __syncthreads();
    }
    // (the loads of Q are issued after this wait, not before it: the compiler's wait for the block ids
    // would wait for them as well)
    bf16x8 qreg[kNQ][4];
    bf16x8 ones;
#pragma unroll
    for (int i = 0; i < 8; ++i) ones[i] = (__bf16)1.0f;
#pragma unroll
    for (int u = 0; u < kNQ; ++u) {
        // lanes behind the last query of the sequence load its first query instead: straight-line loads,
        // finite values, and their columns of the result are never stored
        const uint16_t* qp = a.q + (int64_t)(q_beg + (my_q[u] < sq ? my_q[u] : 0)) * a.q_stride0 + (int64_t)head * kD + 8 * g;
#pragma unroll
        for (int j = 0; j < 4; ++j) qreg[u][j] = as_bf16x8(load16(qp + 32 * j));
    }
    f32x4 acc[kNQ][8];
    // Row sums ride the matrix pipe: ones[16 x 32] . P^T adds the 32 probabilities of a step for every
    // query (one MFMA per tile and step instead of eight vector adds), of the same bf16 values the
    // numerator is built from; all four accumulator rows of a lane hold the same sum.
    f32x4 lacc[kNQ];
    float m_neg[kNQ];
#pragma unroll
    for (int u = 0; u < kNQ; ++u) {
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        m_neg[u] = INFINITY;
        lacc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // Cooperative tile fetch, global memory -> LDS without passing through registers.  One
    // global_load_dwordx4 ... lds of a wavefront fills 1 KiB of LDS, lane l at byte 16 l: four rows
    // of a tile, lane l = chunk position l % 16 of row l / 16, which by the rotation above is chunk
    // (l % 16 - row) % 16 of that row's key.  A tile pair is 16 such loads (8 K, 8 V); wavefront w
    // issues loads w, w + WAVES, ...  Every wavefront issues the same number per tile (a surplus
    // one repeats load 0: same bytes to the same place), so "this tile has landed" is a fixed count
    // of its own outstanding loads followed by the workgroup barrier.
    //
    // The load is issued as inline assembly on purpose.  Through the compiler's builtin every later
    // LDS read is preceded by a wait for ALL outstanding loads (the compiler cannot see that a read
    // touches another ring buffer than the one being filled), which would leave the newest tile half a
    // step to arrive instead of two.  Here the waits are the explicit counts below.  M0 holds the LDS
    // base of the transfer; nothing else in this kernel uses M0 (no other LDS transfer, no indexed
    // register access), so it is not saved: the scalar instructions of a transfer are on the critical
    // path of every step.
    // Address = uniform 64-bit base (scalar registers) + per-lane 32-bit byte offset: no vector
    // arithmetic per transfer.
    typedef __attribute__((address_space(3))) void* lptr_t;
    auto dma16 = [&](const unsigned char* base, uint32_t byte_off, uint32_t lds_addr) {
        __asm__ volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         :: "v"(byte_off), "s"(base), "s"(lds_addr) : "memory", "m0");
    };
    constexpr int kLoads = (16 + WAVES - 1) / WAVES;
    const int tok_stride = (int)a.tok_stride;     // < 2^24 elements (checked on the host)
    // loads 0 .. 7 are the K tile, 8 .. 15 the V tile: with four wavefronts (load w + 4 i) that is a
    // matter of i alone
    auto load_is_k = [&](int i) { return WAVES == 4 ? i < 2 : (wave + i * WAVES < 16 ? wave + i * WAVES : 0) < 8; };
    uint32_t ld_byte[kLoads];                     // byte offset inside a tile of what this lane fetches
    int ld_dst[kLoads];                           // LDS byte offset of the load inside a tile pair (uniform)
    auto ld_key = [&](int i) {                    // key (row of the tile in memory) of load i of this lane:
        const int L = wave + i * WAVES < 16 ? wave + i * WAVES : 0;
        return tile_key(4 * (L & 7) + ((lane >> 2) & 3));              // lane l fills row (l / 4) % 4 of group L,
    };
    auto ld_col = [&](int i) { return (uint32_t)(kvh * kD + ((lane & 3) + 4 * (lane >> 4)) * 8); };   // chunk l % 4 + 4 (l / 16)
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int L = wave + i * WAVES < 16 ? wave + i * WAVES : 0;
        ld_byte[i] = 2 * ((uint32_t)(ld_key(i) * tok_stride) + ld_col(i));   // < 2^31: tok_stride < 2^24, 32 rows
        ld_dst[i] = (L >> 3) * kKTileBytes + (L & 7) * kGroupB;
    }
    // Tiles are fetched in order, so the address of the next one is a running 64-bit byte offset: one
    // addition per tile, a table lookup and a multiplication only where a block begins.  (A step of a
    // wavefront is some 250 instructions issued in order; address arithmetic redone from the step index
    // was 40 scalar instructions of them.)
    const int64_t tile_bytes = 2 * (int64_t)kStep * a.tok_stride;
    int64_t f_byte = a.bt ? 0 : 2 * (int64_t)k_beg * a.tok_stride;   // byte offset of the next tile to fetch
    int f_blk = 0, f_left = 0;    // next block of the table, tiles left in the current one
    const int whole_tiles = sk / kStep;                        // tiles in front of this index are whole
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)lds_all;
    uint32_t ld_lds[kLoads];                                   // LDS address of load i in ring buffer 0 (uniform)
#pragma unroll
    for (int i = 0; i < kLoads; ++i) ld_lds[i] = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)ld_dst[i]);
    // ring_off: byte offset of the ring buffer that takes the tile
    auto fetch = [&](int s, int ring_off) {
        if (a.bt) {
            if (f_left == 0) {
                int blk;
                if (f_blk < kTblLds) blk = __builtin_amdgcn_readfirstlane(lds_tbl[f_blk]);
                else blk = __builtin_amdgcn_readfirstlane(a.bt[(int64_t)b * a.bt_stride0 + f_blk]);   // drains the ring
                blk = blk < 0 ? 0 : (blk >= a.num_blocks ? a.num_blocks - 1 : blk);
                f_byte = 2 * (int64_t)blk * a.blk_stride;
                f_left = steps_per_blk;
                ++f_blk;
            }
            --f_left;
        }
        const unsigned char* kp = reinterpret_cast<const unsigned char*>(a.k) + f_byte;
        const unsigned char* vp = reinterpret_cast<const unsigned char*>(a.v) + f_byte;
        f_byte += tile_bytes;
        if (s < whole_tiles) {
#pragma unroll
            for (int i = 0; i < kLoads; ++i) dma16(load_is_k(i) ? kp : vp, ld_byte[i], ld_lds[i] + (uint32_t)ring_off);
        } else {
            // rows past the end of the sequence (last step only) re-read its last row: finite data whose
            // probabilities are masked to zero, instead of whatever lies behind the sequence
            const int last = sk - 1 - s * kStep;
#pragma unroll
            for (int i = 0; i < kLoads; ++i) {
                const int r = ld_key(i) < last ? ld_key(i) : last;
                dma16(load_is_k(i) ? kp : vp, 2 * ((uint32_t)(r * tok_stride) + ld_col(i)), ld_lds[i] + (uint32_t)ring_off);
            }
        }
    };
    // this wavefront's loads of all tiles but the newest have landed / of all tiles have landed
    auto landed_but_newest = [&]() { __builtin_amdgcn_s_waitcnt(0x0F70 | kLoads); };
    auto landed_all = [&]() { __builtin_amdgcn_s_waitcnt(0x0F70); };

    // Read addresses.  K operand row n of MFMA row tile t is key 8 (n / 4) + 4 t + n % 4 = tile row
    // 16 t + n, K step j is chunk 4 j + g of it.  V keys 8 g + n / 4 (lo) and 8 g + 4 + n / 4 (hi) are
    // tile rows 4 g + n / 4 and 16 more; columns 16 t + 4 (n % 4) .. + 3 are half n % 2 of chunk
    // 2 t + (n % 4) / 2.
    const int k_addr = (n >> 2) * kGroupB + (n & 3) * 64 + g * 16;
    const int v_addr = kKTileBytes + g * kGroupB + (n >> 2) * 64 + ((n & 3) >> 1) * 16 + (n & 1) * 8;

    // tile s lives in ring buffer s % 3: requested at the top of step s - 2, landed (own loads counted,
    // then the barrier) at the end of step s - 1, read during step s; the buffer is requested again at
    // the top of step s + 1, after the barrier that ends step s.
    // The loads of Q are still in flight when the first two tiles are requested, so that the two round
    // trips to memory overlap; one wait for everything follows.  It is written out, although the
    // compiler would wait for Q by itself: the compiler does not see the transfers, so its own wait
    // would sit at the first use of Q inside the loop, as a wait for zero outstanding loads in every
    // step, which drains the ring.
    fetch(0, 0);
    if (nsteps > 1) fetch(1, kTileBytes);
    landed_all();
    __syncthreads();

    // With four wavefronts the loop is unrolled by the ring, so that the buffer of tile s is a constant of
    // each copy and every LDS address of the step is a per-lane register plus an immediate.
    // ring: byte offset of the buffer that holds tile s; ring_next: of the one that takes tile s + 2
    // (plain integers, or compile-time constants in the unrolled loop)
    // inner_tag: a step of the main loop, which is known to request tile s + 2 and to lie in front of the
    // diagonal of every wavefront: no branch for either
    auto step = [&](int s, auto ring_v, auto ring_next_v, auto inner_tag) {
        constexpr bool kInner = decltype(inner_tag)::value;
        const int ring = ring_v, ring_next = ring_next_v;
        if (kInner || s + 2 < nsteps) fetch(s + 2, ring_next);
        const unsigned char* kb = lds_all + ring;
        const int tok0 = s * kStep;

        if (QB == 1 || s < my_steps) {   // wavefronts whose queries end earlier skip the keys they cannot see
        // ---- S^T = K Q^T for both query tiles
        f32x4 sc[kNQ][2];
#pragma unroll
        for (int u = 0; u < kNQ; ++u)
#pragma unroll
            for (int t = 0; t < 2; ++t) sc[u][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u32x4 kf = *reinterpret_cast<const u32x4*>(kb + k_addr + 4 * t * kGroupB + j * 256);
#pragma unroll
                for (int u = 0; u < kNQ; ++u)
                    sc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf), qreg[u][j], sc[u][t], 0, 0, 0);
            }

        // ---- online softmax per query tile.  The running maximum is refreshed only when a row's
        // maximum grows by more than kLazy (log2 units): until then the probabilities are taken
        // relative to the stale maximum (at most 2^kLazy, harmless in float32 and bf16) and the
        // accumulators need no rescaling; the final division by the row sum makes both forms equal.
        bf16x8 pb[kNQ];
#pragma unroll
        for (int u = 0; u < kNQ; ++u) {
            float sv[8];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) sv[4 * t + e] = sc[u][t][e];
            if (!kInner && tok0 + kStep - 1 > lim_lo[u]) {      // wave-uniform: off the diagonal no lane masks anything
                // key tok0 + 8 g + i is masked iff i > rel; written so that nothing but this one
                // subtraction could be computed ahead of the branch
                const int rel = my_limit[u] - tok0 - 8 * g;
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (i > rel) sv[i] = -INFINITY;
            }
            float mx = sv[0];
#pragma unroll
            for (int i = 1; i < 8; ++i) mx = fmaxf(mx, sv[i]);
            mx = max_xor32(max_xor16(mx));
            mx *= a.scale_log2;                                  // scale > 0: the maximum commutes with it
            // m_neg is minus the running maximum, +inf before the first step: key 0 is visible to every
            // query, so step 0 always "grows" (inf > kLazy) and sets it.  (A query without any visible key,
            // sq > sk, keeps +inf; its row is written as zeros at the end.)
            const bool grow = mx + m_neg[u] > kLazy;
            if (__any(grow)) {
                const float alpha = grow ? __builtin_amdgcn_exp2f(-m_neg[u] - mx) : 1.f;
                m_neg[u] = grow ? -mx : m_neg[u];
                lacc[u] *= alpha;
#pragma unroll
                for (int t = 0; t < 8; ++t) acc[u][t] *= alpha;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i)
                pb[u][i] = (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(sv[i], a.scale_log2, m_neg[u]));
            lacc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[u], lacc[u], 0, 0, 0);
        }

        // ---- O^T += V^T P^T, every V fragment used for both query tiles
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const unsigned char* src = kb + v_addr + (t >> 1) * 256 + (t & 1) * 32;
            const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(src));
            const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*)(src + 4 * kGroupB));
            const bf16x8 vt = __builtin_bit_cast(bf16x8, (i16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
            for (int u = 0; u < kNQ; ++u)
                acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt, pb[u], acc[u][t], 0, 0, 0);
        }
        }

        // tile s + 1 must be in LDS for everybody: own loads first, then the barrier
        if (kInner || s + 2 < nsteps) landed_but_newest(); else landed_all();
        __syncthreads();
    };
    // steps in front of inner_end request a tile two steps ahead and end in front of the keys the
    // workgroup's first query cannot see (the earliest diagonal of the workgroup)
    const int wg_lim_lo = a.causal ? (wg_q0 + shift < sk - 1 ? wg_q0 + shift : sk - 1) : sk - 1;
    const int free_steps = wg_lim_lo >= 0 ? (wg_lim_lo + 1) / kStep : 0;
    const int inner_end = nsteps - 2 < free_steps ? nsteps - 2 : free_steps;
    using Inner = std::true_type;
    using Outer = std::false_type;
    if constexpr (WAVES == 4) {
        using B0 = std::integral_constant<int, 0>;
        using B1 = std::integral_constant<int, kTileBytes>;
        using B2 = std::integral_constant<int, 2 * kTileBytes>;
        int s = 0;
        for (; s + 2 < inner_end; s += 3) {
            step(s, B0{}, B2{}, Inner{});
            step(s + 1, B1{}, B0{}, Inner{});
            step(s + 2, B2{}, B1{}, Inner{});
        }
        for (; s + 2 < nsteps; s += 3) {
            step(s, B0{}, B2{}, Outer{});
            step(s + 1, B1{}, B0{}, Outer{});
            step(s + 2, B2{}, B1{}, Outer{});
        }
        if (s < nsteps) step(s, B0{}, B2{}, Outer{});
        if (s + 1 < nsteps) step(s + 1, B1{}, B0{}, Outer{});
    } else {
        // three wavefronts issue six transfers each: the unrolled form runs out of registers
        for (int s = 0, ring = 0, ring_next = 2 * kTileBytes; s < nsteps; ++s) {
            step(s, ring, ring_next, Outer{});
            ring_next = ring;                                            // (s + 3) % 3 = s % 3
            ring = ring == 2 * kTileBytes ? 0 : ring + kTileBytes;
        }
    }

    if (!live) return;
#pragma unroll
    for (int u = 0; u < kNQ; ++u) {
        const float l = lacc[u][0];
        if (my_q[u] < sq) {
            const bool none = my_limit[u] < 0;          // no key visible to this query (sq > sk): zeros, whatever the sums hold
            const float inv = l > 0.f ? 1.f / l : 0.f;
            uint16_t* op = a.out + (int64_t)(q_beg + my_q[u]) * a.out_stride0 + (int64_t)head * kD + 4 * g;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                union { __bf16 hv[4]; u32x2 w; } r;
#pragma unroll
                for (int e = 0; e < 4; ++e) r.hv[e] = (__bf16)(acc[u][t][e] * inv);
                *reinterpret_cast<u32x2*>(op + 16 * t) = none ? u32x2{0u, 0u} : r.w;
            }
        }
    }
}

template <int WAVES, int QB>
int launch_tiled(const PrefillArgs& a, int64_t max_seqlen_q, int64_t num_seqs, int64_t num_kv_heads, hipStream_t st) {
    const int64_t q_per_wg = (int64_t)QB * kQBlock;
    const int parts = a.group / (WAVES / QB);
    dim3 grid((unsigned)((max_seqlen_q + q_per_wg - 1) / q_per_wg), (unsigned)num_seqs, (unsigned)(num_kv_heads * parts));
    hipLaunchKernelGGL((paged_prefill_tile_kernel<WAVES, QB>), grid, dim3(64 * WAVES, 1, 1), kRing * kTileBytes + kTblLds * 4, st, a);
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int infer_paged_prefill_bf16(const void* q, int64_t q_stride0, const void* k, const void* v,
                                        int64_t kv_block_stride, int64_t kv_token_stride, int64_t kv_rows,
                                        void* out, int64_t out_stride0, const int32_t* cu_seqlens_q,
                                        const int32_t* cu_seqlens_k, const int32_t* block_table, int64_t bt_stride0,
                                        int64_t table_cols, int64_t num_seqs, int64_t max_seqlen_q, int64_t num_q_heads,
                                        int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                                        int64_t num_blocks, float scale, int causal, void* stream) {
    if (!q || !k || !v || !out || !cu_seqlens_q || !cu_seqlens_k) return INFER_KV_EINVAL;
    if (num_seqs <= 0 || max_seqlen_q < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || kv_rows <= 0) return INFER_KV_EINVAL;
    if (max_seqlen_q == 0) return INFER_KV_OK;
    if (head_dim != kD) return INFER_KV_EUNSUPPORTED;
    if (num_q_heads % num_kv_heads != 0 || num_q_heads / num_kv_heads > 16) return INFER_KV_EUNSUPPORTED;
    // the row maximum is taken before the scale is applied, which needs a positive scale
    if (!(scale > 0.f)) return INFER_KV_EINVAL;
    if (block_table && (block_size <= 0 || block_size % kStep != 0 || num_blocks <= 0)) return INFER_KV_EUNSUPPORTED;
    if (block_table && (table_cols <= 0 || (num_seqs > 1 && bt_stride0 < table_cols) || table_cols * block_size > 0x7fffffffLL))
        return INFER_KV_EINVAL;
    if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) return INFER_KV_EALIGN;
    if ((q_stride0 | kv_token_stride | out_stride0) & 7) return INFER_KV_EALIGN;
    if (block_table && (kv_block_stride & 7)) return INFER_KV_EALIGN;
    if (kv_token_stride < num_kv_heads * kD || q_stride0 < num_q_heads * kD || out_stride0 < num_q_heads * kD) return INFER_KV_EINVAL;
    if (num_seqs > 65535 || num_kv_heads * 16 > 65535) return INFER_KV_EINVAL;
    if (kv_token_stride > (1 << 24)) return INFER_KV_EUNSUPPORTED;   // 32-bit offsets inside a tile
    const int G = (int)(num_q_heads / num_kv_heads);
    // Workgroup shape: the largest divisor of the group size up to 4 as query heads, times the number
    // of consecutive query blocks that brings the workgroup to 3 - 4 wavefronts.  Small workgroups
    // win: three or four of them share a compute unit, each with its own barrier, where one workgroup
    // of 6 - 8 wavefronts (all heads of a large group) keeps every wavefront of the unit in lockstep
    // (measured on 8 x 2048-token prompts, TFLOP/s: G = 8 as 8 heads 526, as 2 x 4 heads 629; G = 6 as
    // 6 heads 408, as 2 x 3 heads 528; G = 5 as 5 heads 340, as 5 x 1 head with 4 query blocks 507).
    int heads = 1;
    for (int h = G < 4 ? G : 4; h >= 1; --h)
        if (G % h == 0) { heads = h; break; }
    const int qb = heads == 1 ? 4 : (heads == 2 ? 2 : 1);
    PrefillArgs a;
    a.q = (const uint16_t*)q; a.q_stride0 = q_stride0;
    a.k = (const uint16_t*)k; a.v = (const uint16_t*)v;
    a.blk_stride = kv_block_stride; a.tok_stride = kv_token_stride;
    a.out = (uint16_t*)out; a.out_stride0 = out_stride0;
    a.cu_q = cu_seqlens_q; a.cu_k = cu_seqlens_k;
    a.bt = block_table; a.bt_stride0 = bt_stride0;
    a.group = G;
    a.block_size = (int)block_size; a.num_blocks = (int)num_blocks;
    a.max_sk = block_table ? (int)(table_cols * block_size) : 0x7fffffff;
    a.table_cols = block_table ? (int)table_cols : 0;
    a.scale_log2 = scale * 1.4426950408889634f;
    a.causal = causal ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    a.heads_per_wg = heads; a.qblocks_per_wg = qb;
    switch (heads) {
        case 1: return launch_tiled<4, 4>(a, max_seqlen_q, num_seqs, num_kv_heads, st);
        case 2: return launch_tiled<4, 2>(a, max_seqlen_q, num_seqs, num_kv_heads, st);
        case 3: return launch_tiled<3, 1>(a, max_seqlen_q, num_seqs, num_kv_heads, st);
        case 4: return launch_tiled<4, 1>(a, max_seqlen_q, num_seqs, num_kv_heads, st);
        default: return INFER_KV_EUNSUPPORTED;
    }
}
