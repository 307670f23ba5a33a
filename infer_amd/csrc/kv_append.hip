// KV append for gfx950 (MI355X): scatter new K/V rows into the paged caches, keyed by slot.
//
// Replaces store_kvcache_kernel / store_kvcache (infer/ops/attention.py:16-45 of the
// reference): cache.flat[slot * dkv .. +dkv) = row.  Unlike the reference, rows whose slot is
// negative (padding) or past the end of the cache are skipped instead of written out of bounds.
//
// Pure byte movement, 16 bytes per lane per access, nontemporal on both sides, so the result is
// bit-exact by construction and the kernel is bound by HBM bandwidth (rows in, rows out).  Two launch
// shapes:
//   * up to kRingMinRows rows: one wavefront per token copies its K row and its V row, all loads
//     issued before the first store.  A decode step (tens of rows) is launch-latency bound and this
//     is the shortest dependency chain.
//   * more rows (a prefill step): a fixed grid of kRingWorkgroups x 4 wavefronts; wavefront w owns
//     rows w, w + W, w + 2 W, ... and keeps a ring of kRingBytes of row data in registers: the first
//     ring-full of rows is requested at once, then each row is stored and its buffer refilled.  With
//     W = 2048 wavefronts a prefill step of up to 16 K rows is read completely before the first store,
//     so HBM sees a read burst followed by a write burst instead of a fine mix; on this part a copy
//     costs the sum of what its reads and its writes cost alone, and keeping the two apart is worth
//     10 % at 4 K - 16 K rows (13,809 rows: 20.3 -> 18.2 us).  Row data are requested before the slot
//     is known (a padding row costs a wasted read instead of every row a dependent round trip).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/infer_kv.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWavesPerBlock = 4;
constexpr int kRingMinRows = 3072;     // below this the one-row-per-wavefront shape is as fast or faster
constexpr int kRingWorkgroups = 512;   // x 4 wavefronts = 8 per compute unit on 256 units
constexpr int kRingChunks = 32;        // 16-byte registers of row data per lane in the ring (128 VGPRs)

struct AppendArgs {
    const u32x4* key;
    int64_t key_stride_v;     // row strides in 16-byte units
    const u32x4* value;
    int64_t value_stride_v;
    u32x4* k_cache;
    u32x4* v_cache;
    const int32_t* slot_mapping;
    int64_t n_rows;
    int row_chunks;           // 16-byte chunks per row
    int64_t num_slots;
};

// CHUNKS = 16-byte chunks per lane and row when the row is exactly 64 * CHUNKS chunks wide;
// CHUNKS == 0 is the generic strided loop.
template <int CHUNKS>
__global__ void __launch_bounds__(64 * kWavesPerBlock) kv_append_kernel(AppendArgs a) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (row >= a.n_rows) return;
    const int64_t slot = __builtin_amdgcn_readfirstlane(a.slot_mapping[row]);
    if (slot < 0 || slot >= a.num_slots) return;
    const u32x4* ks = a.key + row * a.key_stride_v;
    const u32x4* vs = a.value + row * a.value_stride_v;
    u32x4* kd = a.k_cache + slot * a.row_chunks;
    u32x4* vd = a.v_cache + slot * a.row_chunks;
    if (CHUNKS > 0) {
        u32x4 kr[CHUNKS > 0 ? CHUNKS : 1], vr[CHUNKS > 0 ? CHUNKS : 1];
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) kr[c] = __builtin_nontemporal_load(ks + lane + 64 * c);
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) vr[c] = __builtin_nontemporal_load(vs + lane + 64 * c);
        // streaming stores: measured 8 % faster than plain stores at prefill sizes
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) __builtin_nontemporal_store(kr[c], kd + lane + 64 * c);
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) __builtin_nontemporal_store(vr[c], vd + lane + 64 * c);
    } else {
        for (int c = lane; c < a.row_chunks; c += 64) {
            u32x4 kr = ks[c];
            u32x4 vr = vs[c];
            kd[c] = kr;
            vd[c] = vr;
        }
    }
}

// The ring shape for many rows: DEPTH = kRingChunks / (2 * CHUNKS) rows in flight per wavefront.
template <int CHUNKS>
__global__ void __launch_bounds__(64 * kWavesPerBlock) kv_append_ring_kernel(AppendArgs a) {
    constexpr int DEPTH = kRingChunks / (2 * CHUNKS);
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    const int64_t nw = (int64_t)gridDim.x * kWavesPerBlock;
    u32x4 buf[DEPTH][2 * CHUNKS];
    int64_t slot[DEPTH];
    auto request = [&](int j, int64_t row) {
        const int64_t s = __builtin_amdgcn_readfirstlane(a.slot_mapping[row]);
        slot[j] = s < a.num_slots ? s : -1;
        const u32x4* ks = a.key + row * a.key_stride_v;
        const u32x4* vs = a.value + row * a.value_stride_v;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) buf[j][c] = __builtin_nontemporal_load(ks + lane + 64 * c);
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) buf[j][CHUNKS + c] = __builtin_nontemporal_load(vs + lane + 64 * c);
    };
#pragma unroll
    for (int j = 0; j < DEPTH; ++j)
        if (wave + j * nw < a.n_rows) request(j, wave + j * nw);
    for (int64_t row = wave; row < a.n_rows; row += DEPTH * nw) {
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) {
            const int64_t r = row + j * nw;
            if (r < a.n_rows) {
                const int64_t s = slot[j];
                if (s >= 0) {
                    u32x4* kd = a.k_cache + s * a.row_chunks;
                    u32x4* vd = a.v_cache + s * a.row_chunks;
#pragma unroll
                    for (int c = 0; c < CHUNKS; ++c) __builtin_nontemporal_store(buf[j][c], kd + lane + 64 * c);
#pragma unroll
                    for (int c = 0; c < CHUNKS; ++c) __builtin_nontemporal_store(buf[j][CHUNKS + c], vd + lane + 64 * c);
                }
                if (r + DEPTH * nw < a.n_rows) request(j, r + DEPTH * nw);
            }
        }
    }
}

// The inverse direction for one sequence: token t of the sequence lives at block table[t / block_size],
// offset t % block_size; one wavefront copies one token row into the dense output.
__global__ void __launch_bounds__(64 * kWavesPerBlock) kv_gather_kernel(const u32x4* __restrict__ cache, const int32_t* __restrict__ table,
                                                                        int64_t n_tokens, int row_chunks, int block_size,
                                                                        int num_blocks, u32x4* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (t >= n_tokens) return;
    int blk = __builtin_amdgcn_readfirstlane(table[t / block_size]);
    blk = blk < 0 ? 0 : (blk >= num_blocks ? num_blocks - 1 : blk);     // a corrupt table cannot fault the GPU
    const u32x4* src = cache + ((int64_t)blk * block_size + t % block_size) * row_chunks;
    u32x4* dst = out + t * row_chunks;
    for (int c = lane; c < row_chunks; c += 64) dst[c] = src[c];
}

}  // namespace

extern "C" {

int infer_kv_gather_bf16(const void* cache, const int32_t* block_table_row, int64_t num_tokens, int64_t dkv,
                         int64_t block_size, int64_t num_blocks, void* out, void* stream) {
    if (num_tokens == 0) return INFER_KV_OK;
    if (!cache || !block_table_row || !out) return INFER_KV_EINVAL;
    if (num_tokens < 0 || dkv <= 0 || block_size <= 0 || num_blocks <= 0) return INFER_KV_EINVAL;
    if (block_size > 0x7fffffffLL || num_blocks > 0x7fffffffLL || dkv / 8 > 0x7fffffffLL) return INFER_KV_EINVAL;
    if (dkv % 8 != 0 || (((uintptr_t)cache | (uintptr_t)out) & 15)) return INFER_KV_EALIGN;
    const int64_t groups = (num_tokens + kWavesPerBlock - 1) / kWavesPerBlock;
    if (groups > 0x7fffffffLL) return INFER_KV_EINVAL;
    hipLaunchKernelGGL(kv_gather_kernel, dim3((unsigned)groups, 1, 1), dim3(64 * kWavesPerBlock, 1, 1), 0, (hipStream_t)stream,
                       (const u32x4*)cache, block_table_row, num_tokens, (int)(dkv / 8), (int)block_size, (int)num_blocks,
                       (u32x4*)out);
    return (int)hipGetLastError();
}

int infer_kv_append_bf16(const void* key, int64_t key_stride0, const void* value, int64_t value_stride0,
                         void* k_cache, void* v_cache, const int32_t* slot_mapping, int64_t n_rows, int64_t dkv,
                         int64_t num_slots, void* stream) {
    if (n_rows == 0) return INFER_KV_OK;
    if (!key || !value || !k_cache || !v_cache || !slot_mapping) return INFER_KV_EINVAL;
    if (n_rows < 0 || dkv <= 0 || num_slots <= 0) return INFER_KV_EINVAL;
    if (key_stride0 < dkv || value_stride0 < dkv) return INFER_KV_EINVAL;
    if (dkv % 8 != 0 || key_stride0 % 8 != 0 || value_stride0 % 8 != 0) return INFER_KV_EALIGN;
    if (((uintptr_t)key | (uintptr_t)value | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) return INFER_KV_EALIGN;
    if ((n_rows + kWavesPerBlock - 1) / kWavesPerBlock > 0x7fffffffLL) return INFER_KV_EINVAL;
    if (dkv / 8 > 0x7fffffffLL) return INFER_KV_EINVAL;
    AppendArgs a;
    a.key = (const u32x4*)key;
    a.key_stride_v = key_stride0 / 8;
    a.value = (const u32x4*)value;
    a.value_stride_v = value_stride0 / 8;
    a.k_cache = (u32x4*)k_cache;
    a.v_cache = (u32x4*)v_cache;
    a.slot_mapping = slot_mapping;
    a.n_rows = n_rows;
    a.row_chunks = (int)(dkv / 8);
    a.num_slots = num_slots;
    const bool ring = n_rows > kRingMinRows;
    const int64_t row_groups = (n_rows + kWavesPerBlock - 1) / kWavesPerBlock;
    dim3 grid((unsigned)(ring && row_groups > kRingWorkgroups ? kRingWorkgroups : row_groups), 1, 1);
    dim3 block(64 * kWavesPerBlock, 1, 1);
    hipStream_t st = (hipStream_t)stream;
#define INFER_KV_LAUNCH_APPEND(C)                                                                \
    do {                                                                                         \
        if (ring) hipLaunchKernelGGL(kv_append_ring_kernel<C>, grid, block, 0, st, a);           \
        else hipLaunchKernelGGL(kv_append_kernel<C>, grid, block, 0, st, a);                     \
    } while (0)
    switch (a.row_chunks) {
        case 64: INFER_KV_LAUNCH_APPEND(1); break;
        case 128: INFER_KV_LAUNCH_APPEND(2); break;
        case 256: INFER_KV_LAUNCH_APPEND(4); break;
        default: hipLaunchKernelGGL(kv_append_kernel<0>, dim3((unsigned)row_groups, 1, 1), block, 0, st, a); break;
    }
#undef INFER_KV_LAUNCH_APPEND
    return (int)hipGetLastError();
}

const char* infer_kv_version(void) { return "0.3"; }

const char* infer_kv_strerror(int code) {
    switch (code) {
        case INFER_KV_OK: return "ok";
        case INFER_KV_EINVAL: return "invalid argument (null pointer, non-positive size or inconsistent stride)";
        case INFER_KV_EALIGN: return "pointer or stride not 16-byte aligned";
        case INFER_KV_EWORKSPACE: return "workspace too small";
        case INFER_KV_EUNSUPPORTED: return "shape not built (head_dim must be 128, group size <= 16, block_size % 32 == 0)";
        case INFER_KV_ESTATE: return "block pool invariant violated (see infer_pool_last_error)";
        case INFER_KV_EBUSY: return "the library's scratch array is in use by work pending on another stream";
        case INFER_KV_ENOTINIT: return "first decode call on this device under stream capture: call infer_kv_init() first";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error";
}

}  // extern "C"
