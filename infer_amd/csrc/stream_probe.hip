// Streaming probes: what this GPU sustains for a read-only stream and for a plain copy, measured
// with the same launch shape as the decode kernel (one workgroup of 512 threads per span, 16-byte
// loads, three batches of eight loads in flight per lane).  Not part of the KV-cache path and not part
// of libinfer_kv.so: built as libinfer_kv_probe.so, which only bench.py --ceiling / --counters load, to
// put the kernels' achieved bandwidth next to the practical ceiling of the part.
// Copy shapes: a grid-stride loop, the small append kernel's shape (one wavefront per 4 KiB), and the
// two halves of the KV append on their own (gather the source rows without storing them, scatter
// rows to their slots without loading any).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/infer_kv_probe.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t fold(u32x4 a) { return a.x ^ a.y ^ a.z ^ a.w; }

// Each workgroup reads a contiguous share of the buffer exactly once.  STREAM: with the streaming
// (nontemporal) hint the decode kernel puts on its V loads.
template <bool STREAM>
__device__ __forceinline__ u32x4 probe_load(const u32x4* p) { return STREAM ? __builtin_nontemporal_load(p) : *p; }

template <bool STREAM>
__global__ void __launch_bounds__(512) stream_read_kernel(const u32x4* __restrict__ src, size_t n_vec, uint32_t* sink) {
    const size_t per = n_vec / gridDim.x;
    const u32x4* p = src + per * blockIdx.x;
    uint32_t acc = 0;
    size_t i = threadIdx.x;
    for (; i + 7 * 512 < per; i += 8 * 512) {
        u32x4 r[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) r[u] = probe_load<STREAM>(p + i + u * 512);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= fold(r[u]);
    }
    for (; i < per; i += 512) acc ^= fold(probe_load<STREAM>(p + i));
    if (acc == 0x9e3779b9u) *sink = acc;   // keeps the loads alive; practically never true
}

__global__ void __launch_bounds__(256) stream_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t n_vec) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + 3 * stride < n_vec; i += 4 * stride) {
        u32x4 r[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) r[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(r[u], dst + i + u * stride);
    }
    for (; i < n_vec; i += stride) dst[i] = src[i];
}

// The append kernel's launch shape on contiguous memory: one wavefront copies 4 KiB (a K row and a
// V row of 2 KiB), four loads then four stores per lane, no loop; 256-thread workgroups.
__global__ void __launch_bounds__(256) stream_copy_rows_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                               size_t n_vec) {
    const size_t wave = ((size_t)blockIdx.x * 256 + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    const size_t base = wave * 256;
    if (base + 256 > n_vec) return;
    u32x4 r[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) r[u] = __builtin_nontemporal_load(src + base + lane + 64 * u);
#pragma unroll
    for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(r[u], dst + base + lane + 64 * u);
}

// The decode kernel's two read streams without its arithmetic: eight wavefronts per workgroup, one per KV
// head, steps of 32 tokens over rows of 2 KiB (8 heads x 256 B), two steps requested before either is
// consumed.  V rows are always read as whole rows (four tokens x 256 B per instruction).  K is read either
// in the MFMA-operand pattern of the decode kernel (KPAT 0: 16 tokens x 64 B per instruction, so each
// 128-byte line is touched by two instructions) or as whole rows like V (KPAT 1); KNT / VNT put the
// streaming hint on the K / V loads.
template <int KPAT, bool KNT, bool VNT>
__global__ void __launch_bounds__(512) kv_pattern_read_kernel(const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
                                                               size_t tokens, uint32_t* sink) {
    const int lane = threadIdx.x & 63, h = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;
    const size_t per = tokens / gridDim.x / 32;      // steps per workgroup
    const size_t s0 = per * blockIdx.x;
    const uint32_t tok = 1024;                       // elements per token row
    const uint32_t k_lane = (8 * (n >> 2) + (n & 3)) * tok + 8 * g;
    const uint32_t v_lane = g * tok + 8 * n;
    uint32_t acc = 0;
    for (size_t s = s0; s + 2 <= s0 + per; s += 2) {
        u32x4 r[2][16];
#pragma unroll
        for (int dd = 0; dd < 2; ++dd) {
            const uint16_t* kb = k + (s + dd) * 32 * tok + h * 128;
            const uint16_t* vb = v + (s + dd) * 32 * tok + h * 128;
            if (KPAT == 0) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        r[dd][t * 4 + j] = probe_load<KNT>(reinterpret_cast<const u32x4*>(kb + t * 4 * tok + k_lane + 32 * j));
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) r[dd][i] = probe_load<KNT>(reinterpret_cast<const u32x4*>(kb + i * 4 * tok + v_lane));
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) r[dd][8 + i] = probe_load<VNT>(reinterpret_cast<const u32x4*>(vb + i * 4 * tok + v_lane));
        }
#pragma unroll
        for (int dd = 0; dd < 2; ++dd)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc ^= fold(r[dd][i]);
    }
    if (acc == 0x9e3779b9u) *sink = acc;   // keeps the loads alive; practically never true
}

// Read half of the KV append: every row with a valid slot is loaded (K and V, 2 KiB each), nothing
// is stored.  One wavefront per row, as the append kernel for few rows.
__global__ void __launch_bounds__(256) append_read_half_kernel(const u32x4* __restrict__ key, const u32x4* __restrict__ value,
                                                               const int32_t* __restrict__ slots, int n_rows,
                                                               int num_slots, uint32_t* sink) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int slot = __builtin_amdgcn_readfirstlane(slots[row]);
    if (slot < 0 || slot >= num_slots) return;
    const u32x4* ks = key + (size_t)row * 128;
    const u32x4* vs = value + (size_t)row * 128;
    const u32x4 x = __builtin_nontemporal_load(ks + lane) ^ __builtin_nontemporal_load(ks + lane + 64) ^
                    __builtin_nontemporal_load(vs + lane) ^ __builtin_nontemporal_load(vs + lane + 64);
    if (fold(x) == 0x9e3779b9u) *sink = 1;   // keeps the loads alive; practically never true
}

// Write half: every row with a valid slot is stored to its slot in both caches, nothing is loaded.
__global__ void __launch_bounds__(256) append_write_half_kernel(u32x4* __restrict__ k_cache, u32x4* __restrict__ v_cache,
                                                                const int32_t* __restrict__ slots, int n_rows,
                                                                int num_slots) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int slot = __builtin_amdgcn_readfirstlane(slots[row]);
    if (slot < 0 || slot >= num_slots) return;
    u32x4* kd = k_cache + (size_t)slot * 128;
    u32x4* vd = v_cache + (size_t)slot * 128;
    const u32x4 r = {(uint32_t)row, 1u, 2u, 3u};
    __builtin_nontemporal_store(r, kd + lane);
    __builtin_nontemporal_store(r, kd + lane + 64);
    __builtin_nontemporal_store(r, vd + lane);
    __builtin_nontemporal_store(r, vd + lane + 64);
}

}  // namespace

extern "C" {

int infer_kv_probe_read_kv_pattern(const void* k, const void* v, size_t tokens, int k_whole_rows, int k_hint, int v_hint,
                                   void* sink4, int workgroups, void* stream) {
    if (!k || !v || !sink4 || workgroups <= 0 || tokens < (size_t)workgroups * 64 || (((uintptr_t)k | (uintptr_t)v) & 15))
        return INFER_KV_EINVAL;
    const dim3 grid(workgroups), block(512);
    hipStream_t st = (hipStream_t)stream;
    const uint16_t* kp = (const uint16_t*)k;
    const uint16_t* vp = (const uint16_t*)v;
    uint32_t* sk = (uint32_t*)sink4;
#define INFER_KV_PROBE_PATTERN(P, KN, VN) hipLaunchKernelGGL((kv_pattern_read_kernel<P, KN, VN>), grid, block, 0, st, kp, vp, tokens, sk)
    const int sel = (k_whole_rows ? 4 : 0) | (k_hint ? 2 : 0) | (v_hint ? 1 : 0);
    switch (sel) {
        case 0: INFER_KV_PROBE_PATTERN(0, false, false); break;
        case 1: INFER_KV_PROBE_PATTERN(0, false, true); break;
        case 2: INFER_KV_PROBE_PATTERN(0, true, false); break;
        case 3: INFER_KV_PROBE_PATTERN(0, true, true); break;
        case 4: INFER_KV_PROBE_PATTERN(1, false, false); break;
        case 5: INFER_KV_PROBE_PATTERN(1, false, true); break;
        case 6: INFER_KV_PROBE_PATTERN(1, true, false); break;
        default: INFER_KV_PROBE_PATTERN(1, true, true); break;
    }
#undef INFER_KV_PROBE_PATTERN
    return (int)hipGetLastError();
}

int infer_kv_probe_append_read_half(const void* key, const void* value, const int32_t* slot_mapping, int64_t n_rows,
                                    int64_t num_slots, void* sink4, void* stream) {
    if (!key || !value || !slot_mapping || !sink4 || n_rows <= 0 || n_rows > 0x7fffffffLL || num_slots <= 0 ||
        num_slots > 0x7fffffffLL || (((uintptr_t)key | (uintptr_t)value) & 15))
        return INFER_KV_EINVAL;
    hipLaunchKernelGGL(append_read_half_kernel, dim3((unsigned)((n_rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4*)key, (const u32x4*)value, slot_mapping, (int)n_rows, (int)num_slots, (uint32_t*)sink4);
    return (int)hipGetLastError();
}

int infer_kv_probe_append_write_half(void* k_cache, void* v_cache, const int32_t* slot_mapping, int64_t n_rows,
                                     int64_t num_slots, void* stream) {
    if (!k_cache || !v_cache || !slot_mapping || n_rows <= 0 || n_rows > 0x7fffffffLL || num_slots <= 0 ||
        num_slots > 0x7fffffffLL || (((uintptr_t)k_cache | (uintptr_t)v_cache) & 15))
        return INFER_KV_EINVAL;
    hipLaunchKernelGGL(append_write_half_kernel, dim3((unsigned)((n_rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                       (u32x4*)k_cache, (u32x4*)v_cache, slot_mapping, (int)n_rows, (int)num_slots);
    return (int)hipGetLastError();
}

int infer_kv_probe_read(const void* src, size_t bytes, void* sink4, int workgroups, void* stream) {
    if (!src || !sink4 || bytes < 16 || workgroups <= 0 || ((uintptr_t)src & 15)) return INFER_KV_EINVAL;
    hipLaunchKernelGGL(stream_read_kernel<false>, dim3(workgroups), dim3(512), 0, (hipStream_t)stream, (const u32x4*)src,
                       bytes / 16, (uint32_t*)sink4);
    return (int)hipGetLastError();
}

int infer_kv_probe_read_streaming(const void* src, size_t bytes, void* sink4, int workgroups, void* stream) {
    if (!src || !sink4 || bytes < 16 || workgroups <= 0 || ((uintptr_t)src & 15)) return INFER_KV_EINVAL;
    hipLaunchKernelGGL(stream_read_kernel<true>, dim3(workgroups), dim3(512), 0, (hipStream_t)stream, (const u32x4*)src,
                       bytes / 16, (uint32_t*)sink4);
    return (int)hipGetLastError();
}

int infer_kv_probe_copy(const void* src, void* dst, size_t bytes, int workgroups, void* stream) {
    if (!src || !dst || bytes < 16 || workgroups <= 0 || (((uintptr_t)src | (uintptr_t)dst) & 15)) return INFER_KV_EINVAL;
    hipLaunchKernelGGL(stream_copy_kernel, dim3(workgroups), dim3(256), 0, (hipStream_t)stream, (const u32x4*)src,
                       (u32x4*)dst, bytes / 16);
    return (int)hipGetLastError();
}

int infer_kv_probe_copy_rows(const void* src, void* dst, size_t bytes, void* stream) {
    if (!src || !dst || bytes < 4096 || (((uintptr_t)src | (uintptr_t)dst) & 15)) return INFER_KV_EINVAL;
    const size_t rows = bytes / 4096;           // a tail shorter than 4 KiB is not copied
    if ((rows + 3) / 4 > 0x7fffffffULL) return INFER_KV_EINVAL;
    hipLaunchKernelGGL(stream_copy_rows_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4*)src, (u32x4*)dst, rows * 256);
    return (int)hipGetLastError();
}

}  // extern "C"
