// The small operators a decode step runs around the paged KV-cache path, for gfx950 (MI355X):
//
//   rms_norm_kernel          RMSNorm with optional residual add, the arithmetic of
//                            RMSNorm.rms_forward / add_rms_forward (infer/ops/norm.py:63-86)
//   silu_and_mul_kernel      SwiGLU gate, the arithmetic of act_and_mul_kernel + silu_kernel_vllm
//                            (src/operators/silu/silu.cu:13-31)
//   decode_metadata_kernel   positions / slot_mapping / context_lens of a decode step derived on the
//                            device from the sequence lengths and the block table (the host loop of
//                            ModelRunner.prepare_decode, infer/engine/model_runner.py:110-126)
//
// All three are launch-latency or HBM bound: 16-byte accesses, every byte touched once.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/infer_kv.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
__device__ __forceinline__ float rb(float x) { return (float)(__bf16)x; }   // round to bf16, keep as float
__device__ __forceinline__ uint32_t pack(float lo, float hi) {
    const __bf16 a = (__bf16)lo, b = (__bf16)hi;
    return (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
}
__device__ __forceinline__ void unpack8(u32x4 r, float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { x[2 * i] = bf16_lo(r[i]); x[2 * i + 1] = bf16_hi(r[i]); }
}
__device__ __forceinline__ u32x4 pack8(const float (&x)[8]) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = pack(x[2 * i], x[2 * i + 1]);
    return r;
}

constexpr int kNormThreads = 512;
constexpr int kNormMaxChunks = 2;   // 16-byte chunks per thread: hidden <= 512 * 2 * 8 = 8192

struct NormArgs {
    const float* partial;      // if set: x[row] = bf16(sum over splits of partial[s][row]) instead of reading x
    int splits; int64_t split_stride; int64_t partial_stride0;
    const uint16_t* x; int64_t x_stride0;
    uint16_t* residual; int64_t residual_stride0;
    const uint16_t* weight;
    uint16_t* out; int64_t out_stride0;
    int chunks;       // hidden / 8
    float inv_hidden;
    float eps;
};

// One workgroup of 512 threads per row (one or two 16-byte chunks per thread: many loads in flight).  The row (plus residual) is held in registers as float32 between the two
// passes, so each input byte is read once.  Rounding points of the reference: the residual output
// is bf16(x + residual) while the variance and the scaling use the unrounded float32 sum; the
// scaled value is rounded to bf16 and then multiplied by the bf16 weight (rounded again).
__global__ void __launch_bounds__(kNormThreads) rms_norm_kernel(NormArgs a) {
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const uint16_t* xr = a.x + row * a.x_stride0;
    uint16_t* rr = a.residual ? a.residual + row * a.residual_stride0 : nullptr;

    // the weights do not depend on the reduction: fetch them with the first round of loads
    u32x4 wv[kNormMaxChunks];
#pragma unroll
    for (int j = 0; j < kNormMaxChunks; ++j) {
        const int c = tid + j * kNormThreads;
        if (c < a.chunks) wv[j] = *reinterpret_cast<const u32x4*>(a.weight + 8 * c);
    }
    float v[kNormMaxChunks][8];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kNormMaxChunks; ++j) {
        const int c = tid + j * kNormThreads;
        if (c < a.chunks) {
            if (a.partial) {
                // split-K partial sums of the producing GEMM, added in split order and rounded to bf16
                // once, exactly as the GEMM's own reduction kernel would have done
                const float* pp = a.partial + row * a.partial_stride0 + 8 * c;
                f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
                for (int s = 0; s < a.splits; ++s) {
                    // plain loads: the two halves of a lane's 32 bytes are two instructions on the same lines
                    lo += *reinterpret_cast<const f32x4*>(pp + s * a.split_stride);
                    hi += *reinterpret_cast<const f32x4*>(pp + s * a.split_stride + 4);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) { v[j][e] = rb(lo[e]); v[j][4 + e] = rb(hi[e]); }
            } else {
                unpack8(*reinterpret_cast<const u32x4*>(xr + 8 * c), v[j]);
            }
            if (rr) {
                float r[8];
                unpack8(*reinterpret_cast<const u32x4*>(rr + 8 * c), r);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[j][e] += r[e];
                *reinterpret_cast<u32x4*>(rr + 8 * c) = pack8(v[j]);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += v[j][e] * v[j][e];
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, 64);
    __shared__ float part[kNormThreads / 64];
    if ((tid & 63) == 0) part[tid >> 6] = ss;
    __syncthreads();
    ss = 0.f;
#pragma unroll
    for (int i = 0; i < kNormThreads / 64; ++i) ss += part[i];
    const float rs = rsqrtf(ss * a.inv_hidden + a.eps);

    uint16_t* orow = a.out + row * a.out_stride0;
#pragma unroll
    for (int j = 0; j < kNormMaxChunks; ++j) {
        const int c = tid + j * kNormThreads;
        if (c < a.chunks) {
            float w[8], o[8];
            unpack8(wv[j], w);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = rb(v[j][e] * rs) * w[e];
            *reinterpret_cast<u32x4*>(orow + 8 * c) = pack8(o);
        }
    }
}

struct SiluArgs {
    uint16_t* out; int64_t out_stride0;
    const uint16_t* x; int64_t x_stride0;
    int chunks;            // d / 8
    int64_t total;         // rows * chunks
};

// out[r, j] = bf16(silu(x[r, j])) * x[r, d + j], the product rounded to bf16.
__global__ void __launch_bounds__(256) silu_and_mul_kernel(SiluArgs a) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= a.total) return;
    const int64_t row = i / a.chunks;
    const int c = (int)(i - row * a.chunks);
    const uint16_t* xr = a.x + row * a.x_stride0;
    float g[8], u[8], o[8];
    unpack8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr + 8 * c)), g);
    unpack8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr + 8 * (a.chunks + c))), u);
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = rb(g[e] / (1.0f + expf(-g[e]))) * u[e];
    *reinterpret_cast<u32x4*>(a.out + row * a.out_stride0 + 8 * c) = pack8(o);
}

struct MetaArgs {
    const int32_t* seq_lens;
    const int32_t* block_table; int64_t bt_stride0;
    int batch, block_size, table_cols;
    int64_t position_offset;
    int64_t* positions;
    int32_t* slot_mapping;
    int32_t* context_lens;
};

__global__ void __launch_bounds__(256) decode_metadata_kernel(MetaArgs a) {
    const int b = blockIdx.x * 256 + threadIdx.x;
    if (b >= a.batch) return;
    const int len = a.seq_lens[b];
    int32_t slot = -1, ctx = 0;
    int64_t pos = 0;
    if (len > 0) {
        const int last = len - 1;
        const int col = last / a.block_size;
        ctx = len;
        pos = (int64_t)last + a.position_offset;
        if (col < a.table_cols) {
            const int32_t blk = a.block_table[b * a.bt_stride0 + col];
            if (blk >= 0) slot = blk * a.block_size + (last - col * a.block_size);
        }
    }
    a.positions[b] = pos;
    a.slot_mapping[b] = slot;
    a.context_lens[b] = ctx;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

extern "C" int infer_rms_norm_bf16(const void* x, int64_t x_stride0, void* residual, int64_t residual_stride0,
                                   const void* weight, void* out, int64_t out_stride0, int64_t n_rows,
                                   int64_t hidden, float eps, void* stream) {
    if (n_rows < 0 || hidden <= 0) return INFER_KV_EINVAL;
    if (n_rows == 0) return INFER_KV_OK;
    if (!x || !weight || !out) return INFER_KV_EINVAL;
    if (hidden % 8 != 0 || hidden > 8 * kNormThreads * kNormMaxChunks) return INFER_KV_EUNSUPPORTED;
    if (n_rows > 0x7fffffff) return INFER_KV_EINVAL;
    if (x_stride0 < hidden || out_stride0 < hidden || (residual && residual_stride0 < hidden)) return INFER_KV_EINVAL;
    if (!aligned16(x) || !aligned16(weight) || !aligned16(out) || !aligned16(residual) || x_stride0 % 8 ||
        out_stride0 % 8 || (residual && residual_stride0 % 8))
        return INFER_KV_EALIGN;
    NormArgs a{nullptr, 0, 0, 0, (const uint16_t*)x, x_stride0, (uint16_t*)residual, residual_stride0,
               (const uint16_t*)weight, (uint16_t*)out, out_stride0, (int)(hidden / 8), 1.0f / (float)hidden, eps};
    hipLaunchKernelGGL(rms_norm_kernel, dim3((unsigned)n_rows), dim3(kNormThreads), 0, (hipStream_t)stream, a);
    return (int)hipGetLastError();
}

extern "C" int infer_rms_norm_splitk_bf16(const float* partial, int64_t splits, int64_t split_stride,
                                          int64_t partial_stride0, void* residual, int64_t residual_stride0,
                                          const void* weight, void* out, int64_t out_stride0, int64_t n_rows,
                                          int64_t hidden, float eps, void* stream) {
    if (n_rows < 0 || hidden <= 0 || splits <= 0 || splits > 64) return INFER_KV_EINVAL;
    if (n_rows == 0) return INFER_KV_OK;
    if (!partial || !weight || !out) return INFER_KV_EINVAL;
    if (hidden % 8 != 0 || hidden > 8 * kNormThreads * kNormMaxChunks) return INFER_KV_EUNSUPPORTED;
    if (n_rows > 0x7fffffff) return INFER_KV_EINVAL;
    if (partial_stride0 < hidden || out_stride0 < hidden || (residual && residual_stride0 < hidden)) return INFER_KV_EINVAL;
    if (splits > 1 && split_stride < n_rows * partial_stride0) return INFER_KV_EINVAL;
    if (!aligned16(partial) || !aligned16(weight) || !aligned16(out) || !aligned16(residual) || partial_stride0 % 4 ||
        split_stride % 4 || out_stride0 % 8 || (residual && residual_stride0 % 8))
        return INFER_KV_EALIGN;
    NormArgs a{partial, (int)splits, split_stride, partial_stride0, nullptr, 0, (uint16_t*)residual, residual_stride0,
               (const uint16_t*)weight, (uint16_t*)out, out_stride0, (int)(hidden / 8), 1.0f / (float)hidden, eps};
    hipLaunchKernelGGL(rms_norm_kernel, dim3((unsigned)n_rows), dim3(kNormThreads), 0, (hipStream_t)stream, a);
    return (int)hipGetLastError();
}

extern "C" int infer_silu_and_mul_bf16(void* out, int64_t out_stride0, const void* x, int64_t x_stride0,
                                       int64_t n_rows, int64_t d, void* stream) {
    if (n_rows < 0 || d <= 0) return INFER_KV_EINVAL;
    if (n_rows == 0) return INFER_KV_OK;
    if (!out || !x) return INFER_KV_EINVAL;
    if (d % 8 != 0) return INFER_KV_EUNSUPPORTED;
    if (out_stride0 < d || x_stride0 < 2 * d) return INFER_KV_EINVAL;
    if (!aligned16(out) || !aligned16(x) || out_stride0 % 8 || x_stride0 % 8) return INFER_KV_EALIGN;
    const int64_t total = n_rows * (d / 8);
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffff) return INFER_KV_EINVAL;
    SiluArgs a{(uint16_t*)out, out_stride0, (const uint16_t*)x, x_stride0, (int)(d / 8), total};
    hipLaunchKernelGGL(silu_and_mul_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a);
    return (int)hipGetLastError();
}

extern "C" int infer_decode_metadata(const int32_t* seq_lens, const int32_t* block_table, int64_t bt_stride0,
                                     int64_t batch, int64_t block_size, int64_t table_cols,
                                     int64_t position_offset, int64_t* positions, int32_t* slot_mapping,
                                     int32_t* context_lens, void* stream) {
    if (batch < 0 || block_size <= 0 || table_cols < 0 || bt_stride0 < table_cols) return INFER_KV_EINVAL;
    if (batch == 0) return INFER_KV_OK;
    if (!seq_lens || !block_table || !positions || !slot_mapping || !context_lens) return INFER_KV_EINVAL;
    if (batch > (1 << 24) || block_size > (1 << 20) || table_cols > 0x7fffffff) return INFER_KV_EINVAL;
    MetaArgs a{seq_lens, block_table, bt_stride0, (int)batch, (int)block_size, (int)table_cols, position_offset,
               positions, slot_mapping, context_lens};
    hipLaunchKernelGGL(decode_metadata_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, a);
    return (int)hipGetLastError();
}
