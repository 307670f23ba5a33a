// Split-K weight-streaming GEMM for decode-sized batches on gfx950 (MI355X):
//
//     y[M, N] = x[M, K] . w[N, K]^T          bf16 in, float32 accumulate, bf16 out,  M <= 128
//
// This is `Linear.forward` (infer/ops/MLP.py:103-149, `F.linear`; the op `matmul(input, weight,
// output)` of src/bindings.cpp:7) at the shapes of a decode step whose weight matrix has few rows
// (o_proj, down_proj: N = hidden size).  There a tiled library GEMM has too few output tiles to keep
// 256 compute units streaming; this kernel cuts K as well, so that every unit reads its share of
// the weights exactly once, and pays for it with float32 partial sums that a second kernel adds.
//
// * Grid = (N / 128) x SK.  A workgroup owns 128 weight rows and one K slice; its four wavefronts
//   own two 16-row MFMA tiles each.
// * Weight fragments go from global memory straight into MFMA A-operand registers (16x16x32: lane
//   (j, g) holds w[row j][k0 + 8 g .. + 7], 16 bytes, 64 contiguous bytes per row and instruction),
//   two 128-wide K chunks ahead of use (a ring of three register slots); they are never staged.
//   Plain loads: every 128-byte line is touched by two consecutive instructions, and with the
//   streaming hint some lines are fetched twice (down_proj at 128 rows 34.2 us with the hint, 32.1
//   without; 24.3 and 21.9 us at 16 rows).
// * The activations of a chunk ([M, 128], hot in L2) are staged in LDS once per workgroup (double
//   buffered, 272-byte rows: conflict-free for 16-byte reads of consecutive rows) and read as B
//   operands; every fragment read feeds both row tiles of the wavefront, which halves the LDS
//   traffic per weight byte (LDS delivers 128 B/clk and would otherwise bound the kernel).
// * SK == 1: the accumulators are rounded to bf16 and stored.  SK > 1: float32 partial sums
//   [SK][M][N] go to the workspace and `skinny_gemm_reduce_kernel` adds them and rounds once.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/infer_kv.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kBN = 128;         // weight rows per workgroup
constexpr int kR = 2;            // 16-row weight tiles per wavefront
constexpr int kKC = 128;         // K elements per chunk
constexpr int kXRow = 272;       // LDS bytes per activation row of a chunk (256 + 16)

struct GemmArgs {
    const uint16_t* x; int64_t x_stride0;
    const uint16_t* w;           // [N, K] row-major
    uint16_t* y; int64_t y_stride0;
    float* partial;              // [SK][M][N] when SK > 1
    int m, n, k;
    int chunks;                  // K chunks per split
};

__device__ __forceinline__ u32x4 load16(const uint16_t* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// MT = number of 16-row tiles of the batch (M <= 16 MT)
template <int MT>
__global__ void __launch_bounds__(256) skinny_gemm_kernel(GemmArgs a) {
    __shared__ __attribute__((aligned(16))) unsigned char xs[2][16 * MT * kXRow];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, g = lane >> 4;
    const int split = blockIdx.y;
    const int n0 = blockIdx.x * kBN + wave * 16 * kR;
    const int64_t k_lo = (int64_t)split * a.chunks * kKC;

    // weight streams of this lane: rows n0 + 16 r + j (the tail tile of a ragged N re-reads the last row)
    const uint16_t* wp[kR];
#pragma unroll
    for (int r = 0; r < kR; ++r) {
        const int wrow = n0 + 16 * r + j < a.n ? n0 + 16 * r + j : a.n - 1;
        wp[r] = a.w + (int64_t)wrow * a.k + k_lo + 8 * g;
    }
    // activation staging of this thread: rows (tid >> 4) + 16 i, 16-byte column tid & 15
    const uint16_t* xp[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int r = (tid >> 4) + 16 * i;
        xp[i] = a.x + (int64_t)(r < a.m ? r : a.m - 1) * a.x_stride0 + k_lo + (tid & 15) * 8;
    }
    const int xs_off = (tid >> 4) * kXRow + (tid & 15) * 16;

    u32x4 wreg[3][kR][4];
    u32x4 xreg[MT];
    f32x4 acc[kR][MT];
#pragma unroll
    for (int r = 0; r < kR; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto issue_w = [&](auto SLOT, int c) {
        constexpr int slot = decltype(SLOT)::value;
        // Past the end of the slice every lane requests the same few bytes at the start of the matrix
        // instead (a request that is never used but keeps the count of loads in flight the same on
        // every step, so the waits stay exact): re-reading the last chunk would add 2 chunks of
        // traffic to a slice of 4 to 12.
        const bool live = c < a.chunks;
        const int64_t off = (int64_t)c * kKC;
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint16_t* p = live ? wp[r] + off : a.w;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) wreg[slot][r][kk] = load16(p + 32 * kk);
        }
    };
    auto issue_x = [&](int c) {
        const bool live = c < a.chunks;
#pragma unroll
        for (int i = 0; i < MT; ++i) xreg[i] = load16(live ? xp[i] + c * kKC : a.x);
    };
    auto park_x = [&](int buf) {
#pragma unroll
        for (int i = 0; i < MT; ++i) *reinterpret_cast<u32x4*>(&xs[buf][xs_off + 16 * i * kXRow]) = xreg[i];
    };
    // B fragment of batch tile t at K step kk: lane (j, g) reads x[16 t + j][32 kk + 8 g .. + 7].
    auto compute = [&](auto SLOT, int buf) {
        constexpr int slot = decltype(SLOT)::value;
        const unsigned char* xb = &xs[buf][j * kXRow + 16 * g];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            u32x4 frag[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) frag[t] = *reinterpret_cast<const u32x4*>(xb + 16 * t * kXRow + 64 * kk);
            __builtin_amdgcn_sched_barrier(0);      // all reads of the step first, then its MFMAs
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int r = 0; r < kR; ++r)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wreg[slot][r][kk]),
                                                                        as_bf16x8(frag[t]), acc[r][t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // chunk c: weights in ring slot c % 3, activations in LDS buffer c & 1.  The loads of chunk c + 2
    // are issued before chunk c is consumed, so two chunks (16 KiB per wavefront) stay in flight
    // while the MFMAs run: memory latency, not LDS latency, is what has to be hidden.
    using R0 = std::integral_constant<int, 0>;
    using R1 = std::integral_constant<int, 1>;
    using R2 = std::integral_constant<int, 2>;
    issue_x(0);
    issue_w(R0{}, 0);
    issue_w(R1{}, 1);
    park_x(0);
    issue_x(1);
    __syncthreads();
    auto step = [&](auto SLOT, auto AHEAD, int c) {
        issue_w(AHEAD, c + 2);         // into the slot chunk c - 1 has left
        compute(SLOT, c & 1);
        park_x((c + 1) & 1);           // the buffer chunk c - 1 was read from; all waves are past it
        issue_x(c + 2);
        __syncthreads();
    };
    int c = 0;
    for (; c + 2 < a.chunks; c += 3) {
        step(R0{}, R2{}, c);
        step(R1{}, R0{}, c + 1);
        step(R2{}, R1{}, c + 2);
    }
    if (c < a.chunks) step(R0{}, R2{}, c);
    if (c + 1 < a.chunks) step(R1{}, R0{}, c + 1);

    // accumulator element e of lane (j, g) in tile (r, t) is y[16 t + j][n0 + 16 r + 4 g + e]
#pragma unroll
    for (int r = 0; r < kR; ++r) {
        const int ncol = n0 + 16 * r + 4 * g;
        if (ncol >= a.n) continue;          // N is a multiple of 8: a quad is in or out as a whole
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int row = 16 * t + j;
            if (row >= a.m) continue;
            if (a.partial) {
                *reinterpret_cast<f32x4*>(a.partial + ((int64_t)split * a.m + row) * a.n + ncol) = acc[r][t];
            } else {
                union { __bf16 h[4]; u32x2 u; } o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o.h[e] = (__bf16)acc[r][t][e];
                *reinterpret_cast<u32x2*>(a.y + (int64_t)row * a.y_stride0 + ncol) = o.u;
            }
        }
    }
}

struct ReduceArgs {
    const float* partial;
    uint16_t* y; int64_t y_stride0;
    int m, n, splits;
};

// y[row][8 c .. 8 c + 7] = bf16(sum over splits), one thread per 8 outputs
__global__ void __launch_bounds__(256) skinny_gemm_reduce_kernel(ReduceArgs a) {
    const int per_row = a.n / 8;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)a.m * per_row) return;
    const int row = (int)(i / per_row), c = (int)(i - (int64_t)row * per_row);
    f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < a.splits; ++s) {
        const float* p = a.partial + ((int64_t)s * a.m + row) * a.n + 8 * c;
        lo += *reinterpret_cast<const f32x4*>(p);     // plain loads: lo and hi are two instructions on the same lines
        hi += *reinterpret_cast<const f32x4*>(p + 4);
    }
    union { __bf16 h[8]; u32x4 u; } r;
#pragma unroll
    for (int e = 0; e < 4; ++e) { r.h[e] = (__bf16)lo[e]; r.h[4 + e] = (__bf16)hi[e]; }
    *reinterpret_cast<u32x4*>(a.y + (int64_t)row * a.y_stride0 + 8 * c) = r.u;
}

// Split-K factor: a divisor of the chunk count that brings the grid to at least one workgroup per
// compute unit (256 on MI355X) while leaving every split at least four chunks to stream.
int choose_splits(int64_t n, int64_t k) {
    const int64_t tiles = (n + kBN - 1) / kBN;
    const int64_t chunks = k / kKC;
    int best = 1;
    for (int s = 1; s <= 32; ++s) {
        if (chunks % s != 0 || chunks / s < 4) continue;
        best = s;
        if (tiles * s >= 256) break;
    }
    return best;
}

}  // namespace

extern "C" size_t infer_skinny_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k) {
    if (m <= 0 || m > 128 || n <= 0 || k <= 0 || k % kKC != 0) return 0;
    const int s = choose_splits(n, k);
    return s > 1 ? (size_t)s * (size_t)m * (size_t)n * sizeof(float) : 0;
}

namespace {
// Launches the streaming kernel and, if asked and the shape was split, the reduction.  Returns the
// split count through `splits_out`.
int run_gemm(const void* x, int64_t x_stride0, const void* w, void* y, int64_t y_stride0, int64_t m, int64_t n,
             int64_t k, void* workspace, size_t workspace_bytes, bool reduce, int* splits_out, void* stream) {
    if (m < 0 || n <= 0 || k <= 0) return INFER_KV_EINVAL;
    if (splits_out) *splits_out = 0;
    if (m == 0) return INFER_KV_OK;
    if (!x || !w || !y) return INFER_KV_EINVAL;
    if (m > 128 || k % kKC != 0 || n % 8 != 0) return INFER_KV_EUNSUPPORTED;
    if (x_stride0 < k || y_stride0 < n) return INFER_KV_EINVAL;
    if ((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) || (x_stride0 & 7) || (y_stride0 & 7)) return INFER_KV_EALIGN;
    if (n > (1 << 24) || k > (1 << 24)) return INFER_KV_EINVAL;
    const int splits = choose_splits(n, k);
    const size_t need = splits > 1 ? (size_t)splits * (size_t)m * (size_t)n * sizeof(float) : 0;
    if (need && (!workspace || workspace_bytes < need)) return INFER_KV_EWORKSPACE;
    if (need && ((uintptr_t)workspace & 15)) return INFER_KV_EALIGN;
    GemmArgs a{(const uint16_t*)x, x_stride0, (const uint16_t*)w, (uint16_t*)y, y_stride0,
               splits > 1 ? (float*)workspace : nullptr, (int)m, (int)n, (int)k, (int)(k / kKC / splits)};
    const dim3 grid((unsigned)((n + kBN - 1) / kBN), (unsigned)splits);
    hipStream_t st = (hipStream_t)stream;
    if (m <= 16) hipLaunchKernelGGL(skinny_gemm_kernel<1>, grid, dim3(256), 0, st, a);
    else if (m <= 32) hipLaunchKernelGGL(skinny_gemm_kernel<2>, grid, dim3(256), 0, st, a);
    else if (m <= 64) hipLaunchKernelGGL(skinny_gemm_kernel<4>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(skinny_gemm_kernel<8>, grid, dim3(256), 0, st, a);
    int rc = (int)hipGetLastError();
    if (splits_out) *splits_out = splits;
    if (rc != 0 || splits == 1 || !reduce) return rc;
    ReduceArgs r{(const float*)workspace, (uint16_t*)y, y_stride0, (int)m, (int)n, splits};
    const int64_t items = m * (n / 8);
    hipLaunchKernelGGL(skinny_gemm_reduce_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, st, r);
    return (int)hipGetLastError();
}
}  // namespace

extern "C" int infer_skinny_gemm_bf16(const void* x, int64_t x_stride0, const void* w, void* y, int64_t y_stride0,
                                      int64_t m, int64_t n, int64_t k, void* workspace, size_t workspace_bytes,
                                      void* stream) {
    return run_gemm(x, x_stride0, w, y, y_stride0, m, n, k, workspace, workspace_bytes, true, nullptr, stream);
}

extern "C" int infer_skinny_gemm_partial_bf16(const void* x, int64_t x_stride0, const void* w, void* y,
                                              int64_t y_stride0, int64_t m, int64_t n, int64_t k, void* workspace,
                                              size_t workspace_bytes, int* splits_out, void* stream) {
    if (!splits_out) return INFER_KV_EINVAL;
    return run_gemm(x, x_stride0, w, y, y_stride0, m, n, k, workspace, workspace_bytes, false, splits_out, stream);
}
