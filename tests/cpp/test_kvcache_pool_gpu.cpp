// GPU test of infer::KVCachePool<T> feeding the HIP kernels: a pool over DEVICE storage, sequences
// prefetched and extended, K/V rows appended through infer_kv_append_bf16 at the slots the views'
// block tables give, attention run by infer_paged_decode_bf16 straight from the PagedCacheView
// (layer base pointer, strides, block table).  Inputs and results are written to <outdir> as raw
// little-endian arrays; tests/test_kvcache_pool_gpu.py checks them against the CPU oracle.
// Built by infer_amd/csrc/Makefile (host code only: HIP runtime API + libinfer_kv.so).
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "infer_kv.h"
#include "infer_kv/kvcache.hpp"

#define CHECK(c) do { if (!(c)) { std::fprintf(stderr, "CHECK failed line %d: %s\n", __LINE__, #c); return 1; } } while (0)
#define HIP(c) do { hipError_t e_ = (c); if (e_ != hipSuccess) { std::fprintf(stderr, "HIP error line %d: %s\n", __LINE__, hipGetErrorString(e_)); return 1; } } while (0)

static uint16_t bf16_bits(float x) {   // round to nearest even
    uint32_t u;
    std::memcpy(&u, &x, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename V>
static int dump(const std::string& dir, const char* name, const std::vector<V>& v) {
    const std::string path = dir + "/" + name;
    FILE* f = std::fopen(path.c_str(), "wb");
    if (!f) return 1;
    const size_t n = std::fwrite(v.data(), sizeof(V), v.size(), f);
    std::fclose(f);
    return n == v.size() ? 0 : 1;
}

int main(int argc, char** argv) {
    CHECK(argc == 2);
    const std::string outdir = argv[1];
    using Pool = infer::KVCachePool<uint16_t>;
    const size_t bs = 256, D = 128, Hkv = 8, Hq = 32, layers = 2, nblk = 24, layer = 1;
    infer::KVCachePoolConfig cfg(bs, D, Hkv, layers, /*mla=*/false, nblk);
    uint16_t* storage = nullptr;
    const size_t elems = Pool::storage_elements(cfg);
    HIP(hipMalloc((void**)&storage, elems * sizeof(uint16_t)));
    HIP(hipMemset(storage, 0xff, elems * sizeof(uint16_t)));      // NaN patterns wherever nothing was appended
    Pool pool(cfg, storage);

    const std::vector<size_t> ids = {11, 5, 42};
    const std::vector<int32_t> lens = {300, 37, 700};
    const size_t B = ids.size(), dkv = Hkv * D;
    std::mt19937 rng(7);
    std::normal_distribution<float> nd(0.f, 1.f);

    // interleave the sequences' allocation so that their blocks are not contiguous: prefetch a first
    // piece of each, then grow each to its length minus one (the prefill part)
    for (size_t i = 0; i < B; ++i) pool.prefetch_sequence(ids[i], 1);
    for (size_t i = 0; i < B; ++i) pool.extend_sequence(ids[i], (size_t)lens[i] - 1);

    std::vector<uint16_t> k_rows, v_rows;          // all tokens of all sequences, sequence-major
    std::vector<int32_t> row_seq, row_pos;
    for (size_t i = 0; i < B; ++i)
        for (int32_t t = 0; t < lens[i]; ++t) {
            row_seq.push_back((int32_t)i);
            row_pos.push_back(t);
            for (size_t e = 0; e < dkv; ++e) { k_rows.push_back(bf16_bits(nd(rng))); v_rows.push_back(bf16_bits(nd(rng))); }
        }
    const size_t total = row_seq.size();
    uint16_t *d_k, *d_v;
    HIP(hipMalloc((void**)&d_k, total * dkv * 2));
    HIP(hipMalloc((void**)&d_v, total * dkv * 2));
    HIP(hipMemcpy(d_k, k_rows.data(), total * dkv * 2, hipMemcpyHostToDevice));
    HIP(hipMemcpy(d_v, v_rows.data(), total * dkv * 2, hipMemcpyHostToDevice));

    // step 1 (prefill-like): append every token but the last of each sequence; the last rows get slot -1
    auto slots_for = [&](bool last_only) {
        std::vector<int32_t> s(total, -1);
        for (size_t r = 0; r < total; ++r) {
            const size_t i = (size_t)row_seq[r];
            const bool is_last = row_pos[r] == lens[i] - 1;
            if (is_last != last_only) continue;
            const auto view = pool.get_key_cache(ids[i], layer);
            if ((size_t)row_pos[r] >= view.length) return std::vector<int32_t>();      // the view must cover the token
            s[r] = view.block_table[row_pos[r] / (int32_t)view.block_size] * (int32_t)view.block_size +
                   row_pos[r] % (int32_t)view.block_size;
        }
        return s;
    };
    int32_t* d_slots;
    HIP(hipMalloc((void**)&d_slots, total * 4));
    const auto kview0 = pool.get_key_cache(ids[0], layer);
    const auto vview0 = pool.get_value_cache(ids[0], layer);
    CHECK(kview0.base != vview0.base && kview0.base == storage + (0 * layers + layer) * nblk * bs * dkv);
    std::vector<int32_t> slots1 = slots_for(false);
    CHECK(slots1.size() == total);
    HIP(hipMemcpy(d_slots, slots1.data(), total * 4, hipMemcpyHostToDevice));
    CHECK(infer_kv_append_bf16(d_k, (int64_t)dkv, d_v, (int64_t)dkv, kview0.base, vview0.base, d_slots, (int64_t)total,
                               (int64_t)dkv, (int64_t)(nblk * bs), nullptr) == 0);
    // step 2 (decode-like): every sequence grows by one token; 300 -> stays in its block, 37 too, 700 too;
    // a fourth sequence is added and freed in between so that the free list is not in its initial order
    pool.prefetch_sequence(99, 3 * bs);
    pool.free_sequence(99);
    for (size_t i = 0; i < B; ++i) pool.extend_sequence(ids[i], (size_t)lens[i]);
    std::vector<int32_t> slots2 = slots_for(true);
    CHECK(slots2.size() == total);
    HIP(hipMemcpy(d_slots, slots2.data(), total * 4, hipMemcpyHostToDevice));
    CHECK(infer_kv_append_bf16(d_k, (int64_t)dkv, d_v, (int64_t)dkv, kview0.base, vview0.base, d_slots, (int64_t)total,
                               (int64_t)dkv, (int64_t)(nblk * bs), nullptr) == 0);

    // step 3: decode attention from the views
    size_t cols = 0;
    std::vector<infer::PagedCacheView<uint16_t>> kviews, vviews;
    for (size_t i = 0; i < B; ++i) {
        kviews.push_back(pool.get_key_cache(ids[i], layer));
        vviews.push_back(pool.get_value_cache(ids[i], layer));
        CHECK(kviews[i].length == (size_t)lens[i] && kviews[i].num_blocks_used == (lens[i] + bs - 1) / bs);
        CHECK(kviews[i].base == kview0.base && vviews[i].base == vview0.base);
        if (kviews[i].num_blocks_used > cols) cols = kviews[i].num_blocks_used;
    }
    std::vector<int32_t> table(B * cols, -1);
    for (size_t i = 0; i < B; ++i)
        for (size_t c = 0; c < kviews[i].num_blocks_used; ++c) table[i * cols + c] = kviews[i].block_table[c];
    std::vector<uint16_t> q(B * Hq * D);
    for (auto& x : q) x = bf16_bits(nd(rng));
    uint16_t *d_q, *d_out;
    int32_t *d_table, *d_lens;
    void* d_ws;
    const size_t ws_bytes = infer_paged_decode_workspace_bytes((int64_t)B, (int64_t)Hq, (int64_t)Hkv, (int64_t)D);
    CHECK(ws_bytes > 0);
    HIP(hipMalloc((void**)&d_q, q.size() * 2));
    HIP(hipMalloc((void**)&d_out, q.size() * 2));
    HIP(hipMalloc((void**)&d_table, table.size() * 4));
    HIP(hipMalloc((void**)&d_lens, B * 4));
    HIP(hipMalloc(&d_ws, ws_bytes));
    HIP(hipMemcpy(d_q, q.data(), q.size() * 2, hipMemcpyHostToDevice));
    HIP(hipMemcpy(d_table, table.data(), table.size() * 4, hipMemcpyHostToDevice));
    HIP(hipMemcpy(d_lens, lens.data(), B * 4, hipMemcpyHostToDevice));
    const float scale = 1.0f / std::sqrt((float)D);
    CHECK(infer_paged_decode_bf16(d_q, (int64_t)(Hq * D), kviews[0].base, vviews[0].base, (int64_t)kviews[0].block_stride,
                                  (int64_t)kviews[0].token_stride, d_out, (int64_t)(Hq * D), d_table, (int64_t)cols,
                                  (int64_t)cols, d_lens, (int64_t)B, (int64_t)Hq, (int64_t)Hkv, (int64_t)D, (int64_t)bs,
                                  (int64_t)nblk, scale, 0, d_ws, ws_bytes, nullptr) == 0);
    HIP(hipDeviceSynchronize());

    std::vector<uint16_t> out(q.size()), k_layer(nblk * bs * dkv), v_layer(nblk * bs * dkv);
    HIP(hipMemcpy(out.data(), d_out, out.size() * 2, hipMemcpyDeviceToHost));
    HIP(hipMemcpy(k_layer.data(), kviews[0].base, k_layer.size() * 2, hipMemcpyDeviceToHost));
    HIP(hipMemcpy(v_layer.data(), vviews[0].base, v_layer.size() * 2, hipMemcpyDeviceToHost));
    // the other layer's storage must be untouched
    std::vector<uint16_t> other(nblk * bs * dkv);
    HIP(hipMemcpy(other.data(), storage, other.size() * 2, hipMemcpyDeviceToHost));
    for (uint16_t x : other) CHECK(x == 0xffff);

    // the dense [len, heads, head_size] tensor the reference's getters promise is one gather call on a view
    std::vector<uint16_t> dense_k;
    for (size_t i = 0; i < B; ++i) {
        int32_t* d_row;
        uint16_t* d_dense;
        HIP(hipMalloc((void**)&d_row, kviews[i].num_blocks_used * 4));
        HIP(hipMalloc((void**)&d_dense, (size_t)lens[i] * dkv * 2));
        HIP(hipMemcpy(d_row, kviews[i].block_table, kviews[i].num_blocks_used * 4, hipMemcpyHostToDevice));
        CHECK(infer_kv_gather_bf16(kviews[i].base, d_row, (int64_t)kviews[i].length, (int64_t)dkv, (int64_t)bs, (int64_t)nblk,
                                   d_dense, nullptr) == 0);
        std::vector<uint16_t> host((size_t)lens[i] * dkv);
        HIP(hipMemcpy(host.data(), d_dense, host.size() * 2, hipMemcpyDeviceToHost));
        dense_k.insert(dense_k.end(), host.begin(), host.end());
        HIP(hipFree(d_row));
        HIP(hipFree(d_dense));
    }
    CHECK(dense_k == k_rows);      // sequence-major rows, exactly what was appended

    std::vector<int64_t> meta = {(int64_t)B, (int64_t)Hq, (int64_t)Hkv, (int64_t)D, (int64_t)bs, (int64_t)nblk,
                                 (int64_t)cols, (int64_t)total};
    CHECK(!dump(outdir, "meta.i64", meta) && !dump(outdir, "q.u16", q) && !dump(outdir, "out.u16", out));
    CHECK(!dump(outdir, "k_rows.u16", k_rows) && !dump(outdir, "v_rows.u16", v_rows));
    CHECK(!dump(outdir, "k_layer.u16", k_layer) && !dump(outdir, "v_layer.u16", v_layer));
    CHECK(!dump(outdir, "table.i32", table) && !dump(outdir, "lens.i32", lens));
    CHECK(!dump(outdir, "slots1.i32", slots1) && !dump(outdir, "slots2.i32", slots2));
    pool.free_sequence(ids[0]);
    pool.free_sequence(ids[1]);
    pool.free_sequence(ids[2]);
    CHECK(pool.free_blocks() == nblk);
    std::puts("ok");
    return 0;
}
