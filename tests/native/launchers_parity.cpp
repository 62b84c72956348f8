// Native parity program: drives the C++ launcher mirror (include/rivoli_launchers.hpp) with
// plain HIP allocations and streams — no Python, no torch — and checks the results against the
// CPU oracle (oracle/*.h, test infrastructure). The cases follow the reference's own device
// tests in shape: a slab with a sentinel fill, seeded inputs from the reference's Lcg
// (crates/engine/tests/common/reference.rs:141-162), bit-exact comparison of every byte.
// Built by rivoli_amd/build.py, run by tests/test_gpu_native.py.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <vector>

#include "kvcache_oracle.h"
#include "rivoli_launchers.hpp"
#include "rivoli_pagepool.h"
#include "v4cache_oracle.h"

#define HIP_OK(x)                                                                     \
    do {                                                                              \
        hipError_t e_ = (x);                                                          \
        if (e_ != hipSuccess) {                                                       \
            std::fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
            return 2;                                                                 \
        }                                                                             \
    } while (0)

template <class T>
struct DeviceBuf {
    T* p = nullptr;
    size_t n = 0;
    explicit DeviceBuf(size_t count, int fill = 0) : n(count) {
        if (hipMalloc((void**)&p, count * sizeof(T) + 16) != hipSuccess) p = nullptr;
        if (p) (void)hipMemset(p, fill, count * sizeof(T) + 16);
    }
    explicit DeviceBuf(const std::vector<T>& h) : DeviceBuf(h.size()) {
        if (p) (void)hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice);
    }
    ~DeviceBuf() { (void)hipFree(p); }
    std::vector<T> back() const {
        std::vector<T> h(n);
        (void)hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost);
        return h;
    }
};

static int failures = 0;
static void expect(bool ok, const char* what) {
    std::printf("%s %s\n", ok ? "ok  " : "FAIL", what);
    std::fflush(stdout);
    if (!ok) ++failures;
}

int main() {
    int n_dev = 0;
    HIP_OK(hipGetDeviceCount(&n_dev));
    if (n_dev == 0) {
        std::fprintf(stderr, "no GPU\n");
        return 3;
    }
    HIP_OK(hipSetDevice(0));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    // ---- the fp8 paged cache: append, dense gather, top-k, sparse gather --------------------
    const int W = 576, PT = 64, n_seqs = 3, ctx = 1000, n_pages = 64, k = 128;
    const int blocks = (ctx + PT - 1) / PT;
    uint64_t lcg = 0x5EED0009ull;
    std::vector<float> x((size_t)n_seqs * ctx * W);
    ro_lcg_fill(&lcg, x.data(), x.size());
    for (size_t r = 0; r < (size_t)n_seqs * ctx; r += 97)
        for (int i = 0; i < W; ++i) x[r * W + i] *= 50.0f;  // outlier rows
    std::vector<uint16_t> rows(x.size());
    ro_f32_to_bf16_n(x.data(), rows.data(), x.size());
    // pages from the host allocator, interleaved between the sequences so that tables mix
    rivoli_pagepool* pool_alloc = rivoli_pagepool_create(n_pages, PT);
    std::vector<int> seq_ids(n_seqs), slots((size_t)n_seqs * ctx);
    for (int s = 0; s < n_seqs; ++s) seq_ids[s] = rivoli_pagepool_seq_create(pool_alloc);
    for (int t0 = 0; t0 < ctx; t0 += 100)
        for (int s = 0; s < n_seqs; ++s)
            if (rivoli_pagepool_seq_extend(pool_alloc, seq_ids[s], 100, slots.data() + (size_t)s * ctx + t0) != 0) {
                std::fprintf(stderr, "allocator refused\n");
                return 2;
            }
    std::vector<int> table((size_t)n_seqs * blocks, -1), lens(n_seqs, ctx), cu(n_seqs + 1, 0);
    for (int s = 0; s < n_seqs; ++s) {
        rivoli_pagepool_block_table(pool_alloc, seq_ids[s], table.data() + (size_t)s * blocks, blocks);
        cu[s + 1] = cu[s] + lens[s];
    }
    const size_t page_bytes = rivoli::kv_page_bytes(PT, W);
    expect(page_bytes == ro_kv_page_bytes(PT, W), "page size agrees with the oracle");
    std::vector<uint8_t> want_pool(n_pages * page_bytes, 0xA5);
    ro_kv_append_paged(rows.data(), slots.data(), want_pool.data(), n_seqs * ctx, W, PT, n_pages);

    DeviceBuf<uint16_t> d_rows(rows);
    DeviceBuf<int> d_slots(slots), d_table(table), d_lens(lens), d_cu(cu);
    DeviceBuf<uint8_t> d_pool(n_pages * page_bytes, 0xA5);
    DeviceBuf<unsigned int> d_bad(1);
    try {
        rivoli::launch_kv_append_paged(d_rows.p, d_slots.p, d_pool.p, n_seqs * ctx, W, PT, n_pages, d_bad.p, stream);
        HIP_OK(hipStreamSynchronize(stream));
        expect(d_pool.back() == want_pool && d_bad.back()[0] == 0, "kv_append_paged: pool bytes equal the oracle's");

        std::vector<uint16_t> want_out((size_t)n_seqs * ctx * W);
        ro_kv_gather_paged(want_pool.data(), table.data(), lens.data(), cu.data(), want_out.data(), n_seqs, blocks, W, PT);
        DeviceBuf<uint16_t> d_out(want_out.size());
        rivoli::launch_kv_gather_paged(d_pool.p, d_table.p, d_lens.p, d_cu.p, d_out.p, n_seqs, blocks, W, PT, n_pages,
                                       d_bad.p, stream);
        HIP_OK(hipStreamSynchronize(stream));
        expect(d_out.back() == want_out, "kv_gather_paged: gathered bf16 rows equal the oracle's");

        std::vector<float> scores((size_t)n_seqs * ctx);
        ro_lcg_fill(&lcg, scores.data(), scores.size());
        for (size_t i = 0; i < scores.size(); i += 7) scores[i] = 0.25f;  // ties go to the lower index
        std::vector<uint32_t> want_sel((size_t)n_seqs * k);
        ro_topk_batched(scores.data(), n_seqs, ctx, nullptr, ctx, k, want_sel.data(), 1);
        DeviceBuf<float> d_scores(scores);
        DeviceBuf<unsigned int> d_sel((size_t)n_seqs * k);
        rivoli::launch_index_topk_batched(d_scores.p, n_seqs, ctx, (const int*)nullptr, ctx, k, d_sel.p, (void*)nullptr,
                                          stream);
        HIP_OK(hipStreamSynchronize(stream));
        expect(d_sel.back() == want_sel, "index_topk_batched: selections equal the oracle's");

        std::vector<uint16_t> want_picked((size_t)n_seqs * k * W);
        ro_kv_gather_rows_paged(want_pool.data(), table.data(), want_sel.data(), nullptr, want_picked.data(), n_seqs, k,
                                blocks, W, PT);
        DeviceBuf<uint16_t> d_picked(want_picked.size());
        rivoli::launch_kv_gather_rows_paged(d_pool.p, d_table.p, d_sel.p, (const int*)nullptr, d_picked.p, n_seqs, k,
                                            blocks, W, PT, n_pages, d_bad.p, stream);
        HIP_OK(hipStreamSynchronize(stream));
        expect(d_picked.back() == want_picked, "kv_gather_rows_paged: selected rows equal the oracle's");

        // ---- the second cache format: quantize, ring, rectangle, attention -------------------
        const int n_tok = 40, win = 16, ratio = 4, heads = 64, hd = 512, cap = 4;
        const int n_comp = n_tok / ratio;
        std::vector<float> cache((size_t)(n_tok + n_comp) * hd), q((size_t)n_tok * heads * hd), sink(heads),
            blk_scores((size_t)n_tok * n_comp);
        ro_lcg_fill(&lcg, cache.data(), cache.size());
        ro_lcg_fill(&lcg, q.data(), q.size());
        ro_lcg_fill(&lcg, sink.data(), sink.size());
        ro_lcg_fill(&lcg, blk_scores.data(), blk_scores.size());
        std::vector<uint16_t> tmp(std::max(cache.size(), q.size()));
        auto to_bf16_values = [&](std::vector<float>& v) {  // what the model hands over: bf16 values
            ro_f32_to_bf16_n(v.data(), tmp.data(), v.size());
            for (size_t i = 0; i < v.size(); ++i) {
                const uint32_t b = (uint32_t)tmp[i] << 16;
                std::memcpy(&v[i], &b, 4);
            }
        };
        to_bf16_values(cache);
        to_bf16_values(q);
        std::vector<float> want_cache = cache;
        expect(ro_act_quant_f8_prefix(want_cache.data(), want_cache.data(), n_tok + n_comp, hd, hd - 64, 64) == 0,
               "oracle act_quant accepts the shape");
        DeviceBuf<float> d_cache(cache);
        rivoli::launch_act_quant_f8_prefix(d_cache.p, d_cache.p, n_tok + n_comp, hd, hd - 64, 64, stream);
        HIP_OK(hipStreamSynchronize(stream));
        {
            const std::vector<float> got = d_cache.back();
            expect(std::memcmp(got.data(), want_cache.data(), got.size() * 4) == 0,
                   "act_quant_f8_prefix: rows equal the oracle's bit for bit");
        }
        std::vector<float> want_ring((size_t)win * hd, 0.0f);
        ro_ring_write(want_cache.data(), want_ring.data(), win, hd, n_tok, 0);
        DeviceBuf<float> d_ring((size_t)win * hd);
        rivoli::launch_kv_ring_write(d_cache.p, d_ring.p, win, hd, n_tok, 0, stream);
        HIP_OK(hipStreamSynchronize(stream));
        {
            const std::vector<float> got = d_ring.back();
            expect(std::memcmp(got.data(), want_ring.data(), got.size() * 4) == 0, "kv_ring_write: ring equals the oracle's");
        }
        int cols = 0;
        std::vector<int32_t> want_rect((size_t)n_tok * (win + cap));
        expect(ro_sel_gather_scored(blk_scores.data(), n_comp, win, ratio, cap, n_tok, 0, want_rect.data(), &cols) == 0 &&
                   cols == win + cap,
               "oracle rectangle shape");
        DeviceBuf<float> d_blk(blk_scores);
        DeviceBuf<int> d_rect(want_rect.size());
        int got_cols = 0;
        rivoli::launch_sel_gather_scored(d_blk.p, n_comp, win, ratio, cap, n_tok, 0, d_rect.p, &got_cols, stream);
        HIP_OK(hipStreamSynchronize(stream));
        expect(got_cols == cols && d_rect.back() == std::vector<int>(want_rect.begin(), want_rect.end()),
               "sel_gather_scored: rectangle equals the oracle's");
        const float scale = 1.0f / std::sqrt((float)hd);
        std::vector<float> want_o((size_t)n_tok * heads * hd);
        ro_sparse_attn(q.data(), want_cache.data(), sink.data(), want_rect.data(), n_tok, heads, hd, cols, scale,
                       want_o.data());
        DeviceBuf<float> d_q(q), d_sink(sink), d_o(want_o.size());
        rivoli::launch_gather_attn_shared_kv(d_q.p, d_cache.p, d_sink.p, d_rect.p, n_tok, heads, hd, cols, scale, d_o.p,
                                             stream);
        HIP_OK(hipStreamSynchronize(stream));
        {
            const std::vector<float> got = d_o.back();
            double worst = 0.0, top = 0.0;
            for (size_t i = 0; i < got.size(); ++i) {
                worst = std::max(worst, (double)std::fabs(got[i] - want_o[i]));
                top = std::max(top, (double)std::fabs(want_o[i]));
            }
            // the reference's bar for this kernel (crates/engine/tests/kernel_v4_attend.rs:97-106)
            expect(worst <= top / 128.0, "gather_attn_shared_kv: within 1/128 of the largest element of the oracle's");
        }

        // ---- error behaviour: a guard comes back as the reference words it -------------------
        bool threw = false;
        try {
            rivoli::launch_kv_append_paged(d_rows.p, d_slots.p, d_pool.p, 0, W, PT, n_pages, d_bad.p, stream);
        } catch (const rivoli::LaunchError& e) {
            threw = e.code == 1001 && std::string(e.what()) == "kv_append_paged: argument guard rejected (1001)";
        }
        expect(threw, "a rejected argument raises with the reference's wording");
        threw = false;
        try {
            (void)rivoli::sel_shape(8, 0, 512, 3, 5);
        } catch (const rivoli::LaunchError& e) {
            threw = e.code == 1005;
        }
        expect(threw, "a multi-row decode selection is refused (1005)");
        rivoli::device_sync();
    } catch (const rivoli::LaunchError& e) {
        std::fprintf(stderr, "unexpected launch error: %s\n", e.what());
        return 1;
    }
    rivoli_pagepool_destroy(pool_alloc);
    HIP_OK(hipStreamDestroy(stream));
    std::printf("%s\n", failures == 0 ? "native parity ok" : "native parity FAILED");
    return failures == 0 ? 0 : 1;
}
