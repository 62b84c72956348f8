// The body of the sparse row gather (dequant on load with a `rows` list,
// crates/backend/kernels/attn.hip:125,175), shared by the stand-alone kernel and by the DSA
// selection kernel that gathers the rows it has just selected.
#pragma once

#include "codec.hpp"

namespace rk {

__device__ __forceinline__ u32x4 dequant8_bf16(u32x2 codes, float scale) {
    u32x2 a = dequant4_bf16(codes.x, scale);
    u32x2 b = dequant4_bf16(codes.y, scale);
    u32x4 r = {a.x, a.y, b.x, b.y};
    return r;
}

constexpr unsigned long long kSkipRow = ~0ull;

// Token index -> where its codes and its scale sit in the pool (byte offsets), through one
// sequence's block table. A token past the table or on a page outside the pool yields
// kSkipRow, is counted, and the function returns false. The scale itself is NOT fetched here: every thread loads its rows'
// scales together with the codes, so the chain of dependent memory round trips is row list ->
// block table -> data, not one longer.
__device__ __forceinline__ bool resolve_row(unsigned int tok, const int* __restrict__ table,
                                            int max_blocks_per_seq, int width, int pt, int n_pages,
                                            size_t page_bytes, unsigned int* __restrict__ bad_rows,
                                            unsigned long long* base, unsigned long long* scale_at) {
    const unsigned int blk = tok / (unsigned)pt;
    const unsigned int off = tok - blk * (unsigned)pt;
    int page = -1;
    if (blk < (unsigned)max_blocks_per_seq) page = table[blk];
    *base = kSkipRow;
    *scale_at = 0;
    if ((unsigned)page < (unsigned)n_pages) {
        const size_t pbase = (size_t)page * page_bytes;
        *base = pbase + (size_t)off * width;
        *scale_at = pbase + (size_t)pt * width + (size_t)off * 4;
        return true;
    }
    if (bad_rows) atomicAdd(bad_rows, 1u);
    return false;
}

// Streams `cnt` resolved rows (s_base / s_scale_at in LDS, the caller has synchronised) into
// dst, row r at dst + r * width: every lane loads 8 bytes of codes and stores 16 bytes of bf16,
// UNROLL chunks in flight per thread.
// `plain`: no row is skipped and the rows fill THREADS * UNROLL chunks exactly. That form has no
// branch between its loads and its stores, and it matters: with a condition around any of them
// the compiler can no longer count which memory operations are outstanding at the join and
// falls back to waiting for ALL of them before every store — each store then pays a full
// memory round trip behind the previous one.
template <int THREADS, int UNROLL>
__device__ __forceinline__ void stream_rows(const uint8_t* __restrict__ pool,
                                            const unsigned long long* s_base,
                                            const unsigned long long* s_scale_at, int cnt,
                                            int width, bool plain,
                                            uint16_t* __restrict__ dst_rows) {
    const int cpr = width >> 3;
    const int n_chunks = cnt * cpr;
    u32x4* dst = reinterpret_cast<u32x4*>(dst_rows);
    if (plain) {
        u32x2 raw[UNROLL];
        float scl[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int c = (int)threadIdx.x + u * THREADS;
            const int r = c / cpr;
            const int col = c - r * cpr;
            raw[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(pool + s_base[r]) + col);
            scl[u] = *reinterpret_cast<const float*>(pool + s_scale_at[r]);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            __builtin_nontemporal_store(dequant8_bf16(raw[u], scl[u]),
                                        dst + (int)threadIdx.x + u * THREADS);
        return;
    }
    for (int cb = threadIdx.x; cb < n_chunks; cb += THREADS * UNROLL) {
        u32x2 raw[UNROLL];
        float scl[UNROLL];
        bool live[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int c = cb + u * THREADS;
            live[u] = false;
            if (c < n_chunks) {
                const int r = c / cpr;
                const int col = c - r * cpr;
                const unsigned long long base = s_base[r];
                if (base != kSkipRow) {
                    live[u] = true;
                    raw[u] = __builtin_nontemporal_load(
                        reinterpret_cast<const u32x2*>(pool + base) + col);
                    scl[u] = *reinterpret_cast<const float*>(pool + s_scale_at[r]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int c = cb + u * THREADS;
            if (live[u]) __builtin_nontemporal_store(dequant8_bf16(raw[u], scl[u]), dst + c);
        }
    }
}

static inline bool gather_shape_ok(int width, int page_tokens) {
    return (width % 16) == 0 && (page_tokens % 4) == 0;
}

// The sparse gather's launcher (kv_gather.hip), for callers inside the library.
int gather_rows_launch(const unsigned char* pool, const int* block_table, const unsigned int* rows,
                       const int* n_rows, unsigned short* out, int n_queries, int k, int nr_cap,
                       int max_blocks_per_seq, int width, int page_tokens, int n_pages,
                       unsigned int* bad_rows, void* stream);

}  // namespace rk
