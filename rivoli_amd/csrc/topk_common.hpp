// Pieces the DSA selection shares between the kernels that produce its inputs and the ones
// that run it: the order-preserving score key, the geometry of a query split over many
// workgroups, and the layout of the caller's workspace.
#pragma once

#include "codec.hpp"

namespace rk {

// Order-preserving f32 -> u32 with -0.0 folded onto +0.0
// (crates/backend/kernels/indexer.hip:156-159).
__device__ __forceinline__ uint32_t topk_key(float v) {
    uint32_t b = (v == 0.0f) ? 0u : __float_as_uint(v);
    return b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);
}

// The two orders a selection can run under: the DSA rule above, and IEEE total order
// (f32::total_cmp: -0.0 strictly below +0.0, NaNs ordered by sign and payload), which the
// scored block selection of the second cache format uses.
struct FoldedZeroKey {
    static __device__ __forceinline__ uint32_t of(float v) { return topk_key(v); }
};
struct TotalOrderKey {
    static __device__ __forceinline__ uint32_t of(float v) {
        const uint32_t b = __float_as_uint(v);
        return b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);
    }
};

__device__ __forceinline__ uint32_t lanes_below(unsigned long long mask) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// ---- a query split over the chip --------------------------------------------------------------
constexpr int kSegKeys = 4096;           // scores per segment: one workgroup, 4 per thread
constexpr int kSplitThreads = 1024;
constexpr int kSplitWaves = kSplitThreads / kWave;
constexpr int kTopBits = 12;             // key bits the per-query global histogram resolves
constexpr int kTopBins = 1 << kTopBits;
constexpr int kLowBits = 32 - kTopBits;
constexpr int kMaxSegs = 1024;           // segment tables the finishing kernel holds in LDS
constexpr int kSplitMinScores = 16384;   // shorter queries stay on one workgroup

// Workspace, u32 words per query:
//   [0, 4096)            histogram of the keys' top 12 bits (zero between calls)
//   4096, 4097           pivot bin; how many keys of that bin the selection still needs
//   [4100, 4100 + S)     per segment: keys in the pivot bin (the candidates)
//   [4100 + S, 4100+2S)  per segment: keys in higher bins (selected whatever the low bits say)
//   (padded to 4 words)  S x 4096 candidate keys, segment s at s * 4096
//   S x 128              one bit per score: set where the key's bin is above the pivot bin
//                        (queries of up to kBitsMaxSegs segments, see index_topk.hip)
constexpr int kBitsMaxSegs = 64;         // longer queries take the list-only finishing kernel
constexpr int kWsPivot = kTopBins, kWsNeed = kTopBins + 1, kWsCounts = kTopBins + 4;
__host__ __device__ inline int topk_segments(int nt) { return (nt + kSegKeys - 1) / kSegKeys; }
__host__ __device__ inline size_t topk_ws_cand_offset(int n_segs) {
    return ((size_t)kWsCounts + 2 * (size_t)n_segs + 3) & ~(size_t)3;
}
__host__ __device__ inline size_t topk_ws_bits_offset(int n_segs) {
    return topk_ws_cand_offset(n_segs) + (size_t)n_segs * kSegKeys;
}
__host__ __device__ inline size_t topk_ws_words(int n_segs) {
    return topk_ws_bits_offset(n_segs) + (size_t)n_segs * (kSegKeys / 32);
}
// Whether a call of this shape runs split (so whether a producer should fill the histogram).
inline bool topk_runs_split(int n_queries, int nt) {
    return nt > kSplitMinScores && n_queries <= 65535 && topk_segments(nt) <= kMaxSegs;
}

// Adds the histogram of one workgroup's LDS bins (kTopBins of them) to a query's workspace:
// one global atomic per non-empty bin.
__device__ __forceinline__ void flush_top_bins(const uint32_t* s_hist, uint32_t* w, int tid,
                                               int threads) {
    for (int b = tid; b < kTopBins; b += threads) {
        const uint32_t c = s_hist[b];
        if (c) atomicAdd(&w[b], c);
    }
}

}  // namespace rk
