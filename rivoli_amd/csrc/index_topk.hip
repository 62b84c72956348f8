// DSA row selection: for each query, the k best-scoring token indices, emitted ascending.
//
// Rule (crates/core/src/routing.rs:42-61 followed by sort_unstable, and the reference kernel
// crates/backend/kernels/indexer.hip:143-257): order by score descending with -0.0 == +0.0,
// ties by index ascending; take the first min(k, nt); write that SET in index order. Entries
// past min(k, nt) are not written. NaN scores are out of contract on both sides.
//
// Shape: one 1024-thread workgroup (16 wave64) per query, all queries in one launch. Each
// wave owns a contiguous segment of the score array and keeps its order-preserving u32 keys
// in registers (up to 64 per lane = 65536 scores per query), so the scores are read from
// memory once. Selection is a 4-pass, 8-bit, MSB-first radix select of the k-th largest key.
// Score arrays concentrate in a handful of exponent bytes, so each histogram bin is
// replicated 32 times in LDS, one copy per bank (copy = lane mod 32): a wave's 64 atomic
// increments then never collide inside one instruction whatever the digit distribution.
// Compaction needs no atomics: a selected element's slot is
//   (# keys > pivot before it) + min(# keys == pivot before it, need),
// monotone in the index; within a wave those prefixes are ballots and popcounts, across
// waves one 16-entry prefix. Longer arrays (nt > 65536) stream the keys from memory on every
// sweep with the same code.
// Launch-only; see include/rivoli_kvcache.h for the contract of every entry point.
#include "codec.hpp"

namespace rk {

constexpr int kTopkThreads = 1024;
constexpr int kTopkWaves = kTopkThreads / kWave;
constexpr int kBins = 256;
constexpr int kCopies = 32;

// Order-preserving f32 -> u32 with -0.0 folded onto +0.0
// (crates/backend/kernels/indexer.hip:156-159).
__device__ __forceinline__ uint32_t topk_key(float v) {
    uint32_t b = (v == 0.0f) ? 0u : __float_as_uint(v);
    return b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);
}

__device__ __forceinline__ uint32_t lanes_below(unsigned long long mask) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// One sweep over a lane's elements: a compile-time trip count when the keys live in
// registers (so every key[j] is a register, never scratch), a runtime one when streaming.
template <int ITEMS, class F>
__device__ __forceinline__ void sweep(int steps, F&& body) {
    if constexpr (ITEMS > 0) {
#pragma unroll
        for (int j = 0; j < ITEMS; ++j)
            if (j < steps) body(j);
    } else {
        for (int j = 0; j < steps; ++j) body(j);
    }
}

// ITEMS: keys per lane kept in registers; 0 = re-read the scores on every sweep.
template <int ITEMS>
__global__ __launch_bounds__(kTopkThreads) void index_topk_kernel(
    const float* __restrict__ scores, int stride, const int* __restrict__ nts, int nt_all, int k,
    uint32_t* __restrict__ rows) {
    __shared__ uint32_t s_hist[kBins * kCopies];
    __shared__ uint32_t s_bins[kBins];
    __shared__ uint32_t s_wave[kTopkWaves];
    __shared__ uint32_t s_pivot, s_need;

    const int q = blockIdx.x;
    int nt = nts ? min(nts[q], nt_all) : nt_all;
    if (nt <= 0) return;
    const uint32_t kq = (uint32_t)min(k, nt);
    const float* s = scores + (size_t)q * stride;
    uint32_t* out = rows + (size_t)q * k;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    // Each wave owns per_wave consecutive scores, a multiple of 64, walked 64 at a time.
    const int per_wave = ((nt + kTopkThreads - 1) / kTopkThreads) * kWave;
    const int steps = per_wave / kWave;
    const long long seg0 = (long long)wave * per_wave;
    // element (j, lane) is index seg0 + j*64 + lane; it exists iff j*64 < limit
    const long long rem = (long long)nt - seg0;
    const int limit = (int)(rem < per_wave ? rem : per_wave) - lane;

    uint32_t key[ITEMS ? ITEMS : 1];
    if (ITEMS) {
#pragma unroll
        for (int j = 0; j < ITEMS; ++j)
            key[j] = (j * kWave < limit) ? topk_key(s[seg0 + j * kWave + lane]) : 0u;
    }
    auto key_at = [&](int j) -> uint32_t {
        if (ITEMS) return key[j];
        return (j * kWave < limit) ? topk_key(s[seg0 + (long long)j * kWave + lane]) : 0u;
    };

    uint32_t pivot = 0u, mask = 0u, need = kq;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = tid; i < kBins * kCopies; i += kTopkThreads) s_hist[i] = 0u;
        __syncthreads();
        sweep<ITEMS>(steps, [&](int j) {
            const uint32_t u = key_at(j);
            if (j * kWave < limit && (u & mask) == pivot)
                atomicAdd(&s_hist[((u >> shift) & 0xffu) * kCopies + (lane & (kCopies - 1))], 1u);
        });
        __syncthreads();
        {
            // four threads per bin, eight copies each, rotated so a wave spreads over banks
            const int bin = tid >> 2, part = tid & 3;
            uint32_t sum = 0;
#pragma unroll
            for (int c = 0; c < 8; ++c) sum += s_hist[bin * kCopies + part * 8 + ((c + lane) & 7)];
            sum += __shfl_xor(sum, 1, kWave);
            sum += __shfl_xor(sum, 2, kWave);
            if (part == 0) s_bins[bin] = sum;
        }
        __syncthreads();
        if (wave == 0) {
            // lane L owns bins 4L..4L+3. Walk from the top bin down for the one holding the
            // need-th candidate: the lane whose inclusive suffix count first reaches need.
            uint32_t c[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) c[b] = s_bins[lane * 4 + b];
            const uint32_t tot = c[0] + c[1] + c[2] + c[3];
            uint32_t suffix = tot;
#pragma unroll
            for (int off = 1; off < kWave; off <<= 1) {
                uint32_t v = __shfl_down(suffix, off, kWave);
                if (lane + off < kWave) suffix += v;
            }
            const uint32_t above = suffix - tot;
            if (above < need && need <= suffix) {
                uint32_t acc = above;
                int b = 3;
                for (; b > 0; --b) {
                    if (acc + c[b] >= need) break;
                    acc += c[b];
                }
                s_pivot = pivot | ((uint32_t)(lane * 4 + b) << shift);
                s_need = need - acc;
            }
        }
        __syncthreads();
        pivot = s_pivot;
        need = s_need;
        mask |= 0xffu << shift;
    }

    // Per-wave totals of (key > pivot, key == pivot).
    uint32_t cnt_gt = 0, cnt_eq = 0;
    sweep<ITEMS>(steps, [&](int j) {
        const uint32_t u = key_at(j);
        if (j * kWave < limit) {
            cnt_gt += u > pivot ? 1u : 0u;
            cnt_eq += u == pivot ? 1u : 0u;
        }
    });
    const uint32_t gt_total = wave_sum(cnt_gt), eq_total = wave_sum(cnt_eq);
    if (lane == 0) {
        s_wave[wave] = gt_total;
        s_bins[wave] = eq_total;
    }
    __syncthreads();
    uint32_t run_gt = 0, run_eq = 0;
    for (int w = 0; w < wave; ++w) {
        run_gt += s_wave[w];
        run_eq += s_bins[w];
    }
    sweep<ITEMS>(steps, [&](int j) {
        const uint32_t u = key_at(j);
        const bool live = j * kWave < limit;
        const bool g = live && u > pivot;
        const bool e = live && u == pivot;
        const unsigned long long mg = __ballot(g), me = __ballot(e);
        const uint32_t G = run_gt + lanes_below(mg);
        const uint32_t E = run_eq + lanes_below(me);
        const uint32_t slot = G + (E < need ? E : need);
        // slot < kq holds by construction; the compare keeps a wrong pivot from ever
        // turning into a write outside the caller's buffer
        if ((g || (e && E < need)) && slot < kq)
            out[slot] = (uint32_t)(seg0 + (long long)j * kWave + lane);
        run_gt += (uint32_t)__popcll(mg);
        run_eq += (uint32_t)__popcll(me);
    });
}

static int index_topk_launch(const float* scores, int n_queries, int stride, const int* nts,
                             int nt, int k, unsigned int* rows, hipStream_t stream) {
    if (!scores || !rows) return 1001;
    if (n_queries <= 0 || nt <= 0 || k <= 0) return 1001;
    if (stride < nt) return 1002;
    dim3 grid((unsigned)n_queries), block(kTopkThreads);
    (void)hipGetLastError();
    if (nt <= kTopkThreads * 4)
        hipLaunchKernelGGL(index_topk_kernel<4>, grid, block, 0, stream, scores, stride, nts, nt, k,
                           rows);
    else if (nt <= kTopkThreads * 16)
        hipLaunchKernelGGL(index_topk_kernel<16>, grid, block, 0, stream, scores, stride, nts, nt,
                           k, rows);
    else if (nt <= kTopkThreads * 64)
        hipLaunchKernelGGL(index_topk_kernel<64>, grid, block, 0, stream, scores, stride, nts, nt,
                           k, rows);
    else
        hipLaunchKernelGGL(index_topk_kernel<0>, grid, block, 0, stream, scores, stride, nts, nt, k,
                           rows);
    return launch_status();
}

}  // namespace rk

extern "C" int rivoli_index_topk_batched(const float* scores, int n_queries, int stride,
                                         const int* nts, int nt, int k, unsigned int* rows,
                                         void* stream) {
    return rk::index_topk_launch(scores, n_queries, stride, nts, nt, k, rows, (hipStream_t)stream);
}

extern "C" int rivoli_index_topk(const float* scores, int nt, int k, unsigned int* rows) {
    return rk::index_topk_launch(scores, 1, nt, nullptr, nt, k, rows, nullptr);
}
