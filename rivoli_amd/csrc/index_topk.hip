// DSA row selection: for each query, the k best-scoring token indices, emitted ascending.
//
// Rule (crates/core/src/routing.rs:42-61 followed by sort_unstable, and the reference kernel
// crates/backend/kernels/indexer.hip:143-257): order by score descending with -0.0 == +0.0,
// ties by index ascending; take the first min(k, nt); write that SET in index order. Entries
// past min(k, nt) are not written. NaN scores are out of contract on both sides.
//
// Two shapes share one selection rule.
//
// (1) One workgroup per query (`topk_block`): each wave owns a contiguous segment of the
//     score array and keeps its order-preserving u32 keys in registers (up to 64 per lane),
//     so the scores are read once. Selection is a 4-pass, 8-bit, MSB-first radix select of the
//     k-th largest key. Score arrays concentrate in a handful of exponent bytes, so each
//     histogram bin is replicated 32 times in LDS, one copy per bank (copy = lane mod 32): a
//     wave's 64 atomic increments never collide inside one instruction whatever the digit
//     distribution. Compaction needs no atomics: a selected element's slot is
//       (# keys > pivot before it) + min(# keys == pivot before it, need),
//     monotone in the index; within a wave those prefixes are ballots and popcounts, across
//     waves one short prefix. It needs no scratch memory, so it serves the reference-signature
//     entry point; but 65536 keys x several sweeps on ONE compute unit is issue-bound.
//
// (2) Split across the chip (`topk_hist_kernel` + `topk_select_kernel`), used when the caller
//     supplies a workspace: every 4096-score segment of every query gets its own workgroup.
//     Kernel A histograms the top 12 key bits per query in global memory (LDS histogram first,
//     then one atomic per non-empty bin); the LAST workgroup of a query to finish — decided by
//     a ticket, never by waiting — walks the histogram for the bin that holds the k-th key.
//     Kernel B writes, per segment and in index order, the indices whose key is in that bin or
//     above (at least k of them, typically ~1.5 k); the last workgroup of the query pulls those
//     candidates into LDS, finishes the radix select on the low 20 bits among the bin's
//     members, and emits the selection in index order. If the candidates do not fit in LDS
//     (degenerate score arrays: huge ties) that workgroup runs shape (1) over the query
//     instead — slower, same answer. The workspace is left zeroed for the next call.
// Launch-only; see include/rivoli_kvcache.h for the contract of every entry point.
#include <type_traits>

#include "codec.hpp"

namespace rk {

constexpr int kBins = 256;
constexpr int kCopies = 32;

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

// A load that other workgroups' writes (made visible by a fence + ticket) are seen by.
__device__ __forceinline__ uint32_t load_agent(const uint32_t* p) {
    return __hip_atomic_load(const_cast<uint32_t*>(p), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
}

// One sweep over a lane's elements: a compile-time trip count when the keys live in
// registers (so every key[j] is a register, never scratch), a runtime one when streaming.
template <int ITEMS, class F>
__device__ __forceinline__ void sweep(int steps, F&& body) {
    if constexpr (ITEMS > 0) {
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            if (j < steps) body(j);
            // keep each step's temporaries from being hoisted across steps: with 64 keys per
            // lane live, the register budget (128 at 1024 threads) has no room for that
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
        for (int j = 0; j < steps; ++j) body(j);
    }
}

// Wave 0 only. bins[256] hold counts; finds the highest bin b with
// (count of bins >= b) >= need and publishes {b, need - count of bins > b} to pn[0..1].
// Exactly one lane publishes when the total is >= need.
__device__ __forceinline__ void find_pivot_bin(const uint32_t* bins, uint32_t need, uint32_t* pn,
                                               int lane) {
    uint32_t c[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) c[b] = bins[lane * 4 + b];
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
        pn[0] = (uint32_t)(lane * 4 + b);
        pn[1] = need - acc;
    }
}

// LDS a workgroup of THREADS needs for topk_block, in u32 words.
template <int THREADS>
constexpr int topk_block_lds_words() {
    return kBins * kCopies + kBins + 2 * (THREADS / kWave) + 2;
}

// Shape (1): the whole selection for one query by one workgroup of THREADS threads.
// ITEMS: keys per lane kept in registers; 0 = re-read the scores on every sweep.
// KEY: the order (FoldedZeroKey or TotalOrderKey); `add` is added to every emitted index.
template <int THREADS, int ITEMS, class KEY = FoldedZeroKey>
__device__ __forceinline__ void topk_block(const float* __restrict__ s, int nt, uint32_t kq,
                                           uint32_t* __restrict__ out, uint32_t* lds,
                                           uint32_t add = 0u) {
    constexpr int WAVES = THREADS / kWave;
    constexpr int TPB = THREADS / kBins;  // threads that share one bin's copies
    static_assert(TPB == 1 || TPB == 4, "256 or 1024 threads");
    uint32_t* s_hist = lds;
    uint32_t* s_bins = s_hist + kBins * kCopies;
    uint32_t* s_gt = s_bins + kBins;
    uint32_t* s_eq = s_gt + WAVES;
    uint32_t* s_pn = s_eq + WAVES;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    // Each wave owns per_wave consecutive scores, a multiple of 64, walked 64 at a time.
    const int per_wave = ((nt + THREADS - 1) / THREADS) * kWave;
    const int steps = per_wave / kWave;
    const long long seg0 = (long long)wave * per_wave;
    // element (j, lane) is index seg0 + j*64 + lane; it exists iff j*64 < limit
    const long long rem = (long long)nt - seg0;
    const int limit = (int)(rem < per_wave ? rem : per_wave) - lane;

    uint32_t key[ITEMS ? ITEMS : 1];
    if constexpr (ITEMS > 0) {
        // A wave whose whole segment exists (wave-uniform test) issues every load off one
        // base register before the first use; only the array's last, partial segment takes
        // the predicated path.
        const float* sp = s + seg0 + lane;
        if (rem >= per_wave) {
#pragma unroll
            for (int j = 0; j < ITEMS; ++j)
                key[j] = j < steps ? __float_as_uint(sp[j * kWave]) : 0u;
#pragma unroll
            for (int j = 0; j < ITEMS; ++j)
                key[j] = j < steps ? KEY::of(__uint_as_float(key[j])) : 0u;
        } else {
#pragma unroll
            for (int j = 0; j < ITEMS; ++j)
                key[j] = (j * kWave < limit) ? KEY::of(sp[j * kWave]) : 0u;
        }
    }
    auto key_at = [&](int j) -> uint32_t {
        if constexpr (ITEMS > 0) return key[j];
        return (j * kWave < limit) ? KEY::of(s[seg0 + (long long)j * kWave + lane]) : 0u;
    };

    uint32_t pivot = 0u, mask = 0u, need = kq;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = tid; i < kBins * kCopies; i += THREADS) s_hist[i] = 0u;
        __syncthreads();
        sweep<ITEMS>(steps, [&](int j) {
            const uint32_t u = key_at(j);
            if (j * kWave < limit && (u & mask) == pivot)
                atomicAdd(&s_hist[((u >> shift) & 0xffu) * kCopies + (lane & (kCopies - 1))], 1u);
        });
        __syncthreads();
        {
            // TPB threads per bin, 32/TPB copies each, rotated so a wave spreads over banks
            constexpr int PER = kCopies / TPB;
            const int bin = tid / TPB, part = tid % TPB;
            uint32_t sum = 0;
#pragma unroll
            for (int c = 0; c < PER; ++c)
                sum += s_hist[bin * kCopies + part * PER + ((c + lane) & (PER - 1))];
            if (TPB == 4) {
                sum += __shfl_xor(sum, 1, kWave);
                sum += __shfl_xor(sum, 2, kWave);
            }
            if (part == 0) s_bins[bin] = sum;
        }
        __syncthreads();
        if (wave == 0) find_pivot_bin(s_bins, need, s_pn, lane);
        __syncthreads();
        pivot |= s_pn[0] << shift;
        need = s_pn[1];
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
        s_gt[wave] = gt_total;
        s_eq[wave] = eq_total;
    }
    __syncthreads();
    uint32_t run_gt = 0, run_eq = 0;
    for (int w = 0; w < wave; ++w) {
        run_gt += s_gt[w];
        run_eq += s_eq[w];
    }
    sweep<ITEMS>(steps, [&](int j) {
        const uint32_t u = key_at(j);
        const bool live = j * kWave < limit;
        const bool g = live && u > pivot;
        const bool e = live && u == pivot;
        const unsigned long long mg = __ballot(g), me = __ballot(e);
        if ((mg | me) == 0ull) return;  // wave-uniform: most steps select nothing
        const uint32_t G = run_gt + lanes_below(mg);
        const uint32_t E = run_eq + lanes_below(me);
        const uint32_t slot = G + (E < need ? E : need);
        // slot < kq holds by construction; the compare keeps a wrong pivot from ever
        // turning into a write outside the caller's buffer
        if ((g || (e && E < need)) && slot < kq)
            out[slot] = (uint32_t)(seg0 + (long long)j * kWave + lane) + add;
        run_gt += (uint32_t)__popcll(mg);
        run_eq += (uint32_t)__popcll(me);
    });
}

constexpr int kTopkThreads = 1024;
constexpr int kTopkWaves = kTopkThreads / kWave;

// Shape (1), lean form for register-resident queries (nt <= 65536). A compute unit issues
// about one wave-instruction per cycle, so what a single workgroup pays for is instructions
// per key; sweeping all keys four times plus two compaction sweeps (topk_block) costs ~110 of
// them. Here all keys are swept three times with a few instructions each — one 10-bit
// histogram pass (1024 bins x 8 bank copies), one count, one ordered compaction of the keys
// in the pivot bin or above into LDS — and everything after that (the remaining 22 bits of
// the radix select, the ordered emission) runs over those few thousand candidates only.
// The histogram window adapts to the data (it starts at the highest bit in which the keys
// differ and descends into the pivot bin while that bin is too full), and a pivot value tied
// more often than LDS can list is emitted straight from the registers.
constexpr int kLeanBits = 10;
constexpr int kLeanBins = 1 << kLeanBits;  // == kTopkThreads: one thread per bin
constexpr int kLeanCopies = 8;
constexpr int kLeanCap = 12288;  // candidates held in LDS (index + key)
static_assert(kLeanBins == kTopkThreads, "one thread per bin");
constexpr int kLeanLdsWords = 2 * kLeanCap + kLeanBins * kLeanCopies + 4 * kTopkWaves + 8;
static_assert(kLeanCap < 65536, "emission packs two counts into 16 bits each");

// Sum over the 16 wave slots of v[w] for w < wave (*before) and over all of them (*all).
// Lanes 0..15 read one slot each and a 4-step butterfly adds them: a couple of registers and
// no dependent chain of LDS reads. Every lane of the wave must call it.
__device__ __forceinline__ void wave_slots_prefix(const uint32_t* v, int wave, uint32_t* before,
                                                  uint32_t* all) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t x = lane < kTopkWaves ? v[lane] : 0u;
    uint32_t a = x, b = lane < wave ? x : 0u;
#pragma unroll
    for (int off = kTopkWaves / 2; off > 0; off >>= 1) {
        a += __shfl_xor(a, off, kWave);
        b += __shfl_xor(b, off, kWave);
    }
    *all = __builtin_amdgcn_readfirstlane(a);
    *before = __builtin_amdgcn_readfirstlane(b);
}

// Min and max over the 16 wave slots of lo[w] / hi[w]; every lane of the wave must call it.
__device__ __forceinline__ void wave_slots_minmax(const uint32_t* lo, const uint32_t* hi,
                                                  uint32_t* mn, uint32_t* mx) {
    const int lane = threadIdx.x & (kWave - 1);
    uint32_t a = lane < kTopkWaves ? lo[lane] : ~0u, b = lane < kTopkWaves ? hi[lane] : 0u;
#pragma unroll
    for (int off = kTopkWaves / 2; off > 0; off >>= 1) {
        a = min(a, (uint32_t)__shfl_xor(a, off, kWave));
        b = max(b, (uint32_t)__shfl_xor(b, off, kWave));
    }
    *mn = __builtin_amdgcn_readfirstlane(a);
    *mx = __builtin_amdgcn_readfirstlane(b);
}

template <int ITEMS>
__device__ __forceinline__ void topk_block_lean(const float* __restrict__ s, int nt, uint32_t kq,
                                                uint32_t* __restrict__ out, uint32_t* lds) {
    uint32_t* c_idx = lds;  // the candidates, in index order
    uint32_t* c_key = lds + kLeanCap;
    uint32_t* s_hist = lds + 2 * kLeanCap;  // later reused as the 256-bin histogram
    uint32_t* s_wa = s_hist + kLeanBins * kLeanCopies;
    uint32_t* s_wb = s_wa + kTopkWaves;
    uint32_t* s_pn = s_wb + kTopkWaves;  // [0] bin, [1] need inside it, [2] its count

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    // the wave index as a scalar: everything derived from it (segment base, bounds, the load
    // addresses' base) then lives in scalar registers instead of one vector register per use
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int per_wave = ((nt + kTopkThreads - 1) / kTopkThreads) * kWave;
    const int steps = per_wave / kWave;
    const int seg0 = wave * per_wave;
    const int rem = nt - seg0;
    const int limit = (rem < per_wave ? rem : per_wave) - lane;
    // Wave-uniform: a wave whose whole segment exists needs no per-key bounds test. Each pass
    // below is instantiated for both cases and the wave picks one.
    const bool full = rem >= per_wave;
    auto both = [&](auto&& pass) {
        if (full) pass(std::true_type{});
        else pass(std::false_type{});
    };

    uint32_t key[ITEMS];
    {
        // a scalar base per step plus one per-lane offset register for all 64 loads
        const float* sw = s + seg0;
        if (full) {  // all issued before the first use
#pragma unroll
            for (int j = 0; j < ITEMS; ++j)
                key[j] = j < steps ? __float_as_uint((sw + j * kWave)[lane]) : 0u;
#pragma unroll
            for (int j = 0; j < ITEMS; ++j)
                key[j] = j < steps ? topk_key(__uint_as_float(key[j])) : 0u;
        } else {
#pragma unroll
            for (int j = 0; j < ITEMS; ++j)
                key[j] = (j * kWave < limit) ? topk_key((sw + j * kWave)[lane]) : 0u;
        }
    }

    // ---- where the keys differ: real score arrays (sums of ReLU'd terms, all positive) sit
    // in two or three binades, so a fixed window on the top bits would put nearly every key
    // in one bin. The histogram window starts at the highest bit in which max and min differ.
    uint32_t kmin = ~0u, kmax = 0u;
    both([&](auto F) {
        sweep<ITEMS>(steps, [&](int j) {
            if (decltype(F)::value || j * kWave < limit) {
                kmin = min(kmin, key[j]);
                kmax = max(kmax, key[j]);
            }
        });
    });
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        kmin = min(kmin, (uint32_t)__shfl_xor(kmin, off, kWave));
        kmax = max(kmax, (uint32_t)__shfl_xor(kmax, off, kWave));
    }
    if (lane == 0) {
        s_wa[wave] = kmin;
        s_wb[wave] = kmax;
    }
    __syncthreads();
    wave_slots_minmax(s_wa, s_wb, &kmin, &kmax);
    const uint32_t diff = kmin ^ kmax;
    const int top = diff ? 31 - __builtin_clz(diff) : 0;  // highest bit that is not common
    int shift = top > kLeanBits - 1 ? top - (kLeanBits - 1) : 0;
    int width = top + 1 - shift;
    uint32_t mask = top == 31 ? 0u : (~0u << (top + 1));  // bits every key shares
    uint32_t prefix = kmax & mask;
    uint32_t need = kq;  // how many are still to be taken from the keys matching `prefix`
    uint32_t total;      // how many keys are >= the pivot bin's first key

    // ---- histogram levels: 10 bits at a time below the common prefix, descending into the
    // pivot bin only while it and everything above it are too many to hold as candidates ----
    uint32_t* my_copy = s_hist + (lane & (kLeanCopies - 1));
    for (;;) {
        __syncthreads();  // s_wa / s_pn / s_hist from the previous use are no longer read
        for (int i = tid; i < kLeanBins * kLeanCopies; i += kTopkThreads) s_hist[i] = 0u;
        __syncthreads();
        const uint32_t dmask = (1u << width) - 1u;
        // (conditional on purpose: with unconditional LDS atomics the compiler runs all 64
        // address computations ahead of them and spills the key registers)
        both([&](auto F) {
            sweep<ITEMS>(steps, [&](int j) {
                if ((decltype(F)::value || j * kWave < limit) && (key[j] & mask) == prefix)
                    atomicAdd(&my_copy[__builtin_amdgcn_ubfe(key[j], shift, width) * kLeanCopies], 1u);
            });
        });
        __syncthreads();
        uint32_t cnt = 0;  // thread tid owns bin tid
#pragma unroll
        for (int c = 0; c < kLeanCopies; ++c)
            cnt += s_hist[tid * kLeanCopies + ((c + lane) & (kLeanCopies - 1))];
        uint32_t suffix = cnt;  // keys in this bin and the higher bins of this wave
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            uint32_t v = __shfl_down(suffix, off, kWave);
            if (lane + off < kWave) suffix += v;
        }
        if (lane == 0) s_wa[wave] = suffix;
        __syncthreads();
        uint32_t lower, all;
        wave_slots_prefix(s_wa, wave + 1, &lower, &all);
        const uint32_t above = all - lower + (suffix - cnt);  // higher waves + higher lanes
        if (above < need && need <= above + cnt) {
            s_pn[0] = (uint32_t)tid;
            s_pn[1] = need - above;
            s_pn[2] = cnt;
        }
        __syncthreads();
        prefix |= s_pn[0] << shift;
        mask |= dmask << shift;
        need = s_pn[1];
        total = kq - need + s_pn[2];  // everything already sure (kq - need) plus the pivot bin
        if (total <= (uint32_t)kLeanCap || shift == 0) break;
        const int next = shift > kLeanBits ? shift - kLeanBits : 0;
        width = shift - next;
        shift = next;
    }

    if (total > (uint32_t)kLeanCap) {
        // Every bit is fixed and the pivot VALUE itself is tied too often to list (e.g. a
        // ReLU-sparse array whose tail is all zeros): emit straight from the registers —
        // every key above the pivot, and the first `need` keys equal to it, in index order.
        const uint32_t pivot = prefix;
        uint32_t cnt_gt = 0, cnt_eq = 0;
        both([&](auto F) {
            sweep<ITEMS>(steps, [&](int j) {
                const bool live = decltype(F)::value || j * kWave < limit;
                cnt_gt += (uint32_t)__popcll(__ballot(live && key[j] > pivot));
                cnt_eq += (uint32_t)__popcll(__ballot(live && key[j] == pivot));
            });
        });
        __syncthreads();
        if (lane == 0) {
            s_wa[wave] = cnt_gt;
            s_wb[wave] = cnt_eq;
        }
        __syncthreads();
        uint32_t run_gt, run_eq, unused;
        wave_slots_prefix(s_wa, wave, &run_gt, &unused);
        wave_slots_prefix(s_wb, wave, &run_eq, &unused);
        uint32_t idx = (uint32_t)(seg0 + lane);
        both([&](auto F) {
            sweep<ITEMS>(steps, [&](int j) {
                const bool live = decltype(F)::value || j * kWave < limit;
                const bool g = live && key[j] > pivot, e = live && key[j] == pivot;
                const unsigned long long mg = __ballot(g), me = __ballot(e);
                const uint32_t G = run_gt + lanes_below(mg), E = run_eq + lanes_below(me);
                const uint32_t slot = G + (E < need ? E : need);
                if ((g || (e && E < need)) && slot < kq) out[slot] = idx;
                run_gt += (uint32_t)__popcll(mg);
                run_eq += (uint32_t)__popcll(me);
                idx += kWave;
                asm volatile("" : "+v"(idx));
            });
        });
        return;
    }

    // ---- candidates per wave (a candidate is key >= the pivot bin's first key) ----
    const uint32_t thr = prefix;
    uint32_t mine = 0;
    both([&](auto F) {
        sweep<ITEMS>(steps, [&](int j) {
            const bool is = (decltype(F)::value || j * kWave < limit) && key[j] >= thr;
            mine += (uint32_t)__popcll(__ballot(is));  // scalar popcount: one VALU op per key
        });
    });
    __syncthreads();
    if (lane == 0) s_wb[wave] = mine;
    __syncthreads();
    uint32_t run, unused;
    wave_slots_prefix(s_wb, wave, &run, &unused);

    // ---- ordered compaction of (index, key) into LDS ----
    // the element index is carried as a running register (a per-step constant would be
    // materialised 64 times over and spill)
    uint32_t idx = (uint32_t)(seg0 + lane);
    both([&](auto F) {
        sweep<ITEMS>(steps, [&](int j) {
            const bool is = (decltype(F)::value || j * kWave < limit) && key[j] >= thr;
            const unsigned long long m = __ballot(is);
            if (is) {
                const uint32_t pos = run + lanes_below(m);
                c_idx[pos] = idx;
                c_key[pos] = key[j];
            }
            run += (uint32_t)__popcll(m);
            idx += kWave;
            asm volatile("" : "+v"(idx));  // keep the add where it is
        });
    });
    __syncthreads();

    // ---- the bits below the last window, among the pivot bin's members, 8 at a time ----
    uint32_t* s_bins = s_hist;
    uint32_t pivot = prefix;
    for (int left = shift; left > 0;) {
        const int take = left < 8 ? left : 8;
        const int sh = left - take;
        const uint32_t dmask = (1u << take) - 1u;
        if (tid < kBins) s_bins[tid] = 0u;
        __syncthreads();
        for (uint32_t c = tid; c < total; c += kTopkThreads) {
            const uint32_t u = c_key[c];
            if ((u & mask) == pivot) atomicAdd(&s_bins[(u >> sh) & dmask], 1u);
        }
        __syncthreads();
        if (wave == 0) find_pivot_bin(s_bins, need, s_pn, lane);
        __syncthreads();
        pivot |= s_pn[0] << sh;
        need = s_pn[1];
        mask |= dmask << sh;
        left = sh;
        __syncthreads();
    }

    // ---- ordered emission: each thread owns a run of consecutive candidates ----
    const uint32_t chunk = (total + kTopkThreads - 1) / kTopkThreads;
    const uint32_t c_lo = min((uint32_t)tid * chunk, total), c_hi = min(c_lo + chunk, total);
    uint32_t my_gt = 0, my_eq = 0;
    for (uint32_t c = c_lo; c < c_hi; ++c) {
        const uint32_t u = c_key[c];
        my_gt += u > pivot ? 1u : 0u;
        my_eq += u == pivot ? 1u : 0u;
    }
    // block-wide exclusive prefix of both counts, packed 16:16 (each total <= kLeanCap)
    const uint32_t packed = my_gt | (my_eq << 16);
    uint32_t incl = packed;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        uint32_t v = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += v;
    }
    if (lane == kWave - 1) s_wa[wave] = incl;
    __syncthreads();
    uint32_t before;
    wave_slots_prefix(s_wa, wave, &before, &unused);
    const uint32_t excl = before + incl - packed;
    uint32_t G = excl & 0xffffu, E = excl >> 16;
    for (uint32_t c = c_lo; c < c_hi; ++c) {
        const uint32_t u = c_key[c];
        const bool g = u > pivot, e = u == pivot;
        const uint32_t slot = G + (E < need ? E : need);
        // slot < kq holds by construction; the compare keeps a wrong pivot from ever
        // turning into a write outside the caller's buffer
        if ((g || (e && E < need)) && slot < kq) out[slot] = c_idx[c];
        G += g ? 1u : 0u;
        E += e ? 1u : 0u;
    }
}

template <int ITEMS>
__global__ __launch_bounds__(kTopkThreads) void index_topk_kernel(
    const float* __restrict__ scores, int stride, const int* __restrict__ nts, int nt_all, int k,
    uint32_t* __restrict__ rows) {
    // static LDS: 128 KiB for the lean form (gfx950 has 160 KiB per workgroup), 33 KiB streaming
    __shared__ uint32_t lds[ITEMS > 0 ? kLeanLdsWords : topk_block_lds_words<kTopkThreads>()];
    const int q = blockIdx.x;
    const int nt = nts ? min(nts[q], nt_all) : nt_all;
    if (nt <= 0) return;
    const float* s = scores + (size_t)q * stride;
    uint32_t* out = rows + (size_t)q * k;
    if constexpr (ITEMS > 0)
        topk_block_lean<ITEMS>(s, nt, (uint32_t)min(k, nt), out, lds);
    else
        topk_block<kTopkThreads, 0>(s, nt, (uint32_t)min(k, nt), out, lds);
}

// ---------------------------------------------------------------------------------------------
// Shape (2): a query split over many workgroups.
// ---------------------------------------------------------------------------------------------
constexpr int kSegThreads = 256;
constexpr int kSegWaves = kSegThreads / kWave;
constexpr int kSegKeys = 4096;                     // scores per workgroup
constexpr int kSegItems = kSegKeys / kSegThreads;  // 16 per thread
constexpr int kTopBits = 12;
constexpr int kTopBins = 1 << kTopBits;  // global histogram bins per query
constexpr int kLowBits = 32 - kTopBits;
constexpr int kCandCap = 8192;  // candidates the finishing workgroup can cache in LDS
constexpr int kMaxSegs = 1024;  // segment prefix table held in LDS

// Workspace, u32 words per query: [0,4096) histogram | 4096 ticket A | 4097 ticket B |
// 4098 pivot bin | 4099 need | [4100, 4100+S) per-segment candidate counts | (pad to 4) |
// S x 4096 candidate indices.
constexpr int kWsTicketA = kTopBins, kWsTicketB = kTopBins + 1, kWsPivot = kTopBins + 2,
              kWsNeed = kTopBins + 3, kWsCounts = kTopBins + 4;
__host__ __device__ inline size_t topk_ws_cand_offset(int n_segs) {
    return ((size_t)kWsCounts + (size_t)n_segs + 3) & ~(size_t)3;
}
static inline size_t topk_ws_words(int n_segs) {
    return topk_ws_cand_offset(n_segs) + (size_t)n_segs * kSegKeys;
}

// A workgroup's 4096 keys: element (j, tid) is index seg*4096 + j*256 + tid.
__device__ __forceinline__ void load_segment_keys(const float* __restrict__ s, int nt, int seg,
                                                  uint32_t (&key)[kSegItems], int& limit) {
    const int base = seg * kSegKeys + (int)threadIdx.x;
    limit = nt - base;  // element j exists iff j*256 < limit
    float raw[kSegItems];
#pragma unroll
    for (int j = 0; j < kSegItems; ++j) {
        int i = base + j * kSegThreads;
        raw[j] = s[i < nt ? i : nt - 1];
    }
#pragma unroll
    for (int j = 0; j < kSegItems; ++j) key[j] = topk_key(raw[j]);
}

// Exclusive prefix sum of one value per thread over a 256-thread workgroup, in thread order;
// *total receives the workgroup sum. tmp holds kSegWaves words. Every thread must call it.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* tmp,
                                                         uint32_t* total) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    uint32_t incl = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        uint32_t t = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += t;
    }
    __syncthreads();  // tmp may still be read from a previous use
    if (lane == kWave - 1) tmp[wave] = incl;
    __syncthreads();
    uint32_t before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kSegWaves; ++w) {
        if (w < wave) before += tmp[w];
        all += tmp[w];
    }
    *total = all;
    return before + incl - v;
}

// True in exactly one workgroup of the n that share `ticket`: the last to arrive. Nobody
// waits: the others simply leave. Every wave first drains its own stores into L2, then ONE
// wave publishes the workgroup's writes device-wide (an L2 write-back is expensive, and 256
// workgroups x 4 waves of them were measured to cost more than the kernel's real work).
__device__ __forceinline__ bool last_to_arrive(uint32_t* ticket, uint32_t n, uint32_t* s_flag) {
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0): this wave's global stores have completed
    __syncthreads();
    if (threadIdx.x < kWave) {
        __threadfence();
        if (threadIdx.x == 0) *s_flag = atomicAdd(ticket, 1u);
    }
    __syncthreads();
    const bool last = *s_flag == n - 1;
    if (last) __threadfence();  // the others' writes are visible after the last ticket
    return last;
}

__global__ __launch_bounds__(kSegThreads) void topk_hist_kernel(
    const float* __restrict__ scores, int stride, const int* __restrict__ nts, int nt_all, int k,
    uint32_t* __restrict__ ws, size_t ws_stride) {
    __shared__ uint32_t s_hist[kTopBins];
    __shared__ uint32_t s_scan[kSegWaves];
    __shared__ uint32_t s_flag;
    const int q = blockIdx.y, seg = blockIdx.x, tid = threadIdx.x;
    const int nt = nts ? min(nts[q], nt_all) : nt_all;
    if (nt <= 0) return;
    const uint32_t kq = (uint32_t)min(k, nt);
    uint32_t* w = ws + (size_t)q * ws_stride;

    for (int i = tid; i < kTopBins; i += kSegThreads) s_hist[i] = 0u;
    __syncthreads();
    if (seg * kSegKeys < nt) {
        uint32_t key[kSegItems];
        int limit;
        load_segment_keys(scores + (size_t)q * stride, nt, seg, key, limit);
#pragma unroll
        for (int j = 0; j < kSegItems; ++j)
            if (j * kSegThreads < limit) atomicAdd(&s_hist[key[j] >> kLowBits], 1u);
    }
    __syncthreads();
    for (int b = tid; b < kTopBins; b += kSegThreads) {
        const uint32_t c = s_hist[b];
        if (c) atomicAdd(&w[b], c);
    }
    if (!last_to_arrive(&w[kWsTicketA], gridDim.x, &s_flag)) return;

    // The query's histogram is complete. Thread t owns bins [16t, 16t+16); find the highest
    // bin b with (count of bins >= b) >= kq.
    constexpr int OWN = kTopBins / kSegThreads;
    uint32_t c[OWN], sum = 0;
#pragma unroll
    for (int m = 0; m < OWN; ++m) {
        c[m] = load_agent(&w[tid * OWN + m]);
        sum += c[m];
    }
    uint32_t all = 0;
    const uint32_t below = block_exclusive_scan(sum, s_scan, &all);
    const uint32_t above = all - below - sum;  // candidates in bins owned by higher threads
    if (above < kq && kq <= above + sum) {
        uint32_t acc = above;
        int m = OWN - 1;
        for (; m > 0; --m) {
            if (acc + c[m] >= kq) break;
            acc += c[m];
        }
        w[kWsPivot] = (uint32_t)(tid * OWN + m);
        w[kWsNeed] = kq - acc;
    }
    // leave the histogram and the ticket zeroed for the next call
#pragma unroll
    for (int m = 0; m < OWN; ++m) w[tid * OWN + m] = 0u;
    if (tid == 0) w[kWsTicketA] = 0u;
}

__global__ __launch_bounds__(kSegThreads) void topk_select_kernel(
    const float* __restrict__ scores, int stride, const int* __restrict__ nts, int nt_all, int k,
    uint32_t* __restrict__ rows, uint32_t* __restrict__ ws, size_t ws_stride) {
    // the finishing workgroup's candidate cache (indices, keys); the fallback's LDS aliases it
    __shared__ uint32_t s_mem[2 * kCandCap];
    __shared__ uint32_t s_pref[kMaxSegs + 1];
    __shared__ uint32_t s_cnt[kSegItems * kSegWaves];
    __shared__ uint32_t s_bins[kBins];
    __shared__ uint32_t s_pn[2];
    __shared__ uint32_t s_flag;
    static_assert(topk_block_lds_words<kSegThreads>() <= 2 * kCandCap, "fallback fits the cache");
    static_assert(kSegItems * kSegWaves == kWave, "one wave scans the (step, wave) counts");

    const int q = blockIdx.y, seg = blockIdx.x, tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    const int n_segs = gridDim.x;
    const int nt = nts ? min(nts[q], nt_all) : nt_all;
    if (nt <= 0) return;
    const uint32_t kq = (uint32_t)min(k, nt);
    const float* s = scores + (size_t)q * stride;
    uint32_t* w = ws + (size_t)q * ws_stride;
    uint32_t* cand = w + topk_ws_cand_offset(n_segs);
    const uint32_t p12 = w[kWsPivot];

    // ---- this segment's candidates (key's top bits >= pivot bin), in index order ----
    uint32_t key[kSegItems];
    int limit = 0;
    if (seg * kSegKeys < nt) {
        load_segment_keys(s, nt, seg, key, limit);
    } else {
#pragma unroll
        for (int j = 0; j < kSegItems; ++j) key[j] = 0u;
    }
    uint32_t rank[kSegItems];
    bool sel[kSegItems];
#pragma unroll
    for (int j = 0; j < kSegItems; ++j) {
        sel[j] = j * kSegThreads < limit && (key[j] >> kLowBits) >= p12;
        const unsigned long long m = __ballot(sel[j]);
        rank[j] = lanes_below(m);
        if (lane == 0) s_cnt[j * kSegWaves + wave] = (uint32_t)__popcll(m);
    }
    __syncthreads();
    if (wave == 0) {  // exclusive scan of the 64 (step, wave) counts, which is element order
        const uint32_t v = s_cnt[lane];
        uint32_t incl = v;
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            uint32_t t = __shfl_up(incl, off, kWave);
            if (lane >= off) incl += t;
        }
        s_cnt[lane] = incl - v;
        if (lane == kWave - 1) w[kWsCounts + seg] = incl;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kSegItems; ++j)
        if (sel[j])
            cand[(size_t)seg * kSegKeys + s_cnt[j * kSegWaves + wave] + rank[j]] =
                (uint32_t)(seg * kSegKeys + j * kSegThreads + tid);
    if (!last_to_arrive(&w[kWsTicketB], (uint32_t)n_segs, &s_flag)) return;

    // ---- the query's last workgroup finishes the selection ----
    if (tid == 0) w[kWsTicketB] = 0u;  // left zeroed for the next call
    uint32_t* out = rows + (size_t)q * k;
    uint32_t total = 0;
    bool cached = n_segs <= kMaxSegs;
    if (cached) {
        // thread t owns `per` consecutive segments: load their counts at once, scan, publish
        constexpr int PER_MAX = kMaxSegs / kSegThreads;
        const int per = (n_segs + kSegThreads - 1) / kSegThreads;
        uint32_t cnt[PER_MAX], mine = 0;
#pragma unroll
        for (int i = 0; i < PER_MAX; ++i) {
            const int sg = tid * per + i;
            cnt[i] = (i < per && sg < n_segs) ? load_agent(&w[kWsCounts + sg]) : 0u;
            mine += cnt[i];
        }
        uint32_t acc = block_exclusive_scan(mine, s_cnt, &total);
#pragma unroll
        for (int i = 0; i < PER_MAX; ++i) {
            const int sg = tid * per + i;
            if (i < per && sg < n_segs) s_pref[sg] = acc;
            acc += cnt[i];
        }
        if (tid == 0) s_pref[n_segs] = total;
        __syncthreads();
        cached = total <= (uint32_t)kCandCap;
    }
    if (!cached) {
        // too many candidates to hold (heavy ties): select over the whole query directly
        topk_block<kSegThreads, 0>(s, nt, kq, out, s_mem);
        return;
    }
    // Pull the candidates into LDS in index order: a group of threads per segment, so no
    // thread has to search for the segment an output position belongs to.
    uint32_t* c_idx = s_mem;
    uint32_t* c_key = s_mem + kCandCap;
    {
        const int tps = n_segs < kSegThreads ? kSegThreads / n_segs : 1;  // threads per segment
        const int groups = kSegThreads / tps;
        const int sub = tid % tps;
        for (int sg = tid / tps; sg < n_segs; sg += groups) {
            const uint32_t base = s_pref[sg], n = s_pref[sg + 1] - base;
            const uint32_t* src = cand + (size_t)sg * kSegKeys;
#pragma unroll 4
            for (uint32_t i = sub; i < n; i += tps) {
                const uint32_t idx = load_agent(&src[i]);
                c_idx[base + i] = idx;
                c_key[base + i] = topk_key(s[idx]);
            }
        }
    }
    __syncthreads();

    // Radix select on the low 20 bits among the pivot bin's members: 8 + 8 + 4 bits.
    uint32_t need = w[kWsNeed];
    uint32_t pivot = p12 << kLowBits, mask = ~0u << kLowBits;
    for (int shift = kLowBits - 8;; shift = shift >= 8 ? shift - 8 : 0) {
        const uint32_t dmask = (shift == 0 && (kLowBits % 8)) ? (1u << (kLowBits % 8)) - 1u : 0xffu;
        s_bins[tid] = 0u;
        __syncthreads();
        for (uint32_t c = tid; c < total; c += kSegThreads) {
            const uint32_t u = c_key[c];
            if ((u & mask) == pivot) atomicAdd(&s_bins[(u >> shift) & dmask], 1u);
        }
        __syncthreads();
        if (wave == 0) find_pivot_bin(s_bins, need, s_pn, lane);
        __syncthreads();
        pivot |= s_pn[0] << shift;
        need = s_pn[1];
        mask |= dmask << shift;
        __syncthreads();
        if (shift == 0) break;
    }

    // Ordered emission: 256 candidates per round, running (gt, eq) counts carried across.
    uint32_t run_gt = 0, run_eq = 0;
    for (uint32_t c0 = 0; c0 < total; c0 += kSegThreads) {
        const uint32_t c = c0 + tid;
        const bool live = c < total;
        const uint32_t u = live ? c_key[c] : 0u;
        const bool g = live && u > pivot, e = live && u == pivot;
        const unsigned long long mg = __ballot(g), me = __ballot(e);
        if (lane == 0) {
            s_cnt[wave] = (uint32_t)__popcll(mg);
            s_cnt[kSegWaves + wave] = (uint32_t)__popcll(me);
        }
        __syncthreads();
        uint32_t G = run_gt + lanes_below(mg), E = run_eq + lanes_below(me);
        for (int wv = 0; wv < kSegWaves; ++wv) {
            if (wv < wave) {
                G += s_cnt[wv];
                E += s_cnt[kSegWaves + wv];
            }
            run_gt += s_cnt[wv];
            run_eq += s_cnt[kSegWaves + wv];
        }
        const uint32_t slot = G + (E < need ? E : need);
        if ((g || (e && E < need)) && slot < kq) out[slot] = c_idx[c];
        __syncthreads();
    }
}

static int index_topk_launch(const float* scores, int n_queries, int stride, const int* nts,
                             int nt, int k, unsigned int* rows, void* workspace,
                             hipStream_t stream) {
    if (!scores || !rows) return 1001;
    if (n_queries <= 0 || nt <= 0 || k <= 0) return 1001;
    if (stride < nt) return 1002;
    (void)hipGetLastError();
    const int n_segs = (nt + kSegKeys - 1) / kSegKeys;
    // A query that fits one workgroup's registers (<= 65536 scores) is fastest there; longer
    // ones are split over the chip when the caller brought a workspace. 65535 bounds grid.y.
    if (workspace && nt > kTopkThreads * 64 && n_queries <= 65535) {
        const size_t ws_stride = topk_ws_words(n_segs);
        dim3 grid((unsigned)n_segs, (unsigned)n_queries), block(kSegThreads);
        hipLaunchKernelGGL(topk_hist_kernel, grid, block, 0, stream, scores, stride, nts, nt, k,
                           (uint32_t*)workspace, ws_stride);
        hipLaunchKernelGGL(topk_select_kernel, grid, block, 0, stream, scores, stride, nts, nt, k,
                           rows, (uint32_t*)workspace, ws_stride);
        return launch_status();
    }
    dim3 grid((unsigned)n_queries), block(kTopkThreads);
    if (nt <= kTopkThreads * 4)
        hipLaunchKernelGGL(index_topk_kernel<4>, grid, block, 0, stream, scores, stride, nts,
                           nt, k, rows);
    else if (nt <= kTopkThreads * 16)
        hipLaunchKernelGGL(index_topk_kernel<16>, grid, block, 0, stream, scores, stride,
                           nts, nt, k, rows);
    else if (nt <= kTopkThreads * 64)
        hipLaunchKernelGGL(index_topk_kernel<64>, grid, block, 0, stream, scores, stride,
                           nts, nt, k, rows);
    else
        hipLaunchKernelGGL(index_topk_kernel<0>, grid, block, 0, stream, scores, stride,
                           nts, nt, k, rows);
    return launch_status();
}

// ---------------------------------------------------------------------------------------------
// Scored block selection of the second cache format (crates/engine/src/v4/select.rs:153-188,
// done on the host there): query row t keeps the min(k, limit_t) best of its first limit_t
// block scores under IEEE total order, ties to the lower block, and lists them ascending as
// block + offset, then -1 out to k columns. limit_t = min((t + 1) / ratio, n_comp) at prefill
// (a block is legal once it has closed), n_comp at decode. Where limit_t <= k the row is the
// positional fill offset .. offset + limit_t - 1 whatever the scores say.
// ---------------------------------------------------------------------------------------------
//
// A prefill asks for thousands of short selections at once (a row has at most n_comp scores,
// a few thousand), the opposite of the one long query topk_block is built for: its replicated
// LDS histograms cost more to clear and fold than such a row costs to read. select_bisect
// keeps a row's keys in registers (a wave owns a contiguous run, 64 per step) and finds the
// k-th largest key in two stages. The top 10 bits (sign, exponent, first mantissa bit) come
// from one plain 1024-bin LDS histogram, one atomic per key, walked from the top by one wave.
// The other 22 bits are found by bisection, most significant first — count the keys >=
// candidate, keep the bit when enough remain, stop as soon as a count is exactly what is
// needed (on distinct scores after ~log2(spread / spacing) bits) — over the members of the
// pivot bin only: they are listed in LDS (over the histogram, which is no longer needed) and
// one wave bisects them from its registers, a handful per lane. A bin too full to list (heavy
// ties) is bisected over all the keys instead. The selection is then emitted in index order
// by ballots and prefix counts.
//
constexpr int kSelBits = 10;               // key bits resolved by the histogram
constexpr int kSelBins = 1 << kSelBits;
constexpr int kSelLow = 32 - kSelBits;
constexpr int kSelCand = 1024;             // pivot-bin members listed in LDS
constexpr int kSelMisc = 4 * 16 + 8;       // per-wave slots (up to 16 waves) and the pivot record
constexpr int kSelLdsWords = kSelMisc + (kSelBins > kSelCand ? kSelBins : kSelCand);

template <int WAVES, int ITEMS, class KEY>
__device__ __forceinline__ void select_bisect(const float* __restrict__ s, int nt, uint32_t kq,
                                              uint32_t* __restrict__ out, uint32_t* lds,
                                              uint32_t add) {
    // requires 1 <= kq < nt <= WAVES * 64 * ITEMS; lds holds kSelLdsWords words
    for (int i = threadIdx.x; i < kSelBins; i += WAVES * kWave) lds[kSelMisc + i] = 0u;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int per_wave = ((nt + WAVES * kWave - 1) / (WAVES * kWave)) * kWave;
    const int steps = per_wave / kWave;
    const int seg0 = wave * per_wave;
    const int rem = nt - seg0;
    const int limit = (rem < per_wave ? rem : per_wave) - lane;  // element j exists iff j*64 < limit

    uint32_t key[ITEMS];
    {
        const float* sp = s + seg0 + lane;
#pragma unroll
        for (int j = 0; j < ITEMS; ++j)
            key[j] = j * kWave < limit ? KEY::of(sp[j * kWave]) : 0u;
    }
    __syncthreads();  // the histogram is clear
    // keys >= cand over the whole row, cand >= 1 (so the zero keys of absent elements never
    // count). `turn` alternates the LDS slots so that one barrier per call is enough.
    auto count_ge = [&](uint32_t cand, int turn) -> uint32_t {
        // absent elements hold key 0 < cand, so only whole groups of 8 steps past the row's end
        // are skipped (one scalar branch per group instead of one per key)
        uint32_t c = 0;
#pragma unroll
        for (int j0 = 0; j0 < ITEMS; j0 += 8) {
            if (j0 < steps) {
#pragma unroll
                for (int j = j0; j < j0 + 8 && j < ITEMS; ++j)
                    c += (uint32_t)__popcll(__ballot(key[j] >= cand));
            }
        }
        if constexpr (WAVES > 1) {
            uint32_t* slot = lds + (turn & 1) * WAVES;
            if (lane == 0) slot[wave] = c;
            __syncthreads();
            c = 0;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) c += slot[w];
        }
        return c;
    };

    // ---- the top kSelBits of the k-th largest key, by one LDS histogram -----------------------
    // (sign, exponent and the first mantissa bit of a score): one atomic per key instead of a
    // bisection step per bit. s_hist was cleared and a barrier passed before this point.
    uint32_t* s_hist = lds + kSelMisc;
    uint32_t* s_cand = s_hist;  // the list reuses the histogram once the pivot bin is known
    uint32_t* s_pv = lds + 4 * WAVES;  // [0] pivot bin, [1] keys in higher bins, [2] keys in it, [3] list fill
#pragma unroll
    for (int j0 = 0; j0 < ITEMS; j0 += 8) {
        if (j0 >= steps) break;
#pragma unroll
        for (int j = j0; j < j0 + 8 && j < ITEMS; ++j)
            if (j * kWave < limit) atomicAdd(&s_hist[key[j] >> kSelLow], 1u);
    }
    __syncthreads();
    if (wave == 0) {
        // a lane owns 16 consecutive bins; suffix sums over the lanes find the lane where the
        // running count from the top reaches kq, which then walks its own bins
        uint32_t c[kSelBins / kWave], mine = 0;
#pragma unroll
        for (int i = 0; i < kSelBins / kWave; ++i) {
            c[i] = s_hist[lane * (kSelBins / kWave) + i];
            mine += c[i];
        }
        uint32_t suffix = mine;  // inclusive of this lane, over lanes >= lane
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const uint32_t v = __shfl_down(suffix, off, kWave);
            if (lane + off < kWave) suffix += v;
        }
        const uint32_t above_lane = suffix - mine;
        if (above_lane < kq && kq <= suffix) {
            uint32_t acc = above_lane;
            int i = kSelBins / kWave - 1;
            for (; i > 0; --i) {
                if (acc + c[i] >= kq) break;
                acc += c[i];
            }
            s_pv[0] = (uint32_t)(lane * (kSelBins / kWave) + i);
            s_pv[1] = acc;
            s_pv[2] = c[i];
            s_pv[3] = 0u;
        }
    }
    __syncthreads();
    const uint32_t pbin = s_pv[0], above_bin = s_pv[1], in_bin = s_pv[2];
    const uint32_t need_in_bin = kq - above_bin;  // 1 <= need_in_bin <= in_bin

    // T: select key > T, and the first `need` (in index order) of key == T
    uint32_t T = 0, need = 0;
    if (need_in_bin == in_bin) {
        T = (pbin << kSelLow) - 1u;  // the whole bin is selected (pbin == 0 would need every key: kq < nt)
    } else if (in_bin <= (uint32_t)kSelCand) {
        // ---- the other bits among the bin's members only: they are listed (any order) in LDS
        // and one wave bisects them from registers
        uint32_t fill = 0;  // where this wave's members start in the list
        if constexpr (WAVES > 1) {
            uint32_t mine = 0;
#pragma unroll
            for (int j0 = 0; j0 < ITEMS; j0 += 8) {
                if (j0 >= steps) break;
#pragma unroll
                for (int j = j0; j < j0 + 8 && j < ITEMS; ++j)
                    mine += (uint32_t)__popcll(__ballot(j * kWave < limit && (key[j] >> kSelLow) == pbin));
            }
            uint32_t* s_cnt = lds;  // the count_ge slots are idle here
            if (lane == 0) s_cnt[wave] = mine;
            __syncthreads();
            for (int w = 0; w < wave; ++w) fill += s_cnt[w];
        }
#pragma unroll
        for (int j0 = 0; j0 < ITEMS; j0 += 8) {
            if (j0 >= steps) break;
#pragma unroll
            for (int j = j0; j < j0 + 8 && j < ITEMS; ++j) {
                const bool is = j * kWave < limit && (key[j] >> kSelLow) == pbin;
                const unsigned long long m = __ballot(is);
                if (is) s_cand[fill + lanes_below(m)] = key[j];
                fill += (uint32_t)__popcll(m);
            }
        }
        __syncthreads();
        if (wave == 0) {
            constexpr int CP = kSelCand / kWave;
            uint32_t ck[CP];
            const int csteps = ((int)in_bin + kWave - 1) / kWave;
#pragma unroll
            for (int i = 0; i < CP; ++i) ck[i] = (i * kWave + lane) < (int)in_bin ? s_cand[i * kWave + lane] : 0u;
            auto cand_ge = [&](uint32_t cand) -> uint32_t {  // cand >= 1
                uint32_t c = 0;
#pragma unroll
                for (int i = 0; i < CP; ++i)
                    if (i < csteps) c += (uint32_t)__popcll(__ballot(ck[i] >= cand));
                return c;
            };
            uint32_t p = pbin << kSelLow, t = 0, nd = 0;
            bool exact = false;
            for (int b = kSelLow - 1; b >= 0; --b) {
                const uint32_t cand = p | (1u << b);
                const uint32_t c = cand_ge(cand);
                if (c >= need_in_bin) p = cand;
                if (c == need_in_bin) {
                    exact = true;
                    t = cand - 1u;
                    break;
                }
            }
            if (!exact) {
                // p is the need_in_bin-th largest member: members >= p outnumber it, members > p do not
                t = p;
                const uint32_t higher = (p & ((1u << kSelLow) - 1u)) == ((1u << kSelLow) - 1u) ? 0u : cand_ge(p + 1u);
                nd = need_in_bin - higher;
            }
            if (lane == 0) {
                s_pv[0] = t;
                s_pv[1] = nd;
            }
        }
        __syncthreads();
        T = s_pv[0];
        need = s_pv[1];
    } else {
        // ---- a bin too full to list (heavy ties): bisect its bits over all the keys
        uint32_t p = pbin << kSelLow;
        bool exact = false;
        for (int b = kSelLow - 1; b >= 0; --b) {
            const uint32_t cand = p | (1u << b);
            const uint32_t c = count_ge(cand, b);
            if (c >= kq) p = cand;
            if (c == kq) {
                exact = true;
                T = cand - 1u;
                break;
            }
        }
        if (!exact) {
            // p is the k-th largest key: count(key >= p) > kq > count(key > p)
            T = p;
            const uint32_t above = p == 0xffffffffu ? 0u : count_ge(p + 1u, 1);  // bit 0 used slot 0
            need = kq - above;
        }
    }

    uint32_t cnt_gt = 0, cnt_eq = 0;
    if constexpr (WAVES > 1) {
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const bool live = j * kWave < limit;
            cnt_gt += live && key[j] > T ? 1u : 0u;
            cnt_eq += live && key[j] == T ? 1u : 0u;
        }
    }
    uint32_t run_gt = 0, run_eq = 0;
    if constexpr (WAVES > 1) {
        const uint32_t gt_total = wave_sum(cnt_gt), eq_total = wave_sum(cnt_eq);
        uint32_t* s_gt = lds + 2 * WAVES;
        uint32_t* s_eq = s_gt + WAVES;
        if (lane == 0) {
            s_gt[wave] = gt_total;
            s_eq[wave] = eq_total;
        }
        __syncthreads();
        for (int w = 0; w < wave; ++w) {
            run_gt += s_gt[w];
            run_eq += s_eq[w];
        }
    }
#pragma unroll
    for (int j0 = 0; j0 < ITEMS; j0 += 8) {
        if (j0 >= steps) break;
#pragma unroll
        for (int j = j0; j < j0 + 8 && j < ITEMS; ++j) {
            const bool live = j * kWave < limit;
            const bool g = live && key[j] > T;
            const bool e = live && key[j] == T;
            const unsigned long long mg = __ballot(g), me = __ballot(e);
            const uint32_t G = run_gt + lanes_below(mg);
            // slot < kq holds by construction; the compare keeps a wrong threshold from ever
            // turning into a write outside the caller's buffer
            if (me == 0ull) {  // no key equal to the threshold in this step: the usual case
                const uint32_t slot = G + (run_eq < need ? run_eq : need);
                if (g && slot < kq) out[slot] = (uint32_t)(seg0 + j * kWave + lane) + add;
            } else {
                const uint32_t E = run_eq + lanes_below(me);
                const uint32_t slot = G + (E < need ? E : need);
                if ((g || (e && E < need)) && slot < kq)
                    out[slot] = (uint32_t)(seg0 + j * kWave + lane) + add;
                run_eq += (uint32_t)__popcll(me);
            }
            run_gt += (uint32_t)__popcll(mg);
        }
    }
}

// The limit of query row t, and the rows that need no ranking (everything legal is kept).
__device__ __forceinline__ int select_row_limit(int t, int n_comp, int ratio, int prefill) {
    return prefill ? min((int)(((long long)t + 1) / ratio), n_comp) : n_comp;
}
template <int THREADS>
__device__ __forceinline__ bool select_positional(int32_t* o, int limit, int k, int offset) {
    if (limit > k) return false;
    for (int i = threadIdx.x; i < k; i += THREADS) o[i] = i < limit ? offset + i : -1;
    return true;
}

template <int WAVES, int ITEMS>
__global__ __launch_bounds__(WAVES* kWave) void block_select_bisect_kernel(
    const float* __restrict__ scores, int n_comp, int ratio, int prefill, int k, int offset,
    int32_t* __restrict__ out, int out_stride) {
    __shared__ uint32_t lds[kSelLdsWords];
    const int t = blockIdx.x;
    const int limit = select_row_limit(t, n_comp, ratio, prefill);
    int32_t* o = out + (size_t)t * out_stride;
    if (select_positional<WAVES * kWave>(o, limit, k, offset)) return;
    select_bisect<WAVES, ITEMS, TotalOrderKey>(scores + (size_t)t * n_comp, limit, (uint32_t)k,
                                               reinterpret_cast<uint32_t*>(o), lds,
                                               (uint32_t)offset);
}

// Rows too long for the register form: the single-query radix select, one workgroup per row.
template <int THREADS, int ITEMS>
__global__ __launch_bounds__(THREADS) void block_select_kernel(const float* __restrict__ scores,
                                                               int n_comp, int ratio, int prefill,
                                                               int k, int offset,
                                                               int32_t* __restrict__ out,
                                                               int out_stride) {
    __shared__ uint32_t lds[topk_block_lds_words<THREADS>()];
    const int t = blockIdx.x;
    const int limit = select_row_limit(t, n_comp, ratio, prefill);
    int32_t* o = out + (size_t)t * out_stride;
    if (select_positional<THREADS>(o, limit, k, offset)) return;
    topk_block<THREADS, ITEMS, TotalOrderKey>(scores + (size_t)t * n_comp, limit, (uint32_t)k,
                                              reinterpret_cast<uint32_t*>(o), lds,
                                              (uint32_t)offset);
}

// `out_stride` (>= k) is the distance between the rows of `out`: k for a bare selection, the
// rectangle's width when the selection is the tail of a [window | compressed] row.
static int block_select_launch(const float* scores, int rows, int n_comp, int ratio,
                               int index_topk, int prefill, int offset, int* out, int out_stride,
                               hipStream_t stream) {
    if (!scores || !out) return 1001;
    if (rows <= 0 || n_comp <= 0 || ratio <= 0 || index_topk <= 0 || offset < 0) return 1001;
    if ((long long)offset + n_comp > 0x7fffffffLL) return 1002;
    const int k = index_topk < n_comp ? index_topk : n_comp;
    if (out_stride < k) return 1001;
    (void)hipGetLastError();
    const dim3 grid((unsigned)rows);
#define RK_BISECT(WV, I)                                                                     \
    hipLaunchKernelGGL((block_select_bisect_kernel<WV, I>), grid, dim3(WV* kWave), 0, stream, \
                       scores, n_comp, ratio, prefill ? 1 : 0, k, offset, out, out_stride)
#define RK_SELECT(T, I)                                                                       \
    hipLaunchKernelGGL((block_select_kernel<T, I>), grid, dim3(T), 0, stream, scores, n_comp, \
                       ratio, prefill ? 1 : 0, k, offset, out, out_stride)
    // up to 32 keys per lane; a row takes as few waves as hold it
    if (n_comp <= 64 * 8)
        RK_BISECT(1, 8);
    else if (n_comp <= 64 * 32)
        RK_BISECT(1, 32);
    else if (n_comp <= 128 * 32)
        RK_BISECT(2, 32);
    else if (n_comp <= 256 * 32)
        RK_BISECT(4, 32);
    else if (n_comp <= 512 * 32)
        RK_BISECT(8, 32);
    else if (n_comp <= 1024 * 32)
        RK_BISECT(16, 32);
    else if (n_comp <= 1024 * 64)
        RK_SELECT(1024, 64);
    else
        RK_SELECT(1024, 0);
#undef RK_BISECT
#undef RK_SELECT
    return launch_status();
}

// ---- selection rectangles: [window columns | compressed columns] per query row --------------
// crates/engine/src/v4/select.rs:334-400. The phase is start_pos == 0 (prefill: one row per
// prompt position, values are absolute positions) or not (decode: one row, values are ring
// slots). ratio == 4 is the class with an indexer (geometry.rs:86-92,128-130).
struct SelShape {
    int code, rows, win_cols, n_comp, offset;
};
static SelShape sel_shape(int win, int ratio, int seqlen, int start_pos) {
    SelShape s = {0, 0, 0, 0, 0};
    if (win <= 0 || seqlen <= 0 || start_pos < 0 || ratio < 0) return s.code = 1001, s;
    const bool prefill = start_pos == 0;
    if (!prefill && seqlen != 1) return s.code = 1005, s;
    s.rows = prefill ? seqlen : 1;
    s.win_cols = prefill ? (seqlen < win ? seqlen : win) : win;
    s.n_comp = ratio > 0 ? (int)(((long long)start_pos + s.rows) / ratio) : 0;
    s.offset = prefill ? seqlen : win;  // compress_offset, select.rs:268-270
    return s;
}

// One thread per cell of the first `win_cols + n_pos` columns of a `cols`-wide row: the window
// rule (select.rs:195-216), then the positional block rule (:224-241) for n_pos columns.
__global__ __launch_bounds__(256) void sel_fill_kernel(int win, int ratio, int start_pos,
                                                       int win_cols, int n_pos, int offset,
                                                       int cols, int32_t* __restrict__ out) {
    const int j = blockIdx.y * 256 + threadIdx.x, t = blockIdx.x;  // rows on x: no 65 535 limit
    if (j >= win_cols + n_pos) return;
    int v;
    if (j < win_cols) {
        if (start_pos == 0) {
            const int first = t > win - 1 ? t - (win - 1) : 0;
            v = first + j <= t ? first + j : -1;
        } else if (start_pos >= win - 1) {
            v = (start_pos % win + 1 + j) % win;  // oldest first, from just past the newest slot
        } else {
            v = j <= start_pos ? j : -1;
        }
    } else {
        const int c = j - win_cols;
        v = (start_pos != 0 || c < (t + 1) / ratio) ? c + offset : -1;
    }
    out[(size_t)t * cols + j] = v;
}

static int sel_fill_launch(const SelShape& s, int win, int ratio, int start_pos, int n_pos,
                           int cols, int* out, hipStream_t stream) {
    (void)hipGetLastError();
    const dim3 grid((unsigned)s.rows, (unsigned)((s.win_cols + n_pos + 255) / 256));
    if (grid.y > 65535) return 1002;
    hipLaunchKernelGGL(sel_fill_kernel, grid, dim3(256), 0, stream, win, ratio, start_pos, s.win_cols,
                       n_pos, s.offset, cols, out);
    return launch_status();
}

}  // namespace rk

extern "C" int rivoli_sel_shape(int win, int ratio, int index_topk, int seqlen, int start_pos,
                                int* rows, int* cols) {
    if (index_topk < 0) return 1001;
    const rk::SelShape s = rk::sel_shape(win, ratio, seqlen, start_pos);
    if (s.code) return s.code;
    if (ratio == 4 && s.n_comp > index_topk) return 1006;
    if (rows) *rows = s.rows;
    if (cols) *cols = s.win_cols + s.n_comp;
    return 0;
}

extern "C" int rivoli_sel_gather(int win, int ratio, int index_topk, int seqlen, int start_pos,
                                 int* out, void* stream) {
    int rows, cols;
    const int code = rivoli_sel_shape(win, ratio, index_topk, seqlen, start_pos, &rows, &cols);
    if (code) return code;
    if (!out) return 1001;
    const rk::SelShape s = rk::sel_shape(win, ratio, seqlen, start_pos);
    return rk::sel_fill_launch(s, win, ratio, start_pos, s.n_comp, cols, out, (hipStream_t)stream);
}

extern "C" int rivoli_sel_gather_scored(const float* scores, int n_comp, int win, int ratio,
                                        int index_topk, int seqlen, int start_pos, int* out,
                                        int* cols_out, void* stream) {
    if (ratio <= 0 || index_topk < 0 || n_comp < 0) return 1001;
    const rk::SelShape s = rk::sel_shape(win, ratio, seqlen, start_pos);
    if (s.code) return s.code;
    if (!out || (n_comp > 0 && !scores)) return 1001;
    const int k = index_topk < n_comp ? index_topk : n_comp;
    const int cols = s.win_cols + k;
    if (cols_out) *cols_out = cols;
    const int code = rk::sel_fill_launch(s, win, ratio, start_pos, 0, cols, out, (hipStream_t)stream);
    if (code || k == 0) return code;
    return rk::block_select_launch(scores, s.rows, n_comp, ratio, index_topk, start_pos == 0,
                                   s.offset, out + s.win_cols, cols, (hipStream_t)stream);
}

extern "C" int rivoli_index_select_blocks(const float* scores, int rows, int n_comp, int ratio,
                                          int index_topk, int prefill, int offset, int* out,
                                          void* stream) {
    const int k = index_topk < n_comp ? index_topk : n_comp;
    return rk::block_select_launch(scores, rows, n_comp, ratio, index_topk, prefill, offset, out,
                                   k, (hipStream_t)stream);
}

extern "C" size_t rivoli_index_topk_workspace_bytes(int n_queries, int nt) {
    if (n_queries <= 0 || nt <= 0) return 0;
    const int n_segs = (nt + rk::kSegKeys - 1) / rk::kSegKeys;
    return (size_t)n_queries * rk::topk_ws_words(n_segs) * sizeof(uint32_t);
}

extern "C" int rivoli_index_topk_batched(const float* scores, int n_queries, int stride,
                                         const int* nts, int nt, int k, unsigned int* rows,
                                         void* workspace, void* stream) {
    return rk::index_topk_launch(scores, n_queries, stride, nts, nt, k, rows, workspace,
                                 (hipStream_t)stream);
}

extern "C" int rivoli_index_topk(const float* scores, int nt, int k, unsigned int* rows) {
    return rk::index_topk_launch(scores, 1, nt, nullptr, nt, k, rows, nullptr, nullptr);
}
