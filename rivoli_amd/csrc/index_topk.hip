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
// (2) Split across the chip, used when the caller supplies a workspace: three launches, no
//     workgroup ever waits for another, nothing is elected. `topk_hist_kernel`: every
//     4096-score segment of every query adds the histogram of its keys' top 12 bits to the
//     query's global histogram (LDS first, then one atomic per non-empty bin) — a producer that
//     has the scores in registers anyway (the indexer's score kernel) can do this step itself.
//     `topk_cand_kernel`: every segment re-derives the pivot bin (the one holding the k-th key)
//     from that histogram, counts its keys in higher bins and lists its keys IN the pivot bin.
//     The finishing launch deals a query's selection to workgroups by OUTPUT position, 128
//     slots each, and — when asked to — gathers and dequantizes those rows from the fp8 pages
//     straight away: the selection never waits for a separate gather launch and the gather is
//     balanced whatever the distribution of the selected tokens. Two forms.
//     Queries of up to 64 segments (262144 scores), `topk_finish_bits_kernel`: the candidate
//     launch has also marked every key above the pivot bin in a bitmap of the query (a wave's
//     ballots are its words) and packed each listed key with its position, so the finishing
//     workgroup never reads a score: it finds the exact pivot among the listed keys (two
//     10-bit histogram passes in LDS, looked up by every wave for itself), adds the listed keys
//     that make it to its LDS copy of the bitmap, and a popcount prefix over the bitmap gives
//     every selected index its output position.
//     Longer queries, `topk_finish_kernel`: every workgroup pulls the query's listed keys into
//     LDS, finishes the radix select on the low 20 bits by itself, derives per segment how many
//     keys precede, and re-reads only the segments its slots fall in to emit them in index
//     order. A query whose pivot bin holds more keys than LDS can list (huge ties) finds its
//     pivot by streaming shape (1)'s radix passes over the whole query — slower, same answer.
//     Either way every workgroup repeats the small pivot search on otherwise idle compute
//     units instead of waiting for a hand-over, and the histogram is left zeroed for the next
//     call.
// Launch-only; see include/rivoli_kvcache.h for the contract of every entry point.
#include <mutex>
#include <type_traits>

#include "gather_common.hpp"
#include "topk_common.hpp"

namespace rk {

constexpr int kBins = 256;
constexpr int kCopies = 32;

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
    const uint32_t incl = wave_inclusive_sum(tot);
    const uint32_t above = wave_total(incl) - incl;  // keys in the bins of higher lanes
    if (above < need && need <= above + tot) {
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

// The radix passes of shape (1): the k-th largest key of the elements key_at(j) (element j of a
// lane exists iff j * 64 < limit) and how many keys EQUAL to it the selection takes, found by
// four 8-bit histogram passes, most significant byte first. Every thread of the workgroup calls
// it with the same kq; lds holds topk_block_lds_words<THREADS>() words.
template <int THREADS, int ITEMS, class KeyAt>
__device__ __forceinline__ void radix_pivot(KeyAt&& key_at, int steps, int limit, uint32_t kq,
                                            uint32_t* lds, uint32_t* pivot_out,
                                            uint32_t* need_out) {
    constexpr int WAVES = THREADS / kWave;
    constexpr int TPB = THREADS / kBins;  // threads that share one bin's copies
    static_assert(TPB == 1 || TPB == 4, "256 or 1024 threads");
    uint32_t* s_hist = lds;
    uint32_t* s_bins = s_hist + kBins * kCopies;
    uint32_t* s_pn = s_bins + kBins + 2 * WAVES;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;

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
    *pivot_out = pivot;
    *need_out = need;
}

// Shape (1): the whole selection for one query by one workgroup of THREADS threads.
// ITEMS: keys per lane kept in registers; 0 = re-read the scores on every sweep.
// KEY: the order (FoldedZeroKey or TotalOrderKey); `add` is added to every emitted index.
template <int THREADS, int ITEMS, class KEY = FoldedZeroKey>
__device__ __forceinline__ void topk_block(const float* __restrict__ s, int nt, uint32_t kq,
                                           uint32_t* __restrict__ out, uint32_t* lds,
                                           uint32_t add = 0u) {
    constexpr int WAVES = THREADS / kWave;
    uint32_t* s_gt = lds + kBins * kCopies + kBins;
    uint32_t* s_eq = s_gt + WAVES;

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

    uint32_t pivot, need;
    radix_pivot<THREADS, ITEMS>(key_at, steps, limit, kq, lds, &pivot, &need);

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

// Sum over the 16 wave slots of v[w] for w < wave (*before) and over all of them (*all):
// sixteen independent broadcast reads, which pipeline, instead of a chain of shuffles.
// Every lane of the wave must call it.
__device__ __forceinline__ void wave_slots_prefix(const uint32_t* v, int wave, uint32_t* before,
                                                  uint32_t* all) {
    uint32_t a = 0, b = 0;
#pragma unroll
    for (int w = 0; w < kTopkWaves; ++w) {
        const uint32_t x = v[w];
        a += x;
        b += w < wave ? x : 0u;
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
// Shape (2): a query split over many workgroups (three launches, see the file header).
// ---------------------------------------------------------------------------------------------
constexpr int kCandCap = 8192;    // pivot-bin keys a finishing workgroup can hold in LDS
constexpr int kSlotsPerGroup = 128;  // output positions per finishing workgroup
static_assert(kSegKeys == kSplitThreads * 4, "a wave owns 256 consecutive scores of a segment");
static_assert(kTopBins == kSplitThreads * 4, "a thread owns four consecutive histogram bins");
static_assert(kMaxSegs <= kSplitThreads, "one segment per thread in the finishing kernel");
static_assert(kSplitThreads == kTopkThreads, "the 16-slot wave helpers serve both shapes");

// A wave's 256 consecutive scores of segment `seg` as keys: element j of lane L is index
// seg * 4096 + wave * 256 + j * 64 + L (so a ballot over element j lists 64 consecutive indices
// in lane order) and exists iff j * 64 < *limit.
__device__ __forceinline__ void load_keys4(const float* __restrict__ s, int nt, int seg,
                                           uint32_t (&key)[4], int* limit) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int base = seg * kSegKeys + wave * (4 * kWave) + lane;
    *limit = nt - base;
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = j * kWave < *limit ? s[base + j * kWave] : 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) key[j] = topk_key(v[j]);
}

// The 16 wave slots v[0..16): the sum of those before `wave` (returned) and of all (*all), as
// scalars. One LDS read and a 16-lane DPP scan; every lane of the wave must call it.
__device__ __forceinline__ uint32_t wave_slots_before(const uint32_t* v, int wave, uint32_t* all) {
    const int lane = threadIdx.x & (kWave - 1);
    uint32_t x = v[lane & (kSplitWaves - 1)];
    x += dpp_or_zero<0x111, 0xf>(x);
    x += dpp_or_zero<0x112, 0xf>(x);
    x += dpp_or_zero<0x114, 0xf>(x);
    x += dpp_or_zero<0x118, 0xf>(x);
    *all = (uint32_t)__builtin_amdgcn_readlane((int)x, kSplitWaves - 1);
    return wave ? (uint32_t)__builtin_amdgcn_readlane((int)x, wave - 1) : 0u;
}

// Exclusive prefix sum of one value per thread over the 1024-thread workgroup, in thread
// order; *total receives the workgroup sum. tmp holds 16 words. Every thread must call it.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* tmp,
                                                         uint32_t* total) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t incl = wave_inclusive_sum(v);
    lds_barrier();  // tmp may still be read from a previous use
    if (lane == kWave - 1) tmp[wave] = incl;
    lds_barrier();
    return wave_slots_before(tmp, wave, total) + incl - v;
}

// Launch 1: the per-query histogram of the keys' top 12 bits.
__global__ __launch_bounds__(kSplitThreads) void topk_hist_kernel(
    const float* __restrict__ scores, int stride, const int* __restrict__ nts, int nt_all,
    uint32_t* __restrict__ ws, size_t ws_stride) {
    __shared__ uint32_t s_hist[kTopBins];
    const int q = blockIdx.y, seg = blockIdx.x, tid = threadIdx.x;
    const int nt = nts ? min(nts[q], nt_all) : nt_all;
    if (seg * kSegKeys >= nt) return;
    uint32_t key[4];
    int limit;
    load_keys4(scores + (size_t)q * stride, nt, seg, key, &limit);
#pragma unroll
    for (int i = 0; i < 4; ++i) s_hist[tid + i * kSplitThreads] = 0u;
    lds_barrier();
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (j * kWave < limit) atomicAdd(&s_hist[key[j] >> kLowBits], 1u);
    lds_barrier();
    flush_top_bins(s_hist, ws + (size_t)q * ws_stride, tid, kSplitThreads);
}

// Launch 2: the pivot bin from the histogram; this segment's keys above it counted, its keys
// in it listed (in any order: only their values matter to the pivot).
// BITS (queries of up to kBitsMaxSegs segments): the keys above the pivot bin are also marked,
// one bit per score, in the query's bitmap — a wave's ballots ARE those words — and a listed key
// is packed with where it sits: its low 20 bits (the top 12 are the pivot bin's) over its 12-bit
// position in the segment. The finishing launch then never goes back to the scores.
template <bool BITS>
__global__ __launch_bounds__(kSplitThreads) void topk_cand_kernel(
    const float* __restrict__ scores, int stride, const int* __restrict__ nts, int nt_all, int k,
    uint32_t* __restrict__ ws, size_t ws_stride, int n_segs) {
    __shared__ uint32_t s_wave[kSplitWaves];
    __shared__ uint32_t s_pn[2];
    __shared__ uint32_t s_cnt[2];  // [0] listed, [1] in higher bins
    const int q = blockIdx.y, seg = blockIdx.x, tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nt = nts ? min(nts[q], nt_all) : nt_all;
    if (nt <= 0) return;
    uint32_t* w = ws + (size_t)q * ws_stride;
    uint32_t* bits = w + topk_ws_bits_offset(n_segs) + (size_t)seg * (kSegKeys / 32);
    if (seg * kSegKeys >= nt) {  // a segment past this query's end holds nothing
        if (tid == 0) {
            w[kWsCounts + seg] = 0u;
            w[kWsCounts + n_segs + seg] = 0u;
        }
        if (BITS && tid < kSegKeys / 32) bits[tid] = 0u;
        return;
    }
    const uint32_t kq = (uint32_t)min(k, nt);
    if (tid < 2) s_cnt[tid] = s_pn[tid] = 0u;
    uint32_t key[4];
    int limit;
    load_keys4(scores + (size_t)q * stride, nt, seg, key, &limit);  // before the histogram is used

    // thread t owns bins 4t .. 4t+3; the bin b with (keys in bins > b) < kq <= (keys in bins >= b)
    const u32x4 c4 = reinterpret_cast<const u32x4*>(w)[tid];
    const uint32_t c[4] = {c4.x, c4.y, c4.z, c4.w};
    const uint32_t mine = c[0] + c[1] + c[2] + c[3];
    const uint32_t incl = wave_inclusive_sum(mine);
    if (lane == kWave - 1) s_wave[wave] = incl;
    lds_barrier();
    uint32_t all;
    const uint32_t lower = wave_slots_before(s_wave, wave, &all) + incl;  // up to this thread
    const uint32_t above = all - lower;                                    // in the higher bins
    if (above < kq && kq <= above + mine) {
        uint32_t acc = above;
        int m = 3;
        for (; m > 0; --m) {
            if (acc + c[m] >= kq) break;
            acc += c[m];
        }
        s_pn[0] = (uint32_t)(tid * 4 + m);
        s_pn[1] = kq - acc;
    }
    lds_barrier();
    const uint32_t p12 = s_pn[0];

    uint32_t* list = w + topk_ws_cand_offset(n_segs) + (size_t)seg * kSegKeys;
    uint32_t higher = 0;
    uint32_t word = 0;  // BITS: lane L < 8 keeps word L of the wave's eight bitmap words
    unsigned long long in_pivot[4];
    uint32_t listed = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t bin = key[j] >> kLowBits;
        const bool live = j * kWave < limit;
        const unsigned long long above_mask = __ballot(live && bin > p12);
        higher += (uint32_t)__popcll(above_mask);
        if (BITS) {
            if (lane == 2 * j) word = (uint32_t)above_mask;
            if (lane == 2 * j + 1) word = (uint32_t)(above_mask >> 32);
        }
        in_pivot[j] = __ballot(live && bin == p12);
        listed += (uint32_t)__popcll(in_pivot[j]);
    }
    if (listed) {  // one place in the list for the wave's keys: a single LDS round trip
        uint32_t base = 0;
        if (lane == 0) base = atomicAdd(&s_cnt[0], listed);
        base = __builtin_amdgcn_readfirstlane(base);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t entry =
                BITS ? ((key[j] << kTopBits) | (uint32_t)(wave * (4 * kWave) + j * kWave + lane))
                     : key[j];
            if ((in_pivot[j] >> lane) & 1ull) list[base + lanes_below(in_pivot[j])] = entry;
            base += (uint32_t)__popcll(in_pivot[j]);
        }
    }
    if (BITS && lane < 8) bits[wave * 8 + lane] = word;
    if (lane == 0 && higher) atomicAdd(&s_cnt[1], higher);
    lds_barrier();
    if (tid == 0) {
        w[kWsCounts + seg] = s_cnt[0];
        w[kWsCounts + n_segs + seg] = s_cnt[1];
        if (seg == 0) {
            w[kWsPivot] = p12;
            w[kWsNeed] = s_pn[1];
        }
    }
}

// Launch 3: exact pivot, per-segment prefixes, then this workgroup's output positions — and,
// with a pool, the rows themselves. W / PT: the page geometry at compile time (0 = runtime).
// Two things set this kernel's time before the gather starts. Memory round trips: everything
// the workgroup will need is requested at once, before the first use — the segment counts, the
// head of every segment's list (a wave per segment, 256 keys, requested before the counts say
// how many of them exist), the keys of the three segments its output positions most likely
// fall in, and the query's block-table row. And instruction issue: a vector instruction keeps
// a SIMD busy for four cycles and the sixteen waves share four SIMDs, so bookkeeping that all
// threads repeat costs sixteen times what it costs in one wave; scans over the segments run in
// wave 0 while the others wait at the barrier, and positions come from ballots and scalar
// popcounts rather than from per-thread prefix sums.
constexpr int kSpecSegs = kSplitWaves;  // queries of up to 16 segments fetch list heads early
constexpr int kSpecKeys = 4 * kWave;    // per segment
template <int W, int PT>
__global__ __launch_bounds__(kSplitThreads) void topk_finish_kernel(
    const float* __restrict__ scores, int stride, const int* __restrict__ nts, int nt_all, int k,
    uint32_t* __restrict__ rows, uint32_t* __restrict__ ws, size_t ws_stride, int n_segs,
    const uint8_t* __restrict__ pool, const int* __restrict__ block_table,
    uint16_t* __restrict__ out, int max_blocks_per_seq, int width_rt, int page_tokens_rt,
    int n_pages, size_t page_bytes, unsigned int* __restrict__ bad_rows) {
    // the listed keys; the streaming fallback's histograms alias them
    __shared__ uint32_t s_key[kCandCap > topk_block_lds_words<kSplitThreads>()
                                  ? kCandCap
                                  : topk_block_lds_words<kSplitThreads>()];
    __shared__ uint32_t s_G[kMaxSegs + 1];   // keys above the pivot in the segments before
    __shared__ uint32_t s_E[kMaxSegs + 1];   // keys equal to the pivot in the segments before
    __shared__ uint32_t s_off[kMaxSegs + 1]; // where a segment's listed keys start in s_key
    __shared__ uint32_t s_bins[3][kBins];    // one histogram per radix pass, cleared up front
    __shared__ uint32_t s_pn[3][2];
    __shared__ uint32_t s_wave[2][kSplitWaves];
    __shared__ int s_span[2];
    __shared__ int s_table[kSplitThreads];   // the query's block-table row, when it fits
    __shared__ uint32_t s_tok[kSlotsPerGroup];
    __shared__ unsigned long long s_base[kSlotsPerGroup];
    __shared__ unsigned long long s_scale_at[kSlotsPerGroup];

    const int q = blockIdx.y, tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nt = nts ? min(nts[q], nt_all) : nt_all;
    if (nt <= 0) return;
    const uint32_t kq = (uint32_t)min(k, nt);
    const float* s = scores + (size_t)q * stride;
    uint32_t* w = ws + (size_t)q * ws_stride;
    const uint32_t* lists = w + topk_ws_cand_offset(n_segs);

    // ---- requests ----
    const uint32_t p12 = w[kWsPivot];
    uint32_t need = w[kWsNeed];
    uint32_t n_listed = 0, n_higher = 0;
    if (tid < n_segs) {
        n_listed = w[kWsCounts + tid];
        n_higher = w[kWsCounts + n_segs + tid];
    }
    const bool spec = n_segs <= kSpecSegs;
    uint32_t head[4] = {0u, 0u, 0u, 0u};
    if (spec && wave < n_segs) {  // entries past the segment's count are junk and never used
#pragma unroll
        for (int i = 0; i < 4; ++i) head[i] = lists[(size_t)wave * kSegKeys + lane + i * kWave];
    }
    // output position p of a query with evenly spread winners sits in segment p * S / kq; the
    // spread is never even, so the neighbours on both sides are requested as well
    const int guess = min(n_segs - 1, (int)((long long)blockIdx.x * n_segs / (int)gridDim.x));
    const int g0 = max(guess - 1, 0);
    uint32_t pkey[3][4];
    int plimit[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) load_keys4(s, nt, g0 + i, pkey[i], &plimit[i]);
    const bool table_cached = pool && max_blocks_per_seq <= kSplitThreads;
    int my_page = -1;
    if (table_cached && tid < max_blocks_per_seq)
        my_page = block_table[(size_t)q * max_blocks_per_seq + tid];

    if (blockIdx.x == 0)  // the histogram has served: left zeroed for the next call
        reinterpret_cast<u32x4*>(w)[tid] = u32x4{0u, 0u, 0u, 0u};
    if (tid < 3 * kBins) (&s_bins[0][0])[tid] = 0u;
    if (tid == 0) {
        s_span[0] = n_segs;
        s_span[1] = -1;
    }
    if (tid < n_segs) s_G[tid] = n_higher;

    // ---- where each segment's listed keys go in LDS ----
    if (n_segs <= kWave) {
        if (wave == 0) {  // one wave, the others go straight to the barrier
            const uint32_t incl = wave_inclusive_sum(n_listed);
            if (lane < n_segs) s_off[lane] = incl - n_listed;
            if (lane == n_segs - 1) s_off[n_segs] = incl;
        }
    } else {
        uint32_t all;
        const uint32_t my_off = block_exclusive_scan(n_listed, s_wave[0], &all);
        if (tid < n_segs) s_off[tid] = my_off;
        if (tid == 0) s_off[n_segs] = all;
    }
    lds_barrier();
    const uint32_t total = s_off[n_segs];

    uint32_t pivot;
    if (total <= (uint32_t)kCandCap) {
        // ---- the listed keys into LDS, a wave per segment ----
        for (int sg = wave; sg < n_segs; sg += kSplitWaves) {
            const uint32_t base = s_off[sg], n = s_off[sg + 1] - base;
            const uint32_t* src = lists + (size_t)sg * kSegKeys;
            uint32_t i0 = 0;
            if (spec) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if ((uint32_t)(lane + i * kWave) < n) s_key[base + lane + i * kWave] = head[i];
                i0 = kSpecKeys;
            }
            for (uint32_t i = i0 + lane; i < n; i += kWave) s_key[base + i] = src[i];
        }
        lds_barrier();
        // ---- radix select on the low 20 bits among them: 8 + 8 + 4 ----
        pivot = p12 << kLowBits;
        uint32_t mask = ~0u << kLowBits;
#pragma unroll
        for (int pass = 0; pass < 3; ++pass) {
            const int shift = pass == 0 ? kLowBits - 8 : (pass == 1 ? kLowBits - 16 : 0);
            const uint32_t dmask = pass == 2 ? (1u << (kLowBits - 16)) - 1u : 0xffu;
            for (uint32_t c = tid; c < total; c += kSplitThreads) {
                const uint32_t u = s_key[c];
                if ((u & mask) == pivot) atomicAdd(&s_bins[pass][(u >> shift) & dmask], 1u);
            }
            lds_barrier();
            if (wave == 0) find_pivot_bin(s_bins[pass], need, s_pn[pass], lane);
            lds_barrier();
            pivot |= s_pn[pass][0] << shift;
            need = s_pn[pass][1];
            mask |= dmask << shift;
        }
        // ---- per segment: listed keys above / equal to the pivot, a wave per segment ----
        for (int sg = wave; sg < n_segs; sg += kSplitWaves) {
            const uint32_t base = s_off[sg], n = s_off[sg + 1] - base;
            uint32_t cg = 0, ce = 0;
            for (uint32_t i0 = 0; i0 < n; i0 += kWave) {
                const uint32_t i = i0 + lane;
                const uint32_t u = i < n ? s_key[base + i] : 0u;
                cg += (uint32_t)__popcll(__ballot(i < n && u > pivot));
                ce += (uint32_t)__popcll(__ballot(i < n && u == pivot));
            }
            if (lane == 0) {
                s_G[sg] += cg;  // on top of the segment's keys in higher bins
                s_E[sg] = ce;
            }
        }
    } else {
        // ---- too many keys in the pivot bin to list (huge ties): the radix passes streamed
        // over the whole query, then one more sweep for the per-segment counts ----
        const int per_wave = ((nt + kSplitThreads - 1) / kSplitThreads) * kWave;
        const int steps = per_wave / kWave;
        const long long seg0 = (long long)wave * per_wave;
        const long long rem = (long long)nt - seg0;
        const int limit = (int)(rem < per_wave ? rem : per_wave) - lane;
        auto key_at = [&](int j) -> uint32_t {
            return (j * kWave < limit) ? topk_key(s[seg0 + (long long)j * kWave + lane]) : 0u;
        };
        radix_pivot<kSplitThreads, 0>(key_at, steps, limit, kq, s_key, &pivot, &need);
        lds_barrier();
        if (tid < n_segs) s_G[tid] = s_E[tid] = 0u;
        lds_barrier();
        for (int sg = 0; sg * kSegKeys < nt; ++sg) {
            uint32_t key[4];
            int lim;
            load_keys4(s, nt, sg, key, &lim);
            uint32_t cg = 0, ce = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                cg += (uint32_t)__popcll(__ballot(j * kWave < lim && key[j] > pivot));
                ce += (uint32_t)__popcll(__ballot(j * kWave < lim && key[j] == pivot));
            }
            if (lane == 0) {
                if (cg) atomicAdd(&s_G[sg], cg);
                if (ce) atomicAdd(&s_E[sg], ce);
            }
        }
    }
    lds_barrier();

    // ---- exclusive prefixes over the segments; a key's output position is
    // (keys above the pivot before it) + min(keys equal to the pivot before it, need) ----
    if (n_segs <= kWave) {
        if (wave == 0) {
            const uint32_t g = lane < n_segs ? s_G[lane] : 0u, e = lane < n_segs ? s_E[lane] : 0u;
            const uint32_t gi = wave_inclusive_sum(g), ei = wave_inclusive_sum(e);
            if (lane < n_segs) {
                s_G[lane] = gi - g;
                s_E[lane] = ei - e;
            }
            if (lane == n_segs - 1) {
                s_G[n_segs] = gi;
                s_E[n_segs] = ei;
            }
        }
    } else {
        const uint32_t g_seg = tid < n_segs ? s_G[tid] : 0u, e_seg = tid < n_segs ? s_E[tid] : 0u;
        uint32_t all;
        const uint32_t gp = block_exclusive_scan(g_seg, s_wave[0], &all);
        const uint32_t ep = block_exclusive_scan(e_seg, s_wave[0], &all);
        if (tid < n_segs) {
            s_G[tid] = gp;
            s_E[tid] = ep;
        }
        if (tid == n_segs - 1) {
            s_G[n_segs] = gp + g_seg;
            s_E[n_segs] = ep + e_seg;
        }
    }
    lds_barrier();
    const uint32_t lo = (uint32_t)blockIdx.x * kSlotsPerGroup;
    if (lo >= kq) return;
    const uint32_t hi = min(lo + (uint32_t)kSlotsPerGroup, kq);
    if (tid < n_segs) {  // the segments whose output positions meet [lo, hi)
        const uint32_t a = s_G[tid] + min(s_E[tid], need);
        const uint32_t b = s_G[tid + 1] + min(s_E[tid + 1], need);
        if (a < hi && b > lo) {
            atomicMin(&s_span[0], tid);
            atomicMax(&s_span[1], tid);
        }
    }
    if (table_cached && tid < max_blocks_per_seq) s_table[tid] = my_page;
    lds_barrier();
    const int sg_first = s_span[0], sg_last = s_span[1];
    uint32_t* out_rows = rows + (size_t)q * k;
    // a wave's 256 keys are 256 consecutive indices, element j in lane order: counts and
    // positions are ballots and scalar popcounts (the segments may be visited in any order)
    int turn = 0;
    auto emit = [&](int sg, const uint32_t (&key)[4], int lim) {
        unsigned long long mg[4], me[4];
        uint32_t cg = 0, ce = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool live = j * kWave < lim;
            mg[j] = __ballot(live && key[j] > pivot);
            me[j] = __ballot(live && key[j] == pivot);
            cg += (uint32_t)__popcll(mg[j]);
            ce += (uint32_t)__popcll(me[j]);
        }
        if (lane == 0) s_wave[turn][wave] = cg | (ce << 16);  // at most 256 each
        lds_barrier();
        uint32_t all;
        const uint32_t before = wave_slots_before(s_wave[turn], wave, &all);
        turn ^= 1;
        uint32_t G = s_G[sg] + (before & 0xffffu), E = s_E[sg] + (before >> 16);
        // the wave's 256 keys take the output positions [first, last): nothing to place when
        // they miss this workgroup's (about half of a segment's waves; wave-uniform, and past
        // the barrier)
        const uint32_t first = G + min(E, need), last = G + cg + min(E + ce, need);
        if (last <= lo || first >= hi) return;
        const uint32_t idx0 = (uint32_t)(sg * kSegKeys + wave * (4 * kWave) + lane);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if ((mg[j] | me[j]) == 0ull) continue;  // wave-uniform: nothing of these 64 is taken
            const bool g = (mg[j] >> lane) & 1ull, eq = (me[j] >> lane) & 1ull;
            const uint32_t Gl = G + lanes_below(mg[j]), El = E + lanes_below(me[j]);
            const uint32_t slot = Gl + min(El, need);
            if ((g || (eq && El < need)) && slot >= lo && slot < hi) {
                out_rows[slot] = idx0 + j * kWave;
                s_tok[slot - lo] = idx0 + j * kWave;
            }
            G += (uint32_t)__popcll(mg[j]);
            E += (uint32_t)__popcll(me[j]);
        }
    };
#pragma unroll
    for (int i = 0; i < 3; ++i)  // the segments requested up front, straight from registers
        if (g0 + i >= sg_first && g0 + i <= sg_last) emit(g0 + i, pkey[i], plimit[i]);
    for (int sg = sg_first; sg <= sg_last; ++sg) {
        if (sg >= g0 && sg < g0 + 3) continue;
        uint32_t key[4];
        int lim;
        load_keys4(s, nt, sg, key, &lim);
        emit(sg, key, lim);
    }
    if (!pool) return;

    // ---- the selected rows of [lo, hi): fp8 page rows -> bf16, as the sparse gather does ----
    lds_barrier();
    const int width = W ? W : width_rt;
    const int pt = PT ? PT : page_tokens_rt;
    const int cnt = (int)(hi - lo);
    if (tid < cnt &&
        !resolve_row(s_tok[tid],
                     table_cached ? s_table : block_table + (size_t)q * max_blocks_per_seq,
                     max_blocks_per_seq, width, pt, n_pages, page_bytes, bad_rows, &s_base[tid],
                     &s_scale_at[tid]))
        s_span[0] = -1;  // the span has served; now the flag "a row is skipped"
    lds_barrier();
    constexpr int kUnroll = W ? (kSlotsPerGroup * (W / 8) + kSplitThreads - 1) / kSplitThreads : 4;
    const bool plain = s_span[0] >= 0 && cnt * (width >> 3) == kSplitThreads * kUnroll;
    stream_rows<kSplitThreads, kUnroll>(pool, s_base, s_scale_at, cnt, width, plain,
                                        out + ((size_t)q * k + lo) * width);
}

// Launch 3 for queries of up to kBitsMaxSegs segments: the selection as a bitmap.
// The candidate launch has marked every score above the pivot bin in the query's bitmap and
// listed the pivot bin's keys with their positions, so what is left is small and needs no score:
// (1) one round of requests — the bitmap (a few words per thread), the segments' list lengths,
//     the head of each list (a wave per segment, two entries per lane, asked for before the
//     lengths are known), the query's block-table row;
// (2) the exact pivot among the listed keys' low 20 bits: two 10-bit histogram passes, a bin per
//     thread (or two, or four), the entries staying in registers (list entries past a
//     segment's first 128 are read again from the workspace in each pass);
// (3) the listed keys above the pivot — and those equal to it, all of them or the `need`
//     lowest indices — set their bits in the LDS copy of the bitmap;
// (4) a popcount prefix over the bitmap gives every set bit its output position; the threads
//     whose words hold positions [lo, hi) write those indices out, resolve them through the
//     block table, and the workgroup streams the rows.
// Ties at the pivot value with more equal keys than the selection needs (rare) pick the lowest
// indices by the same machinery: the equal keys alone are marked in a cleared bitmap, the
// popcount prefix finds the index of the need-th of them, and only those up to it are kept.
template <int THREADS>
__device__ __forceinline__ uint32_t waves_before(const uint32_t* v, int wave, uint32_t* all) {
    constexpr int NW = THREADS / kWave;
    static_assert(NW <= 16, "one row of 16 lanes holds the wave slots");
    const int lane = threadIdx.x & (kWave - 1);
    uint32_t x = (lane & 15) < NW ? v[lane & 15] : 0u;
    x += dpp_or_zero<0x111, 0xf>(x);
    x += dpp_or_zero<0x112, 0xf>(x);
    x += dpp_or_zero<0x114, 0xf>(x);
    x += dpp_or_zero<0x118, 0xf>(x);
    *all = (uint32_t)__builtin_amdgcn_readlane((int)x, NW - 1);
    return wave ? (uint32_t)__builtin_amdgcn_readlane((int)x, wave - 1) : 0u;
}

// A 1024-bin histogram kept with a 64-bin summary of it (coarse bin = fine bin / 16): the
// highest fine bin b with (count in bins > b) < need <= (count in bins >= b), found by ONE wave
// from two LDS reads — a lane per coarse bin, then sixteen lanes over the fine bins inside the
// one that holds it — so every wave of a workgroup can look it up for itself and nobody waits
// for a result to be published. Returns b; *need_out = need - (count in bins > b),
// *count_out = count in b. Bins complete and visible on entry; all 64 lanes must call it.
__device__ __forceinline__ uint32_t find_bin_two_level(const uint32_t* coarse, const uint32_t* fine,
                                                       uint32_t need, uint32_t* need_out,
                                                       uint32_t* count_out) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t cc = coarse[lane];
    const uint32_t ci = wave_inclusive_sum(cc);
    const uint32_t above_c = wave_total(ci) - ci;  // in the coarse bins of higher lanes
    const unsigned long long hit_c = __ballot(above_c < need && need <= above_c + cc);
    const int cb = hit_c ? __builtin_ctzll(hit_c) : 0;
    const uint32_t need_f = need - (uint32_t)__builtin_amdgcn_readlane((int)above_c, cb);
    const uint32_t fc = fine[cb * 16 + (lane & 15)];
    uint32_t fi = fc;  // inclusive over each row of 16 lanes (all four rows hold the same)
    fi += dpp_or_zero<0x111, 0xf>(fi);
    fi += dpp_or_zero<0x112, 0xf>(fi);
    fi += dpp_or_zero<0x114, 0xf>(fi);
    fi += dpp_or_zero<0x118, 0xf>(fi);
    const uint32_t above_f = (uint32_t)__builtin_amdgcn_readlane((int)fi, 15) - fi;
    const unsigned long long hit_f =
        __ballot(above_f < need_f && need_f <= above_f + fc) & 0xffffull;
    const int fb = hit_f ? __builtin_ctzll(hit_f) : 0;
    *need_out = need_f - (uint32_t)__builtin_amdgcn_readlane((int)above_f, fb);
    *count_out = (uint32_t)__builtin_amdgcn_readlane((int)fc, fb);
    return (uint32_t)(cb * 16 + fb);
}

template <int W, int PT, int THREADS, int SLOTS, int WPT>
__global__ __launch_bounds__(THREADS) void topk_finish_bits_kernel(
    const int* __restrict__ nts, int nt_all, int k, uint32_t* __restrict__ rows,
    uint32_t* __restrict__ ws, size_t ws_stride, int n_segs, const uint8_t* __restrict__ pool,
    const int* __restrict__ block_table, uint16_t* __restrict__ out, int max_blocks_per_seq,
    int width_rt, int page_tokens_rt, int n_pages, size_t page_bytes,
    unsigned int* __restrict__ bad_rows) {
    constexpr int NW = THREADS / kWave;
    constexpr int ROUNDS = (kBitsMaxSegs + NW - 1) / NW;  // segments a wave may own
    constexpr int TPT = 1024 / THREADS;                   // block-table entries a thread caches
    constexpr int kMini = kWave;  // keys of the pivot's 10-bit bin one wave ranks by itself
    __shared__ uint32_t s_bm[THREADS * WPT];
    __shared__ uint32_t s_fine[2][1024];  // [0]: bits 19..10 of the listed keys, [1]: bits 9..0
    __shared__ uint32_t s_coarse[2][64];  // their 64-bin summaries
    __shared__ uint32_t s_mini[kMini + 1];  // [kMini]: how many
    __shared__ uint32_t s_inc[THREADS];
    __shared__ uint32_t s_wv[16];
    __shared__ uint32_t s_tie[2];
    __shared__ int s_skipped;
    __shared__ int s_table[1024];
    __shared__ unsigned long long s_base[SLOTS];
    __shared__ unsigned long long s_scale_at[SLOTS];

    const int q = blockIdx.y, tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nt = nts ? min(nts[q], nt_all) : nt_all;
    if (nt <= 0) return;
    const uint32_t kq = (uint32_t)min(k, nt);
    const uint32_t lo = (uint32_t)blockIdx.x * SLOTS;
    if (lo >= kq) return;  // (workgroup 0, which also puts the histogram back to zero, never is)
    const uint32_t hi = min(lo + (uint32_t)SLOTS, kq);
    uint32_t* w = ws + (size_t)q * ws_stride;
    const uint32_t* lists = w + topk_ws_cand_offset(n_segs);
    const int n_words = n_segs * (kSegKeys / 32);

    // ---- (1) requests ----
    uint32_t need = w[kWsNeed];
    uint32_t n_listed[ROUNDS];
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        const int sg = wave + r * NW;
        n_listed[r] = sg < n_segs ? w[kWsCounts + sg] : 0u;  // one address per wave
    }
    uint32_t head[2] = {0u, 0u};
    if (wave < n_segs) {  // entries past the list's length are junk and never used
        head[0] = lists[(size_t)wave * kSegKeys + lane];
        head[1] = lists[(size_t)wave * kSegKeys + lane + kWave];
    }
    uint32_t bw[WPT];
    {
        const uint32_t* bits = w + topk_ws_bits_offset(n_segs);
#pragma unroll
        for (int j = 0; j < WPT; ++j) bw[j] = tid * WPT + j < n_words ? bits[tid * WPT + j] : 0u;
    }
    const bool table_cached = pool && max_blocks_per_seq <= 1024;
    int my_page[TPT];
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
        my_page[i] = -1;
        if (table_cached && tid + i * THREADS < max_blocks_per_seq)
            my_page[i] = block_table[(size_t)q * max_blocks_per_seq + tid + i * THREADS];
    }
    if (blockIdx.x == 0)  // the histogram has served: left zeroed for the next call
        for (int i = tid; i < kTopBins / 4; i += THREADS)
            reinterpret_cast<u32x4*>(w)[i] = u32x4{0u, 0u, 0u, 0u};
    for (int i = tid; i < 2 * 1024; i += THREADS) (&s_fine[0][0])[i] = 0u;
    if (tid < 2 * 64) (&s_coarse[0][0])[tid] = 0u;
    if (tid == 0) {
        s_skipped = 0;
        s_mini[kMini] = 0u;
    }
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) n_listed[r] = __builtin_amdgcn_readfirstlane(n_listed[r]);
#pragma unroll
    for (int j = 0; j < WPT; ++j) s_bm[tid * WPT + j] = bw[j];
#pragma unroll
    for (int i = 0; i < TPT; ++i)
        if (table_cached && tid + i * THREADS < max_blocks_per_seq)
            s_table[tid + i * THREADS] = my_page[i];
    lds_barrier();

    // every listed entry of the segments this wave owns: f(entry, segment)
    auto for_each_listed = [&](auto&& f) {
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) {
            const int sg = wave + r * NW;
            const uint32_t n = n_listed[r];
            const uint32_t* src = lists + (size_t)sg * kSegKeys;
            if (r == 0) {
                if ((uint32_t)lane < n) f(head[0], sg);
                if ((uint32_t)(lane + kWave) < n) f(head[1], sg);
            }
            for (uint32_t i = (r == 0 ? 2 * kWave : 0) + lane; i < n; i += kWave) f(src[i], sg);
        }
    };

    // ---- (2) the exact pivot: bits 19..10 of the listed keys, then bits 9..0 ----
    for_each_listed([&](uint32_t e, int) {
        atomicAdd(&s_fine[0][e >> 22], 1u);
        atomicAdd(&s_coarse[0][e >> 26], 1u);
    });
    lds_barrier();
    uint32_t n_hi;
    const uint32_t p_hi = find_bin_two_level(s_coarse[0], s_fine[0], need, &need, &n_hi);
    // the keys of that bin: few enough (about one, on scores without heavy ties) for a wave to
    // rank among themselves — every wave does, so nothing is published — else a second histogram
    const bool mini = n_hi <= (uint32_t)kMini;
    for_each_listed([&](uint32_t e, int) {
        if ((e >> 22) != p_hi) return;
        if (mini) {
            s_mini[atomicAdd(&s_mini[kMini], 1u)] = e >> 12;
        } else {
            atomicAdd(&s_fine[1][(e >> 12) & 1023u], 1u);
            atomicAdd(&s_coarse[1][(e >> 16) & 63u], 1u);
        }
    });
    lds_barrier();
    uint32_t pivot, n_equal;  // low 20 bits of the k-th largest key; how many keys equal it
    if (mini) {
        const uint32_t mine = (uint32_t)lane < n_hi ? s_mini[lane] : 0u;
        uint32_t gt = 0, eq = 0;
        for (uint32_t j = 0; j < n_hi; ++j) {
            const uint32_t other = (uint32_t)__builtin_amdgcn_readlane((int)mine, (int)j);
            gt += other > mine ? 1u : 0u;
            eq += other == mine ? 1u : 0u;
        }
        const unsigned long long hit =
            __ballot((uint32_t)lane < n_hi && gt < need && need <= gt + eq);
        const int at = hit ? __builtin_ctzll(hit) : 0;
        pivot = (uint32_t)__builtin_amdgcn_readlane((int)mine, at);
        need -= (uint32_t)__builtin_amdgcn_readlane((int)gt, at);
        n_equal = (uint32_t)__builtin_amdgcn_readlane((int)eq, at);
    } else {
        pivot = (p_hi << 10) | find_bin_two_level(s_coarse[1], s_fine[1], need, &need, &n_equal);
    }
    // need: keys equal to the pivot that are selected

    // ---- (3) the listed keys' bits ----
    uint32_t last_equal = 0xffffffffu;  // equal keys at indices up to this one are selected
    if (n_equal > need) {               // uniform: ties by index, lowest first
#pragma unroll
        for (int j = 0; j < WPT; ++j) s_bm[tid * WPT + j] = 0u;
        lds_barrier();
        for_each_listed([&](uint32_t e, int sg) {
            if ((e >> 12) == pivot) {
                const uint32_t idx = (uint32_t)sg * kSegKeys + (e & 4095u);
                atomicOr(&s_bm[idx >> 5], 1u << (idx & 31u));
            }
        });
        lds_barrier();
        uint32_t ew[WPT], cnt = 0;
#pragma unroll
        for (int j = 0; j < WPT; ++j) cnt += (uint32_t)__popc(ew[j] = s_bm[tid * WPT + j]);
        const uint32_t incl = wave_inclusive_sum(cnt);
        if (lane == kWave - 1) s_wv[wave] = incl;
        lds_barrier();
        uint32_t all;
        uint32_t before = waves_before<THREADS>(s_wv, wave, &all) + incl - cnt;
        if (before < need && need <= before + cnt) {  // the need-th equal key is in these words
#pragma unroll
            for (int j = 0; j < WPT; ++j) {
                uint32_t x = ew[j];
                while (x) {
                    const int b = __builtin_ctz(x);
                    x &= x - 1u;
                    if (++before == need) s_tie[0] = (uint32_t)(tid * WPT + j) * 32u + (uint32_t)b;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < WPT; ++j) s_bm[tid * WPT + j] = bw[j];
        lds_barrier();
        last_equal = s_tie[0];
    }
    for_each_listed([&](uint32_t e, int sg) {
        const uint32_t low = e >> 12, idx = (uint32_t)sg * kSegKeys + (e & 4095u);
        if (low > pivot || (low == pivot && idx <= last_equal))
            atomicOr(&s_bm[idx >> 5], 1u << (idx & 31u));
    });
    lds_barrier();

    // ---- (4) output positions from a popcount prefix; this workgroup's are [lo, hi) ----
    // Position p belongs to the thread whose prefix is the last one <= p; one thread per
    // position looks its own bit up (the wave from the sixteen wave totals, the thread by a
    // search over that wave's running counts, then a select inside the word), so a word with
    // every bit set costs what an almost empty one costs.
    uint32_t cnt = 0;
#pragma unroll
    for (int j = 0; j < WPT; ++j) cnt += (uint32_t)__popc(s_bm[tid * WPT + j]);
    const uint32_t incl = wave_inclusive_sum(cnt);
    s_inc[tid] = incl;
    if (lane == kWave - 1) s_wv[wave] = incl;  // (the tie path's readers are a barrier back)
    lds_barrier();
    const int width = W ? W : width_rt;
    const int pt = PT ? PT : page_tokens_rt;
    if (tid < (int)(hi - lo)) {
        // (no cross-lane operation in here: the lanes of a partly filled last wave are off)
        const uint32_t p = lo + (uint32_t)tid;
        int wv = 0;
        uint32_t before = 0, upto = 0;  // selected before wave wv, which holds position p
#pragma unroll
        for (int i = 0; i < NW - 1; ++i) {
            upto += s_wv[i];
            const bool past = upto <= p;
            wv += past ? 1 : 0;
            before = past ? upto : before;
        }
        const uint32_t* inc = s_inc + wv * kWave;
        int at = 0;  // threads of that wave wholly before p
#pragma unroll
        for (int step = kWave / 2; step > 0; step >>= 1)
            if (before + inc[at + step - 1] <= p) at += step;
        if (at) before += inc[at - 1];
        const int t = wv * kWave + at;
        uint32_t r = p - before, x = 0;
        int j = 0;
#pragma unroll
        for (int i = 0; i < WPT; ++i) {  // the word that holds it
            const uint32_t y = s_bm[t * WPT + i];
            const uint32_t c = (uint32_t)__popc(y);
            const bool here = i == j && r < c;
            x = here ? y : x;
            const bool past = i == j && !here;
            r -= past ? c : 0u;
            j += past ? 1 : 0;
        }
        uint32_t bit = 0;  // its r-th set bit
#pragma unroll
        for (int half = 16; half > 0; half >>= 1) {
            const uint32_t c = (uint32_t)__popc(x & ((1u << half) - 1u));
            if (r >= c) {
                r -= c;
                bit += (uint32_t)half;
                x >>= half;
            }
        }
        const uint32_t tok = (uint32_t)(t * WPT + j) * 32u + bit;
        rows[(size_t)q * k + p] = tok;
        if (pool &&
            !resolve_row(tok, table_cached ? s_table : block_table + (size_t)q * max_blocks_per_seq,
                         max_blocks_per_seq, width, pt, n_pages, page_bytes, bad_rows, &s_base[tid],
                         &s_scale_at[tid]))
            s_skipped = 1;
    }
    if (!pool) return;
    lds_barrier();
    const int n_mine = (int)(hi - lo);
    constexpr int kUnroll = W ? (SLOTS * (W / 8) + THREADS - 1) / THREADS : 4;
    const bool plain = !s_skipped && n_mine * (width >> 3) == THREADS * kUnroll;
    stream_rows<THREADS, kUnroll>(pool, s_base, s_scale_at, n_mine, width, plain,
                                  out + ((size_t)q * k + lo) * width);
}

struct GatherArgs {  // the page pool a selection gathers from; pool == nullptr: indices only
    const uint8_t* pool;
    const int* block_table;
    uint16_t* out;
    int max_blocks_per_seq, width, page_tokens, n_pages;
    unsigned int* bad_rows;
};

// The bitmap finishing kernel in the shape the query length asks for: WPT bitmap words per
// thread hold 16 segments (WPT x THREADS = 2048 words) or kBitsMaxSegs of them.
template <int THREADS, int SLOTS, class... Args>
static void finish_bits_launch_shape(bool fixed, int n_segs, int kmax, int n_queries,
                                     hipStream_t stream, Args... args) {
    const dim3 grid((unsigned)((kmax + SLOTS - 1) / SLOTS), (unsigned)n_queries), block(THREADS);
    constexpr int kShort = 16 * (kSegKeys / 32) / THREADS, kLong = kBitsMaxSegs * (kSegKeys / 32) / THREADS;
    if (n_segs <= 16) {
        if (fixed)
            hipLaunchKernelGGL((topk_finish_bits_kernel<576, 64, THREADS, SLOTS, kShort>), grid, block,
                               0, stream, args...);
        else
            hipLaunchKernelGGL((topk_finish_bits_kernel<0, 0, THREADS, SLOTS, kShort>), grid, block, 0,
                               stream, args...);
    } else {
        if (fixed)
            hipLaunchKernelGGL((topk_finish_bits_kernel<576, 64, THREADS, SLOTS, kLong>), grid, block,
                               0, stream, args...);
        else
            hipLaunchKernelGGL((topk_finish_bits_kernel<0, 0, THREADS, SLOTS, kLong>), grid, block, 0,
                               stream, args...);
    }
}
template <class... Args>
static void finish_bits_launch(bool fixed, int n_segs, int kmax, int n_queries, hipStream_t stream,
                               Args... args) {
    // 128 output positions per 1024-thread workgroup: 256 workgroups for 16 queries x 2048, one
    // per compute unit (64 per 512 threads and 32 per 256 measure 3 % and 20 % slower there)
    finish_bits_launch_shape<1024, 128>(fixed, n_segs, kmax, n_queries, stream, args...);
}

static int index_topk_launch(const float* scores, int n_queries, int stride, const int* nts,
                             int nt, int k, unsigned int* rows, void* workspace, bool hist_ready,
                             const GatherArgs& ga, hipStream_t stream) {
    if (!scores || !rows) return 1001;
    if (n_queries <= 0 || nt <= 0 || k <= 0) return 1001;
    if (stride < nt) return 1002;
    (void)hipGetLastError();
    // A short query is fastest on one workgroup; longer ones are split over the chip when the
    // caller brought a workspace.
    if (workspace && topk_runs_split(n_queries, nt)) {
        const int n_segs = topk_segments(nt);
        const size_t ws_stride = topk_ws_words(n_segs);
        uint32_t* ws = (uint32_t*)workspace;
        const dim3 seg_grid((unsigned)n_segs, (unsigned)n_queries), block(kSplitThreads);
        if (!hist_ready)
            hipLaunchKernelGGL(topk_hist_kernel, seg_grid, block, 0, stream, scores, stride, nts, nt,
                               ws, ws_stride);
        const int kmax = k < nt ? k : nt;
        const size_t page_bytes = (size_t)ga.page_tokens * ga.width + (size_t)ga.page_tokens * 4;
        const bool fixed = ga.pool && ga.width == 576 && ga.page_tokens == 64;
        if (n_segs <= kBitsMaxSegs) {
            hipLaunchKernelGGL(topk_cand_kernel<true>, seg_grid, block, 0, stream, scores, stride,
                               nts, nt, k, ws, ws_stride, n_segs);
            finish_bits_launch(fixed, n_segs, kmax, n_queries, stream, nts, nt, k, rows, ws,
                               ws_stride, n_segs, ga.pool, ga.block_table, ga.out,
                               ga.max_blocks_per_seq, ga.width, ga.page_tokens, ga.n_pages,
                               page_bytes, ga.bad_rows);
            return launch_status();
        }
        hipLaunchKernelGGL(topk_cand_kernel<false>, seg_grid, block, 0, stream, scores, stride, nts,
                           nt, k, ws, ws_stride, n_segs);
        const dim3 out_grid((unsigned)((kmax + kSlotsPerGroup - 1) / kSlotsPerGroup),
                            (unsigned)n_queries);
        if (fixed)
            hipLaunchKernelGGL((topk_finish_kernel<576, 64>), out_grid, block, 0, stream, scores,
                               stride, nts, nt, k, rows, ws, ws_stride, n_segs, ga.pool,
                               ga.block_table, ga.out, ga.max_blocks_per_seq, ga.width,
                               ga.page_tokens, ga.n_pages, page_bytes, ga.bad_rows);
        else
            hipLaunchKernelGGL((topk_finish_kernel<0, 0>), out_grid, block, 0, stream, scores, stride,
                               nts, nt, k, rows, ws, ws_stride, n_segs, ga.pool, ga.block_table,
                               ga.out, ga.max_blocks_per_seq, ga.width, ga.page_tokens, ga.n_pages,
                               page_bytes, ga.bad_rows);
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

    // Every load of the row is in flight before the first is used: an element past the row's
    // end reads the row's last score instead (and becomes key 0), because a load under a
    // per-lane condition is a branch with a wait of its own — 32 memory round trips in a row.
    // The wave-uniform choice among 8, 16, 24 or 32 loads keeps short rows from paying for
    // long ones; each arm is straight-line code.
    uint32_t key[ITEMS];
    {
        float v[ITEMS];
        const uint32_t first = (uint32_t)(seg0 + lane), last = (uint32_t)(nt - 1);
        auto fetch = [&](auto n_tag) {
            constexpr int N = decltype(n_tag)::value;
#pragma unroll
            for (int j = 0; j < ITEMS; ++j)
                v[j] = j < N ? s[min(first + (uint32_t)(j * kWave), last)] : 0.0f;
        };
        if (ITEMS <= 8 || steps > 24)
            fetch(std::integral_constant<int, ITEMS>{});
        else if (steps > 16)
            fetch(std::integral_constant<int, 24>{});
        else if (steps > 8)
            fetch(std::integral_constant<int, 16>{});
        else
            fetch(std::integral_constant<int, 8>{});
        // ---- the top kSelBits of the k-th largest key, by one LDS histogram -------------------
        // (sign, exponent and the first mantissa bit of a score): one atomic per key instead
        // of a bisection step per bit. The atomic sits with the key's conversion so that the
        // per-element "exists" masks do not stay live (32 of them overflow the scalar file).
        __syncthreads();  // the histogram is clear (the loads above are in flight meanwhile)
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            key[j] = 0u;
            if (j * kWave < limit) {
                key[j] = KEY::of(v[j]);
                atomicAdd(&lds[kSelMisc + (key[j] >> kSelLow)], 1u);
            }
        }
    }
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

    uint32_t* s_hist = lds + kSelMisc;
    uint32_t* s_cand = s_hist;  // the list reuses the histogram once the pivot bin is known
    uint32_t* s_pv = lds + 4 * WAVES;  // [0] pivot bin, [1] keys in higher bins, [2] keys in it, [3] list fill
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
    // Absent elements hold key 0, which no test below can tell from a live key 0 — and none has
    // to: they sit past every live element in index order, and kq < nt leaves at least one live
    // key unselected, so ties at the threshold are used up before an absent element's turn. Only
    // the list must not meet them (the histogram did not count them), hence pbin != 0 there.
    if (need_in_bin == in_bin) {
        T = (pbin << kSelLow) - 1u;  // the whole bin is selected (pbin == 0 would need every key: kq < nt)
    } else if (pbin != 0u && in_bin <= (uint32_t)kSelCand) {
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
                    mine += (uint32_t)__popcll(__ballot((key[j] >> kSelLow) == pbin));
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
                const bool is = (key[j] >> kSelLow) == pbin;
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

    // ---- emission in index order. A wave's share of the selection comes from ballots (scalar
    // popcounts), and its compares are kept apart from the emission's by passing T through an
    // empty asm: shared, their 64 masks would have to stay live across the exchange.
    T = __builtin_amdgcn_readfirstlane(T);  // the same in every lane: say so to the compiler
    need = __builtin_amdgcn_readfirstlane(need);
    const bool ties = need != 0u;  // distinct keys end the bisection on an exact count: need == 0
    uint32_t run_gt = 0, run_eq = 0;
    if constexpr (WAVES > 1) {
        uint32_t Tc = T;
        asm volatile("" : "+s"(Tc));
        uint32_t gt_total = 0, eq_total = 0;
#pragma unroll
        for (int j0 = 0; j0 < ITEMS; j0 += 8) {
            if (j0 >= steps) break;
#pragma unroll
            for (int j = j0; j < j0 + 8 && j < ITEMS; ++j) {
                gt_total += (uint32_t)__popcll(__ballot(key[j] > Tc));
                if (ties) eq_total += (uint32_t)__popcll(__ballot(key[j] == Tc));
            }
        }
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
    // slot < kq holds by construction; the compare keeps a wrong threshold from ever turning
    // into a write outside the caller's buffer
    if (!ties) {
#pragma unroll
        for (int j0 = 0; j0 < ITEMS; j0 += 8) {
            if (j0 >= steps) break;
#pragma unroll
            for (int j = j0; j < j0 + 8 && j < ITEMS; ++j) {
                const bool g = key[j] > T;
                const unsigned long long mg = __ballot(g);
                const uint32_t slot = run_gt + lanes_below(mg);
                if (g && slot < kq) out[slot] = (uint32_t)(seg0 + j * kWave + lane) + add;
                run_gt += (uint32_t)__popcll(mg);
            }
        }
        return;
    }
#pragma unroll
    for (int j0 = 0; j0 < ITEMS; j0 += 8) {
        if (j0 >= steps) break;
#pragma unroll
        for (int j = j0; j < j0 + 8 && j < ITEMS; ++j) {
            const bool g = key[j] > T;
            const bool e = key[j] == T;
            const unsigned long long mg = __ballot(g), me = __ballot(e);
            const uint32_t G = run_gt + lanes_below(mg);
            const uint32_t E = run_eq + lanes_below(me);
            const uint32_t slot = G + (E < need ? E : need);
            if ((g || (e && E < need)) && slot < kq)
                out[slot] = (uint32_t)(seg0 + j * kWave + lane) + add;
            run_eq += (uint32_t)__popcll(me);
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

// ---------------------------------------------------------------------------------------------
// The selection workspace for callers that cannot allocate: one array per GPU, inside the
// library's own image, held until the process ends. Sized for 16 queries of 65536 scores.
// ---------------------------------------------------------------------------------------------
constexpr size_t kStaticWsWords = 1179648;  // 4.5 MiB
constexpr int kStaticWsMaxDevices = 64;
static __device__ __align__(256) uint32_t scratch[kStaticWsWords];
static std::mutex g_scratch_mutex;
static uint32_t* g_scratch_ptr[kStaticWsMaxDevices];  // per device: where ITS copy of the array is

// The current device's copy of `scratch` (looked up once per device); 0, a guard code, or
// -(int)hipError_t.
static int static_workspace(uint32_t** out) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return -(int)e;
    if (device < 0 || device >= kStaticWsMaxDevices) return 1002;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return -(int)e;
        if (!p) return -(int)hipErrorInvalidSymbol;
        g_scratch_ptr[device] = (uint32_t*)p;
    }
    *out = g_scratch_ptr[device];
    return 0;
}

// The histogram of every query back to zero (a fill kernel, so that the call can sit in a
// captured graph): the array keeps what the last call left, and a call of another shape left
// its lists where this one's histograms are.
__global__ __launch_bounds__(kSplitThreads) void topk_ws_clear_kernel(uint32_t* __restrict__ ws,
                                                                      size_t ws_stride) {
    reinterpret_cast<u32x4*>(ws + (size_t)blockIdx.x * ws_stride)[threadIdx.x] = u32x4{0u, 0u, 0u, 0u};
}

// What both forms of the select-and-gather call refuse before anything is launched.
static int dsa_guard(const float* scores, int n_queries, int stride, int nt, int k,
                     const unsigned int* rows, const unsigned char* pool, const int* block_table,
                     const unsigned short* out, int max_blocks_per_seq, int width, int page_tokens,
                     int n_pages) {
    if (!scores || !rows || !pool || !block_table || !out) return 1001;
    if (n_queries <= 0 || nt <= 0 || k <= 0) return 1001;
    if (max_blocks_per_seq <= 0 || width <= 0 || page_tokens <= 0 || n_pages <= 0) return 1001;
    if (stride < nt || n_queries > 65535) return 1002;
    if (!gather_shape_ok(width, page_tokens) || !aligned16(pool) || !aligned16(out)) return 1004;
    return 0;
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
    return (size_t)n_queries * rk::topk_ws_words(rk::topk_segments(nt)) * sizeof(uint32_t);
}

extern "C" int rivoli_index_topk_batched(const float* scores, int n_queries, int stride,
                                         const int* nts, int nt, int k, unsigned int* rows,
                                         void* workspace, void* stream) {
    if (workspace && !rk::aligned16(workspace)) return 1004;
    const rk::GatherArgs none = {nullptr, nullptr, nullptr, 0, 0, 0, 0, nullptr};
    return rk::index_topk_launch(scores, n_queries, stride, nts, nt, k, rows, workspace, false, none,
                                 (hipStream_t)stream);
}

extern "C" int rivoli_index_topk(const float* scores, int nt, int k, unsigned int* rows) {
    const rk::GatherArgs none = {nullptr, nullptr, nullptr, 0, 0, 0, 0, nullptr};
    return rk::index_topk_launch(scores, 1, nt, nullptr, nt, k, rows, nullptr, false, none, nullptr);
}

extern "C" int rivoli_dsa_select_gather_paged(const float* scores, int n_queries, int stride,
                                              const int* nts, int nt, int k, unsigned int* rows,
                                              void* workspace, int hist_ready,
                                              const unsigned char* pool, const int* block_table,
                                              unsigned short* out, int max_blocks_per_seq,
                                              int width, int page_tokens, int n_pages,
                                              unsigned int* bad_rows, void* stream) {
    using namespace rk;
    const int refused = dsa_guard(scores, n_queries, stride, nt, k, rows, pool, block_table, out,
                                  max_blocks_per_seq, width, page_tokens, n_pages);
    if (refused) return refused;
    if (workspace && !aligned16(workspace)) return 1004;
    const GatherArgs ga = {pool, block_table, out, max_blocks_per_seq, width, page_tokens, n_pages,
                           bad_rows};
    const bool split = workspace && nt > 0 && n_queries > 0 && topk_runs_split(n_queries, nt);
    if (hist_ready && !split) return 1001;  // nothing could have filled a histogram for this shape
    if (split)
        return index_topk_launch(scores, n_queries, stride, nts, nt, k, rows, workspace,
                                 hist_ready != 0, ga, (hipStream_t)stream);
    // short queries: one workgroup per query selects, the sparse gather follows on the stream
    const GatherArgs none = {nullptr, nullptr, nullptr, 0, 0, 0, 0, nullptr};
    const int code = index_topk_launch(scores, n_queries, stride, nts, nt, k, rows, nullptr, false,
                                       none, (hipStream_t)stream);
    if (code) return code;
    return gather_rows_launch(pool, block_table, rows, nts, out, n_queries, k,
                                        k < nt ? k : nt, max_blocks_per_seq, width, page_tokens,
                                        n_pages, bad_rows, stream);
}

extern "C" int rivoli_dsa_select_gather_paged_noalloc(const float* scores, int n_queries,
                                                      int stride, const int* nts, int nt, int k,
                                                      unsigned int* rows, const unsigned char* pool,
                                                      const int* block_table, unsigned short* out,
                                                      int max_blocks_per_seq, int width,
                                                      int page_tokens, int n_pages,
                                                      unsigned int* bad_rows, void* stream) {
    using namespace rk;
    const int refused = dsa_guard(scores, n_queries, stride, nt, k, rows, pool, block_table, out,
                                  max_blocks_per_seq, width, page_tokens, n_pages);
    if (refused) return refused;
    uint32_t* ws = nullptr;
    if (topk_runs_split(n_queries, nt)) {
        const size_t ws_stride = topk_ws_words(topk_segments(nt));
        if ((size_t)n_queries * ws_stride > kStaticWsWords) return 1002;
        const int code = static_workspace(&ws);
        if (code) return code;
        (void)hipGetLastError();
        hipLaunchKernelGGL(topk_ws_clear_kernel, dim3((unsigned)n_queries), dim3(kSplitThreads), 0,
                           (hipStream_t)stream, ws, ws_stride);
        const int launched = launch_status();
        if (launched) return launched;
    }
    return rivoli_dsa_select_gather_paged(scores, n_queries, stride, nts, nt, k, rows, ws, 0, pool,
                                          block_table, out, max_blocks_per_seq, width, page_tokens,
                                          n_pages, bad_rows, stream);
}
