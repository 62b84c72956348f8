// The second cache format's block indexer: the Hadamard + simulated-fp4 spread of its q rows
// and of its compressor's pooled rows, and the block scorer that ranks compressed blocks for a
// query (crates/backend/kernels/blockindex.hip:99-136 and :209-235, launchers :241-281; CPU
// statements crates/oracles/src/v4oracle/numerics.rs:245-353 and
// crates/engine/tests/kernel_v4_indexer.rs:437-462). Both are bit-exact by construction: every
// value is produced by the reference's tree of f32 operations; what differs is who computes
// which value and where the operands wait.
//
// Spread. The reference gives a row to a 128-thread workgroup and walks LDS log2(d) times with
// a barrier per stage, then hands each fp4 block of 32 to one thread. Here a lane holds four
// consecutive values of a row (one 16-byte load and store, a wave moves 1 KiB per instruction),
// d / 4 neighbouring lanes hold a row, and a wave holds 64 / (d / 4) rows. The butterflies of
// stages 1 and 2 pair values of one lane; stage h >= 4 pairs lane L with lane L ^ (h / 4): the
// lane whose bit is clear holds the pair's first value and computes a + b, the other computes
// a - b from the same two numbers. A block of 32 is eight lanes; its amax is a maximum (exact
// in any order) over three lane exchanges. No LDS, no barrier; 8 bytes of traffic per value.
//
// Scorer. score[t][c] = bf16(sum_h bf16(relu(bf16(q[t][h] . kv[c])) * w[t][h])), the dot a
// sequential f32 fold of separately rounded products and the head sum a sequential f32 fold
// (blockindex.hip:138-207 argues each). That order rules out the matrix cores and any split of
// a dot over lanes; what is free is where the operands come from. A lane owns block c and
// keeps its 128-value row in registers for the whole launch; a wave's 64 lanes share the query,
// so q[t][h][i] and w[t][h] are wave-uniform and come through scalar loads straight into the
// multiply's scalar operand. Per (t, h) a wave issues 128 multiplies and 128 adds for 64
// scores and reads 512 bytes through the scalar cache: bound by vector issue, two
// instructions per multiply-add because the reference's rounding is two roundings.
// Widths other than 128 re-read the block's row through the vector cache instead.
#include "codec.hpp"

#include <cmath>

#include "rivoli_kvcache.h"

#pragma clang fp contract(off)

namespace rk {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr float kFp4Max = 6.0f;
constexpr float kFp4MaxInv = 1.0f / kFp4Max;
constexpr float kFp4AmaxFloor = kFp4Max * 1.17549435082228750797e-38f;  // 6 * 2^-126 (actquant.hpp:51)
constexpr int kSpreadMaxD = 256;   // blockindex.hip:40-42
constexpr int kSpreadThreads = 256;
constexpr int kSpreadInFlight = 4;  // row groups per wave, all requested before the first is used

__device__ __forceinline__ float round_bf16(float x) {
    return __uint_as_float((uint32_t)f32_to_bf16(x) << 16);
}

// formats.hpp:285-293 followed by its decode, for |q| <= 6: the nearest of {0, .5, 1, 1.5, 2, 3,
// 4, 6}, a tie to the even mantissa. The grid is spaced .5 below 2, 1 below 4 and 2 above, and
// on each stretch "tie to the even mantissa" is "tie to the even multiple of the spacing"
// (.25 -> 0, .75 -> 1, 1.25 -> 1, 1.75 -> 2, 2.5 -> 2, 3.5 -> 4, 5 -> 4: the reference's own
// table), which is what adding and subtracting 2^22, 2^23 or 2^24 does in round-to-nearest-even
// f32 arithmetic: two compares and two additions where counting midpoints takes fourteen
// instructions. A NaN passes no midpoint there and becomes a zero with its sign; here too.
__device__ __forceinline__ float e2m1_round_trip(float q) {
    const float a = fabsf(q);
    const float magic = a < 2.0f ? 4194304.0f : (a < 4.0f ? 8388608.0f : 16777216.0f);
    float v = (a + magic) - magic;
    v = a != a ? 0.0f : v;
    return __builtin_signbit(q) ? -v : v;
}

// LPR: lanes per row (d / 4). scale = 1 / sqrt(d), taken on the host (a correctly rounded
// square root and a true divide, blockindex.hip:107-113).
template <int LPR>
__global__ __launch_bounds__(kSpreadThreads) void f4_rotated_kernel(float* __restrict__ x,
                                                                     long long rows, float scale) {
    constexpr int kRowsPerWave = kWave / LPR;
    constexpr int d = LPR * 4;
    const int lane = threadIdx.x & (kWave - 1);
    const long long wave = (long long)blockIdx.x * (kSpreadThreads / kWave) + (threadIdx.x >> 6);
    const long long row0 = wave * (kRowsPerWave * kSpreadInFlight) + lane / LPR;
    const int col = (lane % LPR) * 4;

    f32x4 v[kSpreadInFlight];
#pragma unroll
    for (int u = 0; u < kSpreadInFlight; ++u) {
        const long long r = row0 + (long long)u * kRowsPerWave;
        // unconditional: a row past the end re-reads the last row and is not stored
        v[u] = *reinterpret_cast<const f32x4*>(x + (r < rows ? r : rows - 1) * d + col);
    }
#pragma unroll
    for (int u = 0; u < kSpreadInFlight; ++u) {
        float e[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
        // stages h = 1, 2: inside the lane
        {
            const float a0 = e[0] + e[1], a1 = e[0] - e[1], a2 = e[2] + e[3], a3 = e[2] - e[3];
            e[0] = a0 + a2, e[2] = a0 - a2, e[1] = a1 + a3, e[3] = a1 - a3;
        }
        // stages h = 4 .. d / 2: lane L with lane L ^ (h / 4)
#pragma unroll
        for (int m = 1; m < LPR; m <<= 1) {
            const bool upper = (lane & m) != 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float other = __shfl_xor(e[i], m, kWave);
                e[i] = upper ? other - e[i] : e[i] + other;
            }
        }
        // the bf16 store between rotation and quantization (blockindex.hip:91-96)
        float amax = kFp4AmaxFloor;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            e[i] = round_bf16(e[i] * scale);
            amax = fmaxf(amax, fabsf(e[i]));
        }
        // a block of 32 is 8 lanes; d = 32 is the whole row
#pragma unroll
        for (int m = 1; m < 8; m <<= 1) amax = fmaxf(amax, __shfl_xor(amax, m, kWave));
        // actquant.hpp:65-75: the smallest power of two >= amax / 6, by exponent surgery
        const uint32_t b = __float_as_uint(amax * kFp4MaxInv);
        const int ex = (int)((b >> 23) & 0xffu) - 127 + ((b & 0x7fffffu) ? 1 : 0);
        const float s = __uint_as_float((uint32_t)(ex + 127) << 23);
        // x / s for a power of two s is x * (1 / s) exactly whenever 1 / s is a normal number
        // (one multiply instead of the divide's dozen instructions); the divide stays for the
        // scales at the ends of the exponent range
        const bool by_reciprocal = ex >= -126 && ex <= 126;
        const float rinv = __uint_as_float((uint32_t)(127 - ex) << 23);
        f32x4 out;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float q = by_reciprocal ? e[i] * rinv : e[i] / s;
            q = q < -kFp4Max ? -kFp4Max : (q > kFp4Max ? kFp4Max : q);  // a NaN stays a NaN
            out[i] = round_bf16(e2m1_round_trip(q) * s);
        }
        const long long r = row0 + (long long)u * kRowsPerWave;
        if (r < rows) *reinterpret_cast<f32x4*>(x + r * d + col) = out;
    }
}

// ---- the block scorer -------------------------------------------------------------------------
constexpr int kScoreThreads = 256;           // four waves, 64 blocks each
constexpr int kScoreQueriesPerGroup = 16;    // queries a workgroup walks with its rows held

// The scalar operands of one 32-term chunk of a dot. Scalar loads return out of order, so the
// only wait there is waits for all of them: a chunk is requested one whole chunk of
// arithmetic (64 vector instructions) before it is used and nothing else is outstanding then.
struct QChunk {
    float v[32];
};
__device__ __forceinline__ void load_chunk(QChunk& c, const float* __restrict__ p) {
#pragma unroll
    for (int i = 0; i < 32; ++i) c.v[i] = p[i];
}
// Waits for the chunk here: placed before the next chunk is requested, the wait covers this
// chunk alone (requested a chunk ago); left to the first use it would also cover the request
// just made.
__device__ __forceinline__ void arrived(const QChunk& c) {
    asm volatile("" ::"s"(c.v[0]), "s"(c.v[16]));
}
template <int OFF>
__device__ __forceinline__ float fold_chunk(float dot, const QChunk& c, const float (&row)[128]) {
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const float prod = c.v[i] * row[OFF + i];
        dot = dot + prod;
    }
    return dot;
}

// bf16 first, then the relu (blockindex.hip:224-228; the sign of a zero cannot reach the
// output), the weight, the term's own bf16 store, the f32 head sum.
__device__ __forceinline__ float head_term(float dot, float weight) {
    dot = round_bf16(dot);
    dot = dot > 0.0f ? dot : 0.0f;
    const float term = dot * weight;
    return round_bf16(term);
}

// Which (query group, block group) a workgroup owns. The full rectangle runs block groups
// fastest (ratio == 0): the workgroups that share a query group start together, one per die,
// and their q rows are fetched from memory once for all of them (7.0 ms against 7.4 at 8 192 x
// 2 048). The prefill form runs query groups fastest: workgroups are dealt to the 8 dies in
// turn, and with block groups fastest (often 8 of them) each die would own one block group,
// whose work shrinks with its index — the first die would do an eighth of the rectangle alone
// while the last one idles (6.8 ms against 3.4).
__device__ __forceinline__ int query_group(int ratio) { return ratio > 0 ? blockIdx.x : blockIdx.y; }
__device__ __forceinline__ int block_group(int ratio) { return ratio > 0 ? blockIdx.y : blockIdx.x; }

// The first of the workgroup's queries [t0, t1) this wave scores. ratio > 0 is a prefill whose
// selection ranks block c for query t only when c < (t + 1) / ratio (a block is legal once it
// has closed): a wave's 64 blocks start at cw, and no query before ratio * (cw + 1) - 1 can
// rank any of them.
__device__ __forceinline__ int first_query(int t0, int t1, int ratio, long long cw) {
    if (ratio <= 0) return t0;
    const long long first = (cw + 1) * ratio - 1;
    return first > t0 ? (int)(first < t1 ? first : t1) : t0;
}

// The lane's block row, 128 values, into registers.
__device__ __forceinline__ void load_row(float (&row)[128], const float* __restrict__ kvr) {
#pragma unroll
    for (int i = 0; i < 128; i += 4) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(kvr + i);
        row[i] = v.x, row[i + 1] = v.y, row[i + 2] = v.z, row[i + 3] = v.w;
    }
}

// One head term, bf16(relu(bf16(q . row)) * weight), for each (query, head) pair g in [g0, g1):
// the pairs' 128-value q rows are contiguous and are walked as one run through two chunk
// buffers. on_term(g, term) receives them in order.
template <class OnTerm>
__device__ __forceinline__ void walk_pairs(const float* __restrict__ q, const float* __restrict__ w,
                                           const float (&row)[128], size_t g0, size_t g1,
                                           OnTerm&& on_term) {
    constexpr int HD = 128;
    if (g0 >= g1) return;  // (wave-uniform) no pair: the first chunk below would be pair g1's
    const float* qp = q + g0 * HD;
    QChunk a, b;
    load_chunk(a, qp);
    for (size_t g = g0; g < g1; ++g) {
        float dot = 0.0f;
        arrived(a);
        const float weight = w[g];
        load_chunk(b, qp + 32);
        __builtin_amdgcn_sched_barrier(0);
        dot = fold_chunk<0>(dot, a, row);
        __builtin_amdgcn_sched_barrier(0);
        arrived(b);
        load_chunk(a, qp + 64);
        __builtin_amdgcn_sched_barrier(0);
        dot = fold_chunk<32>(dot, b, row);
        __builtin_amdgcn_sched_barrier(0);
        arrived(a);
        load_chunk(b, qp + 96);
        __builtin_amdgcn_sched_barrier(0);
        dot = fold_chunk<64>(dot, a, row);
        __builtin_amdgcn_sched_barrier(0);
        arrived(b);
        load_chunk(a, g + 1 < g1 ? qp + HD : qp);  // the next pair's first chunk; the last re-reads its own
        __builtin_amdgcn_sched_barrier(0);
        dot = fold_chunk<96>(dot, b, row);
        __builtin_amdgcn_sched_barrier(0);
        on_term(g, head_term(dot, weight));
        qp += HD;
    }
}

// hd = 128, many (query, block group) pairs: a lane owns a block for the workgroup's queries
// and folds the head terms itself, in head order.
__global__ __launch_bounds__(kScoreThreads) void index_score_blocks_128_kernel(
    const float* __restrict__ q, const float* __restrict__ kv, const float* __restrict__ w,
    float* __restrict__ score, int s, int n_comp, int heads, int t_per_group, int ratio) {
    const long long c = (long long)block_group(ratio) * kScoreThreads + threadIdx.x;
    const int t1 = min(s, query_group(ratio) * t_per_group + t_per_group);
    const long long cw = (long long)block_group(ratio) * kScoreThreads +
                         (__builtin_amdgcn_readfirstlane((int)threadIdx.x) & ~(kWave - 1));
    const int t0 = first_query(query_group(ratio) * t_per_group, t1, ratio, cw);
    if (t0 >= t1) return;  // wave-uniform; the kernel has no barrier
    float row[128];
    load_row(row, kv + (size_t)(c < n_comp ? c : n_comp - 1) * 128);
    float acc = 0.0f;
    int hh = 0, t = t0;
    walk_pairs(q, w, row, (size_t)t0 * heads, (size_t)t1 * heads, [&](size_t, float term) {
        acc = acc + term;
        if (++hh == heads) {
            if (c < n_comp) score[(size_t)t * n_comp + c] = round_bf16(acc);
            acc = 0.0f, hh = 0, ++t;
        }
    });
}

// hd = 128, few (query, block group) pairs (a decode step: one query): the plain kernel would
// occupy n_comp / 256 compute units for 64 heads' worth of arithmetic each. Here a workgroup
// owns 64 blocks and its eight waves each take an eighth of the heads: the dots of different
// heads are independent, only their sum has an order. The head terms meet in LDS and the first
// wave folds them in head order, as the reference does.
constexpr int kSplitWavesPerGroup = 8;
constexpr int kSplitMaxHeads = 128;  // 32 KiB of terms
__global__ __launch_bounds__(kSplitWavesPerGroup* kWave) void index_score_blocks_128_split_kernel(
    const float* __restrict__ q, const float* __restrict__ kv, const float* __restrict__ w,
    float* __restrict__ score, int s, int n_comp, int heads, int ratio) {
    extern __shared__ float terms[];  // [heads][64]
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const long long cw = (long long)blockIdx.x * kWave;
    const long long c = cw + lane;
    const int t0 = first_query(0, s, ratio, cw);  // the same for every wave: the barriers below are safe
    const int per = (heads + kSplitWavesPerGroup - 1) / kSplitWavesPerGroup;
    const int h0 = min(wave * per, heads), h1 = min(h0 + per, heads);
    float row[128];
    load_row(row, kv + (size_t)(c < n_comp ? c : n_comp - 1) * 128);
    for (int t = t0; t < s; ++t) {
        const size_t base = (size_t)t * heads;
        walk_pairs(q, w, row, base + h0, base + h1,
                   [&](size_t g, float term) { terms[(g - base) * kWave + lane] = term; });
        __syncthreads();
        if (wave == 0) {
            float acc = 0.0f;
            for (int hh = 0; hh < heads; ++hh) acc = acc + terms[hh * kWave + lane];
            if (c < n_comp) score[(size_t)t * n_comp + c] = round_bf16(acc);
        }
        __syncthreads();
    }
}

// Any other width: the block's row is re-read through the vector cache for every head.
__global__ __launch_bounds__(kScoreThreads) void index_score_blocks_any_kernel(
    const float* __restrict__ q, const float* __restrict__ kv, const float* __restrict__ w,
    float* __restrict__ score, int s, int n_comp, int heads, int hd, int t_per_group, int ratio) {
    const long long c = (long long)block_group(ratio) * kScoreThreads + threadIdx.x;
    const float* const kvr = kv + (size_t)(c < n_comp ? c : n_comp - 1) * hd;
    const int t1 = min(s, query_group(ratio) * t_per_group + t_per_group);
    const long long cw = (long long)block_group(ratio) * kScoreThreads +
                         (__builtin_amdgcn_readfirstlane((int)threadIdx.x) & ~(kWave - 1));
    const int t0 = first_query(query_group(ratio) * t_per_group, t1, ratio, cw);
    for (int t = t0; t < t1; ++t) {
        float acc = 0.0f;
        for (int hh = 0; hh < heads; ++hh) {
            const float* const qh = q + ((size_t)t * heads + hh) * hd;  // wave-uniform
            float dot = 0.0f;
            for (int i = 0; i < hd; ++i) {
                const float prod = qh[i] * kvr[i];
                dot = dot + prod;
            }
            acc = acc + head_term(dot, w[(size_t)t * heads + hh]);
        }
        if (c < n_comp) score[(size_t)t * n_comp + c] = round_bf16(acc);
    }
}

}  // namespace rk

extern "C" int rivoli_act_quant_f4_rotated(float* x, int rows, int d, void* stream) {
    if (rows <= 0 || d <= 0) return 1001;
    if (d > rk::kSpreadMaxD) return 1002;
    if (d & (d - 1)) return 1003;
    if (d % 32) return 1004;
    if (!x) return 1001;
    if (!rk::aligned16(x)) return 1004;  // rows are moved 16 bytes at a time
    (void)hipGetLastError();
    const float scale = 1.0f / std::sqrt((float)d);
    const int lpr = d / 4;
    const long long rows_per_group = (long long)(rk::kWave / lpr) * rk::kSpreadInFlight *
                                     (rk::kSpreadThreads / rk::kWave);
    const dim3 grid((unsigned)((rows + rows_per_group - 1) / rows_per_group)), block(rk::kSpreadThreads);
    hipStream_t st = (hipStream_t)stream;
    switch (lpr) {
        case 8: hipLaunchKernelGGL(rk::f4_rotated_kernel<8>, grid, block, 0, st, x, (long long)rows, scale); break;
        case 16: hipLaunchKernelGGL(rk::f4_rotated_kernel<16>, grid, block, 0, st, x, (long long)rows, scale); break;
        case 32: hipLaunchKernelGGL(rk::f4_rotated_kernel<32>, grid, block, 0, st, x, (long long)rows, scale); break;
        default: hipLaunchKernelGGL(rk::f4_rotated_kernel<64>, grid, block, 0, st, x, (long long)rows, scale); break;
    }
    return rk::launch_status();
}

namespace rk {
static int score_blocks_launch(const float* q, const float* kv, const float* w, float* score, int s,
                               int n_comp, int heads, int hd, int ratio, hipStream_t st) {
    if (s <= 0 || heads <= 0 || hd <= 0) return 1001;
    // refused, not an empty success: the reference produces no score tensor at all before the
    // first block completes (blockindex.hip:268-273)
    if (n_comp <= 0) return 1005;
    if (!q || !kv || !w || !score) return 1001;
    (void)hipGetLastError();
    // enough workgroups to fill the part while a workgroup keeps its rows for several queries
    const unsigned c_groups = (unsigned)(((long long)n_comp + kScoreThreads - 1) / kScoreThreads);
    int t_per_group = kScoreQueriesPerGroup;
    while (t_per_group > 1 && (long long)c_groups * ((s + t_per_group - 1) / t_per_group) < 2048) t_per_group >>= 1;
    if (ratio <= 0)
        while ((s + t_per_group - 1) / t_per_group > 65535) t_per_group <<= 1;  // the grid's second extent
    const unsigned t_groups = (unsigned)((s + t_per_group - 1) / t_per_group);
    if (ratio > 0 && c_groups > 65535u) return 1002;  // more than 2^24 blocks
    const dim3 grid = ratio > 0 ? dim3(t_groups, c_groups) : dim3(c_groups, t_groups);
    const dim3 block(kScoreThreads);
    if (hd == 128 && aligned16(kv) && (long long)s * c_groups < 256 && heads <= kSplitMaxHeads) {
        const unsigned groups = (unsigned)(((long long)n_comp + kWave - 1) / kWave);
        hipLaunchKernelGGL(index_score_blocks_128_split_kernel, dim3(groups), dim3(kSplitWavesPerGroup * kWave),
                           (size_t)heads * kWave * sizeof(float), st, q, kv, w, score, s, n_comp, heads, ratio);
        return launch_status();
    }
    if (hd == 128 && aligned16(kv))
        hipLaunchKernelGGL(index_score_blocks_128_kernel, grid, block, 0, st, q, kv, w, score, s, n_comp,
                           heads, t_per_group, ratio);
    else
        hipLaunchKernelGGL(index_score_blocks_any_kernel, grid, block, 0, st, q, kv, w, score, s, n_comp,
                           heads, hd, t_per_group, ratio);
    return launch_status();
}
}  // namespace rk

extern "C" int rivoli_index_score_blocks(const float* q, const float* kv, const float* w,
                                         float* score, int s, int n_comp, int heads, int hd,
                                         void* stream) {
    return rk::score_blocks_launch(q, kv, w, score, s, n_comp, heads, hd, 0, (hipStream_t)stream);
}

extern "C" int rivoli_index_score_blocks_prefill(const float* q, const float* kv, const float* w,
                                                 float* score, int s, int n_comp, int heads, int hd,
                                                 int ratio, void* stream) {
    if (ratio <= 0) return 1001;
    return rk::score_blocks_launch(q, kv, w, score, s, n_comp, heads, hd, ratio, (hipStream_t)stream);
}
