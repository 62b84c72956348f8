// Attention over an explicit index list into ONE f32 buffer whose rows are key and value at
// once, for every head of a query (multi-query attention with K = V): the consumer of the
// second cache format's [ring | compressed] rows.
//
//     o[t][h] = bf16( sum_j p_j * kv[idx[t][j]] ),
//     p_j = exp(l_j - mx) / (sum_j exp(l_j - mx) + exp(sink[h] - mx)),  l_j = scale * q[t][h] . kv[idx[t][j]]
//
// over the slots with idx >= 0 (-1 masks a slot; it is never dereferenced). The sink is part
// of the denominator only. A query with no live slot gets NaN. This is the reference's
// gather_attn_shared_kv (crates/backend/kernels/attn.hip:325-443, launcher :446-465), which
// runs one workgroup per (query, head): every head re-reads the query's rows (64 times at 64
// heads) and each thread walks a whole row for its logit.
//
// Here a query's rows are read ONCE for all heads. For d = 512 a 512-thread workgroup (8 waves)
// owns a query and a block of 64 heads; waves w and w+4 share heads 16(w&3)..+15 and split the
// 512 contraction dims of the scores and the 512 output columns between them. Slots move in
// tiles of 32: wave w fetches the 4 rows of its tile positions (2 KiB each, fully coalesced),
// rounds them to bf16 (exact for cache rows, which are fp8-simulated or bf16-rounded values;
// other inputs lose bits below the 8th of the mantissa) and writes them row-major into LDS
// once. Scores S^T[slot][head] = K . Q^T run on v_mfma_f32_16x16x32_bf16 with the tile's rows
// as A and the wave's query heads as B, resident in registers as bf16 hi (+ lo: ~17 bits of
// q; the softmax scale is applied to the scores, so a bf16-valued q is exact in hi alone);
// the two halves of a pair meet through LDS. With slots as the tile's rows a lane ends
// up with 8 slots of ONE head, which is the A layout of the value MFMA, so P never leaves
// registers; the value operand is the same LDS tile through the transposing load
// (ds_read_b64_tr_b16). Online softmax in base 2 with a lazily moved reference maximum; three
// LDS tiles rotate so one barrier per tile suffices. Other widths (and rows that must not be
// rounded to bf16) take an f32 kernel: a wave per (query, head), lanes over the dims, one
// online-softmax pass over the list.
// Launch-only; see include/rivoli_kvcache.h for the contract.
#include "attend_common.hpp"

namespace rk {

constexpr int kGaD = 512;
constexpr int kGaThreads = 512;
constexpr int kGaWaves = kGaThreads / kWave;
constexpr int kGaTile = 32;                       // slots per LDS tile
constexpr int kGaKStepsHalf = kGaD / 32 / 2;      // 8 K-steps of the score contraction per wave of a pair
constexpr int kGaColTilesHalf = kGaD / 16 / 2;    // 16 output column tiles per wave of a pair
constexpr int kGaRowBytes = kGaD * 2 + 16;        // row-major tile: 1024 B of bf16 + 16 B pad
constexpr int kGaTileBytes = kGaTile * kGaRowBytes;
constexpr int kGaBufs = 3;
constexpr int kGaXchBytes = 2 * kGaWaves * kWave * 8 * 4;
constexpr int kGaSmemBytes = kGaBufs * kGaTileBytes + kGaBufs * kGaTile * 4 + kGaXchBytes;
static_assert(kGaSmemBytes <= 160 * 1024, "one workgroup per CU must fit the 160 KiB of LDS");

// Which row of a 16-row half of the LDS tile holds slot s of the half (the slot is the row index
// of the score MFMA's A operand and the contraction index of the value MFMA). The two ways the
// tile is read want different things of the row stride (1040 B = 65 granules of 16 B): the score
// side's 16-byte reads go eight lanes — eight consecutive slots — at a time and need their rows
// distinct mod 8; the transposing reads of the value side go sixteen lanes at a time, slots
// 4g .. 4g+3 with 32 bytes each, and need those four rows two apart mod 8 or neighbouring rows
// meet in half their banks (measured: one stalled LDS cycle for every cycle of those reads).
// Slots 0..3 -> rows 0 2 4 6, 4..7 -> 1 3 5 7, 8..11 -> 8 10 12 14, 12..15 -> 9 11 13 15.
__device__ __forceinline__ int row_of_slot(int s) { return 2 * (s & 7) + (s >> 3); }
__device__ __forceinline__ int slot_of_row(int p) { return 8 * (p & 1) + (p >> 1); }
// Staging wave w writes rows tile_pos_of(w, i) of the tile; the mask bias of such a row is kept
// at its slot's contraction index, 8 (s >> 2) + 4 half + (s & 3).
__device__ __forceinline__ int bias_index_of(int wave, int i) {
    const int s = slot_of_row(4 * (wave >> 1) + i);
    return 8 * (s >> 2) + 4 * (wave & 1) + (s & 3);
}

struct GatherAttnArgs {
    const float* q;      // [m][h][512]
    const float* kv;     // [rows][512]
    const float* sink;   // [h]
    const int* idxs;     // [m][topk]
    int h, topk;
    int n_kv;            // rows of kv; an index at or past it is treated as masked
    float qscale;        // softmax scale * log2(e)
    float* o;            // [m][h][512]
    int n_splits;        // > 1: blockIdx.z owns a share of the query's tiles and writes a partial
    float* part_acc;     // [m][n_splits][h][512] unnormalised accumulators
    float* part_ml;      // [m][n_splits][h][2] reference maximum (log2 units), sum of weights
};

// How many workgroups share one query's list: a pure function of the call's shape. Splitting
// pays when the queries alone cannot fill the part (decode: one query) and a share still
// holds a couple of tiles.
constexpr int kGaTargetGroups = 256;
constexpr int kGaMinTilesPerSplit = 2;
constexpr int kGaMaxSplits = 32;
static inline int gather_attn_splits(int m, int h, int topk) {
    const long long per_split = (long long)m * ((h + 63) / 64);
    const int tiles = (topk + kGaTile - 1) / kGaTile;
    long long n = (kGaTargetGroups + per_split - 1) / per_split;
    if (n > tiles / kGaMinTilesPerSplit) n = tiles / kGaMinTilesPerSplit;
    if (n > kGaMaxSplits) n = kGaMaxSplits;
    return n < 2 ? 1 : (int)n;
}

template <int QSPLIT, int PSPLIT>
__global__ __launch_bounds__(kGaThreads) void gather_attn_d512_kernel(const GatherAttnArgs a) {
    constexpr int kFragBlock = QSPLIT == 2 ? 2 : 4;   // score side, K-steps requested together
    constexpr int kValueAhead = QSPLIT == 2 ? 4 : 8;  // value side, fragments requested together
    __shared__ __attribute__((aligned(16))) uint8_t smem[kGaSmemBytes];
    const lds_ptr<uint8_t> kr = (lds_ptr<uint8_t>)smem;                     // [kGaBufs] row-major tiles
    const lds_ptr<float> sbias = (lds_ptr<float>)(kr + kGaBufs * kGaTileBytes);  // [kGaBufs][32]: 0 or -inf
    const lds_ptr<f32x4> xch = (lds_ptr<f32x4>)(sbias + kGaBufs * kGaTile);  // [2 parities][8 waves][64 lanes][2]

    const size_t t = blockIdx.x;
    const int hb = blockIdx.y;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hw = wave & 3;     // which 16 heads of the block
    const int half = wave >> 2;  // which half of the contraction dims / of the output columns
    const int g = lane >> 4, n16 = lane & 15;
    const int all_tiles = (a.topk + kGaTile - 1) / kGaTile;
    const int split = blockIdx.z;
    const int tile0 = (int)((long long)split * all_tiles / a.n_splits);  // this workgroup's tiles
    const int n_tiles = (int)((long long)(split + 1) * all_tiles / a.n_splits) - tile0;
    const int* const ix = a.idxs + t * a.topk;

    // ---- a tile's slots: lanes 0..3 hold the wave's 4 list entries ------------------------
    const int my_pos0 = tile_pos_of(wave, 0);  // the wave's 4 slots are consecutive tile positions
    // The fetch is unconditional (a position past the list reads the list's last entry) and
    // apart from the test of what it returns: a load under a per-lane condition compiles to a
    // branch that waits for its own data, and that wait (vmcnt(0)) would also drain the rows
    // requested for the tiles ahead — one exposed memory round trip per tile.
    auto list_fetch = [&](int tile) -> int {
        const long long pos = (long long)(tile0 + tile) * kGaTile + my_pos0 + (lane & 3);
        return ix[pos < a.topk ? pos : a.topk - 1];
    };
    auto list_entry = [&](int tile, int p) -> int {
        const long long pos = (long long)(tile0 + tile) * kGaTile + my_pos0 + (lane & 3);
        return (tile < n_tiles && lane < 4 && pos < a.topk && (unsigned)p < (unsigned)a.n_kv) ? p : -1;
    };
    struct RawTile {
        float4 row[4][2];
        float bias;  // lanes 0..3: 0, or -inf for a masked slot
        int live;    // bit i: row i was listed (a masked slot fetches row 0 and is staged as zeros)
    };
    auto issue_loads = [&](RawTile& r, int entry) {
        r.live = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int p = __builtin_amdgcn_readlane(entry, i);
            r.live |= (p >= 0 ? 1 : 0) << i;
            const float4* src = reinterpret_cast<const float4*>(a.kv + (size_t)(p >= 0 ? p : 0) * kGaD) + 2 * lane;
            r.row[i][0] = src[0], r.row[i][1] = src[1];
        }
        r.bias = entry >= 0 ? 0.0f : -INFINITY;
    };
    auto pack2 = [](float lo, float hi) -> uint32_t {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        const bf16x2 p = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, p);
    };
    auto stage = [&](const RawTile& r, int buf) {
        const lds_ptr<uint8_t> krb = kr + buf * kGaTileBytes;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u32x4 v = {pack2(r.row[i][0].x, r.row[i][0].y), pack2(r.row[i][0].z, r.row[i][0].w),
                       pack2(r.row[i][1].x, r.row[i][1].y), pack2(r.row[i][1].z, r.row[i][1].w)};
            if (!((r.live >> i) & 1)) v = u32x4{0u, 0u, 0u, 0u};
            *(lds_ptr<u32x4>)(krb + (my_pos0 + i) * kGaRowBytes + 16 * lane) = v;
        }
        if (lane < 4) sbias[buf * kGaTile + bias_index_of(wave, lane)] = r.bias;
    };

    // ---- prologue ------------------------------------------------------------------------
    // Everything the first tiles need is requested before anything is waited for: the list
    // entries of tiles 0..3, the query (oldest request, so its wait leaves the rows in
    // flight), the rows of tiles 0 and 1. Then: query -> B-operand fragments, tiles 0 and 1
    // staged, tile 2 requested.
    const int f0 = list_fetch(0), f1 = list_fetch(1), f2 = list_fetch(2), f3 = list_fetch(3);
    // this wave's half of its 16 query heads as the B operand, for the whole kernel
    bf16x8 qh[kGaKStepsHalf], ql[QSPLIT == 2 ? kGaKStepsHalf : 1];
    RawTile raw;
    raw.live = 0;
    {
        const int head = hb * 64 + 16 * hw + n16;
        const bool live = head < a.h;
        const float* qa = a.q + (t * a.h + (live ? head : 0)) * kGaD + half * (kGaD / 2) + 128 * (g & 1) + 8 * (g >> 1);
        float4 qv[kGaKStepsHalf][2];
#pragma unroll
        for (int j = 0; j < kGaKStepsHalf; ++j) {
            const float4* src = reinterpret_cast<const float4*>(qa + 16 * j);
            qv[j][0] = src[0], qv[j][1] = src[1];  // a head past h reads head 0 and is zeroed below
        }
        const int e0 = list_entry(0, f0), e1 = list_entry(1, f1);
        RawTile second;
        issue_loads(raw, e0);
        if (n_tiles > 1) issue_loads(second, e1);
#pragma unroll
        for (int j = 0; j < kGaKStepsHalf; ++j) {
            const float v[8] = {qv[j][0].x, qv[j][0].y, qv[j][0].z, qv[j][0].w,
                                qv[j][1].x, qv[j][1].y, qv[j][1].z, qv[j][1].w};
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float x = live ? v[i] : 0.0f;  // unscaled: a bf16-valued q stays exact in its hi part
                const __bf16 hi = (__bf16)x;
                qh[j][i] = hi;
                if (QSPLIT == 2) ql[j][i] = (__bf16)(x - (float)hi);
            }
        }
        stage(raw, 0);
        if (n_tiles > 1) stage(second, 1);
    }
    // A query that is bf16-valued (the model's is: its rotary stores bf16, crates/backend/kernels/
    // mla.hip:432) has no remainder: its lo fragments are zeros, their products exact zeros, and
    // the wave leaves those matrix instructions out — a quarter of the kernel's — with the same
    // sums to the bit.
    bool q_has_lo = false;
    if (QSPLIT == 2) {
        uint32_t any = 0;
#pragma unroll
        for (int j = 0; j < kGaKStepsHalf; ++j) {
            const u32x4 w = __builtin_bit_cast(u32x4, ql[j]);
            any |= w.x | w.y | w.z | w.w;
        }
        q_has_lo = __builtin_amdgcn_ballot_w64((any & 0x7fff7fffu) != 0) != 0;
    }
    if (n_tiles > 2) issue_loads(raw, list_entry(2, f2));
    int entry_next = list_entry(3, f3);
    __syncthreads();

    f32x4 o[kGaColTilesHalf];
#pragma unroll
    for (int nt = 0; nt < kGaColTilesHalf; ++nt) o[nt] = f32x4{0, 0, 0, 0};
    float m_ref = -INFINITY, l_sum = 0.0f;

    // Scores of one staged tile: this wave's half of the dims, S^T[slot][head], two 16-slot
    // halves. The operand fragments of a block of K-steps are requested one block ahead of the
    // MFMAs that use them: every wave of the workgroup runs the same phase at the same time, so
    // without the lookahead LDS sits idle while the matrix cores work and the matrix cores while
    // LDS delivers — the tile then costs the sum of the two, not the larger.
    auto scores_of = [&](int b, f32x4& s0, f32x4& s1) {
        const lds_ptr<uint8_t> krb = kr + b * kGaTileBytes + half * (kGaKStepsHalf * 64);
        // K-step j, lane group g: the 8 dims at bytes 256 (g & 1) + 32 j + 16 (g >> 1) of the
        // wave's half row (the query fragments follow the same rule). A 16-byte LDS read is
        // served sixteen lanes at a time, and those are lanes 0-3, 12-15, 20-23, 24-27 of a
        // 32-lane half, then the rest: eight rows from one lane group, the other eight from
        // the next. With rows an odd number of 16-byte granules apart the sixteen meet in no
        // bank exactly when the two lane groups read the same position mod 256 bytes.
        const int col = 256 * (g & 1) + 16 * (g >> 1);
        const lds_ptr<bf16x8> a0p = (lds_ptr<bf16x8>)(krb + row_of_slot(n16) * kGaRowBytes + col);
        const lds_ptr<bf16x8> a1p = (lds_ptr<bf16x8>)(krb + (16 + row_of_slot(n16)) * kGaRowBytes + col);
        s0 = f32x4{0, 0, 0, 0}, s1 = f32x4{0, 0, 0, 0};
        bf16x8 fa0[2][kFragBlock], fa1[2][kFragBlock];
#pragma unroll
        for (int i = 0; i < kFragBlock; ++i) fa0[0][i] = a0p[i * 2], fa1[0][i] = a1p[i * 2];
#pragma unroll
        for (int j0 = 0; j0 < kGaKStepsHalf; j0 += kFragBlock) {
            const int cur = (j0 / kFragBlock) & 1;
            if (j0 + kFragBlock < kGaKStepsHalf) {
#pragma unroll
                for (int i = 0; i < kFragBlock; ++i)
                    fa0[cur ^ 1][i] = a0p[(j0 + kFragBlock + i) * 2], fa1[cur ^ 1][i] = a1p[(j0 + kFragBlock + i) * 2];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < kFragBlock; ++i) {
                const int j = j0 + i;
                s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa0[cur][i], qh[j], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa1[cur][i], qh[j], s1, 0, 0, 0);
            }
            if (QSPLIT == 2) {
                // (the sums are used here so that the products above stay in front of the branch)
                asm volatile("" : "+v"(s0), "+v"(s1));
                if (q_has_lo) {
#pragma unroll
                    for (int i = 0; i < kFragBlock; ++i) {
                        const int j = j0 + i;
                        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa0[cur][i], ql[j], s0, 0, 0, 0);
                        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa1[cur][i], ql[j], s1, 0, 0, 0);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Iteration t: BARRIER -> the pair's scores of tile t meet -> scores of tile t+1 go to the
    // matrix cores -> softmax of tile t (vector ALU, while those run) -> values of tile t ->
    // this wave's half of the scores of tile t+1 to the exchange -> stage tile t+2 (in registers
    // since iteration t-1) -> request tile t+3 from memory. A wave past the barrier knows that
    // every wave has finished tile t-1 (so its LDS tile, (t+2) mod 3, may be overwritten), has
    // staged tile t+1 and has written its scores of tile t.
    int buf = 0;  // tile mod 3
    f32x4 s0, s1;
    scores_of(0, s0, s1);
    {
        const lds_ptr<f32x4> x = xch + ((0 * kGaWaves + wave) * kWave + lane) * 2;
        x[0] = s0, x[1] = s1;
    }
    for (int tile = 0; tile < n_tiles; ++tile) {
        const int fetch_ahead = list_fetch(tile + 4);  // looked at when this iteration ends
        const lds_ptr<f32x4> xch_peer = xch + (((tile & 1) * kGaWaves + (wave ^ 4)) * kWave + lane) * 2;
        const lds_ptr<f32x4> xch_next = xch + ((((tile + 1) & 1) * kGaWaves + wave) * kWave + lane) * 2;
        const int buf_next = buf == 2 ? 0 : buf + 1;
        // value-side operand of column tile nt: for each of the lane's 8 contraction indices
        // (slots 4g..4g+3 of both 16-slot halves) the value of column 16*nt' + n16. One
        // transposing load hands a lane element e of the 8-byte chunk that lane
        // 4e + (n16 >> 2) of its 16-lane row addressed, position n16 & 3 — so lane i
        // addresses slot 4g + (i >> 2), columns 16*nt' + 4*(i & 3) .. +3.
        const lds_ptr<uint8_t> vrow = kr + buf * kGaTileBytes + row_of_slot(4 * g + (n16 >> 2)) * kGaRowBytes +
                                      (half * (kGaD / 2) + 4 * (n16 & 3)) * 2;
        auto vt_frag = [&](int nt) -> bf16x8 {
            typedef short s16x4 __attribute__((ext_vector_type(4)));
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr<s16x4>)(vrow + nt * 32));
            const s16x4 hi =
                __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr<s16x4>)(vrow + 16 * kGaRowBytes + nt * 32));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            return __builtin_bit_cast(bf16x8, both);
        };
        const f32x4 ba = *(lds_ptr<f32x4>)(sbias + buf * kGaTile + 8 * g);
        const f32x4 bb = *(lds_ptr<f32x4>)(sbias + buf * kGaTile + 8 * g + 4);
        __syncthreads();  // both halves of every score of this tile are in LDS
        {
            const f32x4 p0 = xch_peer[0], p1 = xch_peer[1];
            s0 += p0, s1 += p1;  // a + b == b + a: the pair works on identical numbers
        }
        // ---- online softmax over the lane's 8 slots of head n16 ---------------------------
        bf16x8 p, p_lo;
        auto softmax_tile = [&]() {
            const float bias[8] = {ba.x, ba.y, ba.z, ba.w, bb.x, bb.y, bb.z, bb.w};
            float v[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[i] = __builtin_fmaf(s0[i], a.qscale, bias[i]);  // -inf where the slot is masked
                v[4 + i] = __builtin_fmaf(s1[i], a.qscale, bias[4 + i]);
            }
            float tmax =
                fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7])));
            tmax = rows_max(tmax);
            const bool grow = tmax > m_ref + kLazyRescale;  // false while everything is masked
            if (__builtin_amdgcn_ballot_w64(grow) != 0) {
                const float corr = grow ? __builtin_amdgcn_exp2f(m_ref - tmax) : 1.0f;  // 2^-inf = 0 at first
                if (grow) m_ref = tmax;
                l_sum *= corr;
                float c[4];  // the lane's accumulators are heads 4g+i; corr lives in lanes n16 == head
#pragma unroll
                for (int i = 0; i < 4; ++i) c[i] = __shfl(corr, 4 * g + i, kWave);
#pragma unroll
                for (int nt = 0; nt < kGaColTilesHalf; ++nt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[nt][i] *= c[i];
            }
            const float mu = m_ref == -INFINITY ? 0.0f : m_ref;
            // The value MFMA sees bf16(p_j), as hi + lo when PSPLIT == 2. Carried once, the
            // denominator sums the rounded weights — the ones the numerator really holds — so
            // the result is an exactly normalised average under weights perturbed by one bf16
            // rounding each.
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float e = __builtin_amdgcn_exp2f(v[i] - mu);  // masked -> 0
                const __bf16 w = (__bf16)e;
                p[i] = w;
                if (PSPLIT == 2) {
                    p_lo[i] = (__bf16)(e - (float)w);
                    l_sum += e;
                } else {
                    l_sum += (float)w;
                }
            }
        };
        // the next tile's scores go to the matrix cores before this tile's softmax occupies
        // the vector ALU (the two waves of a pair share a SIMD; running them in opposite order —
        // one starting an iteration with the scores, the other ending it with them — measured
        // 4 % slower)
        f32x4 ns0, ns1;
        const bool more = tile + 1 < n_tiles;
        auto softmax_and_values = [&]() {
            // the value side's first fragments come out of LDS while the softmax runs, every
            // later block while the block before it is in the matrix cores
            bf16x8 fb[2][kValueAhead];
#pragma unroll
            for (int i = 0; i < kValueAhead; ++i) fb[0][i] = vt_frag(i);
            __builtin_amdgcn_sched_barrier(0);
            softmax_tile();
            // O[head][col] += P . V over this wave's 256 columns
#pragma unroll
            for (int n0 = 0; n0 < kGaColTilesHalf; n0 += kValueAhead) {
                const int cur = (n0 / kValueAhead) & 1;
                if (n0 + kValueAhead < kGaColTilesHalf) {
#pragma unroll
                    for (int i = 0; i < kValueAhead; ++i) fb[cur ^ 1][i] = vt_frag(n0 + kValueAhead + i);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < kValueAhead; ++i) {
                    o[n0 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p, fb[cur][i], o[n0 + i], 0, 0, 0);
                    if (PSPLIT == 2)
                        o[n0 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_lo, fb[cur][i], o[n0 + i], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        if (more) scores_of(buf_next, ns0, ns1);
        softmax_and_values();

        if (more) {
            xch_next[0] = ns0, xch_next[1] = ns1;
            s0 = ns0, s1 = ns1;
        }
        // ---- stage tile + 2, request tile + 3 ---------------------------------------------
        if (tile + 2 < n_tiles) stage(raw, buf == 0 ? 2 : buf - 1);
        // the list entry fetched at the top is looked at BEFORE the rows are requested: past
        // the conditional request the compiler no longer knows how many loads are in flight
        // and would wait for all of them
        const int entry_now = entry_next;
        entry_next = list_entry(tile + 4, fetch_ahead);
        asm volatile("" : "+v"(entry_next));  // here, not wherever the scheduler would sink it
        if (tile + 3 < n_tiles) issue_loads(raw, entry_now);
        buf = buf_next;
    }

    // ---- epilogue: the sink joins the denominator, the quotient is rounded to bf16 ---------
    l_sum = rows_sum(l_sum);
    if (a.n_splits > 1) {
        // a share of the list: unnormalised accumulators and (m, l) for the combine kernel
        const size_t rec = (t * a.n_splits + split) * a.h;
        const int head0 = hb * 64 + 16 * hw;
        const int col0 = half * (kGaD / 2) + n16;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int head = head0 + 4 * g + i;
            if (head < a.h) {
                float* const dst = a.part_acc + (rec + head) * kGaD;
#pragma unroll
                for (int nt = 0; nt < kGaColTilesHalf; ++nt) dst[col0 + 16 * nt] = o[nt][i];
            }
        }
        if (half == 0 && g == 0 && head0 + n16 < a.h) {
            a.part_ml[(rec + head0 + n16) * 2] = m_ref;
            a.part_ml[(rec + head0 + n16) * 2 + 1] = l_sum;
        }
        return;
    }
    {
        const int head = hb * 64 + 16 * hw + n16;
        const float sk = head < a.h ? a.sink[head] : 0.0f;
        // the slots' weights are 2^(l2 - m_ref), so the sink's is 2^(sink * log2 e - m_ref);
        // nothing live: m_ref is still -inf and the query's output is NaN
        l_sum = m_ref == -INFINITY ? NAN : l_sum + exp2f(sk * kLog2e - m_ref);
    }
    // the lane's accumulators are heads 4g+i; their denominators live in lanes with n16 == 4g+i
    float l_h[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) l_h[i] = __shfl(l_sum, 4 * g + i, kWave);
    const int head0 = hb * 64 + 16 * hw;
    const int col0 = half * (kGaD / 2) + n16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int head = head0 + 4 * g + i;
        if (head < a.h) {
            float* const dst = a.o + (t * a.h + head) * kGaD;
#pragma unroll
            for (int nt = 0; nt < kGaColTilesHalf; ++nt)
                dst[col0 + 16 * nt] = (float)(__bf16)(o[nt][i] / l_h[i]);
        }
    }
}

// Split plan: o[t][head] = bf16(sum_r w_r acc_r / (sum_r w_r l_r + 2^(sink * log2 e - max m))),
// w_r = 2^(m_r - max m), over the query's shares in ascending order. Nothing live anywhere: NaN.
__global__ __launch_bounds__(128) void gather_attn_combine_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml,
    const float* __restrict__ sink, int n_splits, int h, float* __restrict__ o) {
    const int head = blockIdx.x;
    const size_t t = blockIdx.y;
    const size_t rec0 = t * n_splits * h + head;
    float m_g = -INFINITY;
    for (int r = 0; r < n_splits; ++r) m_g = fmaxf(m_g, part_ml[(rec0 + (size_t)r * h) * 2]);
    float4 sum = {0, 0, 0, 0};
    float l_g = NAN;
    if (m_g != -INFINITY) {
        l_g = 0.0f;
        for (int r = 0; r < n_splits; ++r) {
            const size_t rec = rec0 + (size_t)r * h;
            const float m_r = part_ml[rec * 2];
            if (m_r == -INFINITY) continue;
            const float w = exp2f(m_r - m_g);
            l_g += part_ml[rec * 2 + 1] * w;
            const float4 v = reinterpret_cast<const float4*>(part_acc + rec * kGaD)[threadIdx.x];
            sum.x += v.x * w, sum.y += v.y * w, sum.z += v.z * w, sum.w += v.w * w;
        }
        l_g += exp2f(sink[head] * kLog2e - m_g);
    }
    float4* const dst = reinterpret_cast<float4*>(o + (t * h + head) * kGaD) + threadIdx.x;
    *dst = float4{(float)(__bf16)(sum.x / l_g), (float)(__bf16)(sum.y / l_g), (float)(__bf16)(sum.z / l_g),
                  (float)(__bf16)(sum.w / l_g)};
}

// Any width, and rows kept exactly as they are (no rounding to bf16): a wave per (query, head),
// the four heads of a workgroup walking the same query's list together so that a listed row
// comes out of the first-level cache for three of them. A lane owns dims lane, lane + 64, ...:
// the query and the running output sit in its registers, a slot is one coalesced pass over the
// row (kept for the value side), a butterfly sum, and an online-softmax update. One pass over
// the list, no LDS, no barrier; a masked slot (index outside [0, n_kv)) is never dereferenced.
constexpr int kGaRowThreads = 256;
constexpr int kGaRowDims = 16;  // dims per lane: d <= 1024

__global__ __launch_bounds__(kGaRowThreads) void gather_attn_rowwise_kernel(
    const float* __restrict__ q, const float* __restrict__ kv, const float* __restrict__ sink,
    const int* __restrict__ idxs, int h, int d, int topk, int n_kv, float scale,
    float* __restrict__ o) {
    const int lane = threadIdx.x & (kWave - 1);
    const int head = (int)blockIdx.x * (kGaRowThreads / kWave) + (threadIdx.x >> 6);
    if (head >= h) return;
    const size_t t = blockIdx.y;
    const float* qrow = q + (t * h + head) * d;
    const int* list = idxs + t * topk;
    const int steps = (d + kWave - 1) / kWave;  // wave-uniform
    float qv[kGaRowDims], acc[kGaRowDims];
#pragma unroll
    for (int c = 0; c < kGaRowDims; ++c) {
        const int i = lane + c * kWave;
        qv[c] = (c < steps && i < d) ? qrow[i] * (scale * kLog2e) : 0.0f;  // scores in log2 units
        acc[c] = 0.0f;
    }
    float top = -INFINITY, denom = 0.0f;
    for (int j = 0; j < topk; ++j) {
        const int row = list[j];
        if ((unsigned)row >= (unsigned)n_kv) continue;  // masked (wave-uniform)
        const float* src = kv + (size_t)row * d;
        float val[kGaRowDims], dot = 0.0f;
#pragma unroll
        for (int c = 0; c < kGaRowDims; ++c) {
            const int i = lane + c * kWave;
            val[c] = (c < steps && i < d) ? src[i] : 0.0f;
            dot += qv[c] * val[c];
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, kWave);
        const float top_new = fmaxf(top, dot);
        const float keep = exp2f(top - top_new), w = exp2f(dot - top_new);  // 2^-inf = 0 on the first slot
        denom = denom * keep + w;
#pragma unroll
        for (int c = 0; c < kGaRowDims; ++c) acc[c] = acc[c] * keep + w * val[c];
        top = top_new;
    }
    // the sink joins the denominator only; a query whose every slot is masked has no maximum
    // to measure the sink against and comes out NaN, as in the reference (attn.hip:415-420)
    const float total = top == -INFINITY ? NAN : denom + exp2f(sink[head] * kLog2e - top);
    float* orow = o + (t * h + head) * d;
#pragma unroll
    for (int c = 0; c < kGaRowDims; ++c) {
        const int i = lane + c * kWave;
        if (c < steps && i < d) orow[i] = (float)(__bf16)(acc[c] / total);
    }
}

static int gather_attn_launch(const float* q, const float* kv, const float* sink, const int* idxs,
                              int m, int h, int d, int topk, int n_kv, float scale, int precise,
                              float* o, float* partial, hipStream_t stream) {
    if (!q || !kv || !sink || !idxs || !o) return 1001;
    if (m <= 0 || h <= 0 || d <= 0 || topk <= 0 || n_kv <= 0) return 1001;
    (void)hipGetLastError();
    if (precise < 3 && d == kGaD && aligned16(q) && aligned16(kv) && aligned16(o) && (h + 63) / 64 <= 65535) {
        GatherAttnArgs a;
        a.q = q, a.kv = kv, a.sink = sink, a.idxs = idxs;
        a.h = h, a.topk = topk, a.n_kv = n_kv, a.qscale = scale * kLog2e, a.o = o;
        // a caller without a partial buffer gets the one-workgroup-per-query plan
        a.n_splits = partial && aligned16(partial) ? gather_attn_splits(m, h, topk) : 1;
        a.part_acc = partial;
        a.part_ml = partial ? partial + (size_t)m * a.n_splits * h * kGaD : nullptr;
        const dim3 grid((unsigned)m, (unsigned)((h + 63) / 64), (unsigned)a.n_splits);
        if (precise >= 2)
            hipLaunchKernelGGL((gather_attn_d512_kernel<2, 2>), grid, dim3(kGaThreads), 0, stream, a);
        else if (precise == 1)
            hipLaunchKernelGGL((gather_attn_d512_kernel<2, 1>), grid, dim3(kGaThreads), 0, stream, a);
        else
            hipLaunchKernelGGL((gather_attn_d512_kernel<1, 1>), grid, dim3(kGaThreads), 0, stream, a);
        const int rc = launch_status();
        if (rc != 0 || a.n_splits == 1) return rc;  // a split plan has fewer than 256 queries
        hipLaunchKernelGGL(gather_attn_combine_kernel, dim3((unsigned)h, (unsigned)m), dim3(128), 0, stream,
                           a.part_acc, a.part_ml, sink, a.n_splits, h, o);
        return launch_status();
    }
    // the reference launcher's limits, kept (attn.hip:450-458): d within 1024, its LDS budget
    if (d > kGaRowDims * kWave || m > 65535) return 1002;
    if (((size_t)d + (size_t)topk + 256 + 2) * sizeof(float) > 65536) return 1006;
    hipLaunchKernelGGL(gather_attn_rowwise_kernel,
                       dim3((unsigned)((h + kGaRowThreads / kWave - 1) / (kGaRowThreads / kWave)), (unsigned)m),
                       dim3(kGaRowThreads), 0, stream, q, kv, sink, idxs, h, d, topk, n_kv, scale, o);
    return launch_status();
}

}  // namespace rk

extern "C" int rivoli_gather_attn_shared_kv(const float* q, const float* kv, const float* sink,
                                            const int* idxs, int m, int h, int d, int topk,
                                            float scale, float* o, void* stream) {
    return rk::gather_attn_launch(q, kv, sink, idxs, m, h, d, topk, 0x7fffffff, scale, 2, o, nullptr,
                                  (hipStream_t)stream);
}

extern "C" int rivoli_gather_attn_shared_kv_bounded(const float* q, const float* kv,
                                                    const float* sink, const int* idxs, int m,
                                                    int h, int d, int topk, int n_kv, float scale,
                                                    int precise, float* o, void* stream) {
    return rk::gather_attn_launch(q, kv, sink, idxs, m, h, d, topk, n_kv, scale, precise, o, nullptr,
                                  (hipStream_t)stream);
}

extern "C" size_t rivoli_gather_attn_scratch_floats(int m, int h, int d, int topk) {
    if (m <= 0 || h <= 0 || topk <= 0 || d != rk::kGaD) return 0;
    const int n = rk::gather_attn_splits(m, h, topk);
    return n > 1 ? (size_t)m * n * h * (rk::kGaD + 2) : 0;
}

extern "C" int rivoli_gather_attn_shared_kv_split(const float* q, const float* kv, const float* sink,
                                                  const int* idxs, int m, int h, int d, int topk,
                                                  int n_kv, float scale, int precise, float* o,
                                                  float* partial, void* stream) {
    if (rivoli_gather_attn_scratch_floats(m, h, d, topk) > 0 && (!partial || !rk::aligned16(partial)))
        return 1001;
    return rk::gather_attn_launch(q, kv, sink, idxs, m, h, d, topk, n_kv, scale, precise, o, partial,
                                  (hipStream_t)stream);
}
