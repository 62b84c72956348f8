// MLA decode attention in latent space, reading the paged fp8 cache directly.
//
// For one decoded token per sequence and every head h:
//
//     clat_h = sum_t softmax_t((qabs_h . L_t + qrope_h . R_t) * scale) * L_t
//
// which is what the reference's mla_latent_attend computes over its linear slabs
// (crates/backend/kernels/attn.hip:1-17,119-233; combine :235-277). Here a token is one
// 576-byte row of e4m3 codes (512 latent + 64 rope) with ONE f32 scale, so
//     L_t = s_t * dec(c_t[0:512]),  R_t = s_t * dec(c_t[512:576]),
// the per-token scale factors out of both contractions, and the codes themselves (exact in
// bf16) are what the matrix cores see:
//     score_t = s_t * scale * (q . dec(c_t)),     clat_h = sum_t (p_t * s_t) * dec(c_t[0:512]).
// Nothing is materialised: a token costs 580 bytes of HBM traffic instead of the 580 + 1152
// + 1152 of gather-then-attend.
//
// Mapping. A 512-thread workgroup (8 waves, two per SIMD) owns a block of 64 heads and a run
// of 32-token tiles: all of one sequence for small calls; otherwise an equal share of the
// whole batch's tiles, dealt from the device-side lengths, which may cover parts of several
// sequences (one partial record per part). Waves w and w+4 share heads 16(w&3)..+15 and split the
// work on them: each takes half of the 576 contraction dims of the scores and half of the
// 512 output columns. That halves the query registers and the accumulators a wave carries
// (the whole kernel fits the 256 registers a wave gets at two waves per SIMD, so every MFMA
// keeps its accumulator in place), and the second wave per SIMD covers the first one's
// softmax and staging. Tokens move in tiles of 32:
//   * staging: wave w fetches 4 tokens of the tile (one fully coalesced 512-byte run per
//     token for the latent, 64 bytes for the rope), converts e4m3 -> bf16 in registers and
//     writes them row-major [token][dim] into LDS, once. The score contraction (over dims)
//     reads its operands from that tile directly; the value contraction (over tokens)
//     reads the same tile through gfx950's transposing LDS load (ds_read_b64_tr_b16), so no
//     second, transposed copy is written. Three tiles rotate: a tile is staged two
//     iterations before it is consumed and loaded from memory one iteration before that,
//     which leaves ONE barrier per tile (the one the score exchange needs anyway).
//   * scores: S^T[token][head] = K . Q^T with v_mfma_f32_16x16x32_bf16, A = the tile's rows
//     from LDS, B = the wave's half of its query heads, resident in registers for the whole
//     kernel (optionally as bf16 hi + lo, two MFMAs per step, ~17 bits of q). The two
//     partial sums of a pair meet through LDS; both waves then run the same softmax on the
//     same numbers. With tokens as the tile's rows a lane ends up holding 8 tokens of ONE
//     head, which is exactly the A-operand layout of the value MFMA — P never leaves
//     registers. The tile's token order inside the value contraction is whatever that
//     layout implies; the transposing loads address the rows in the same order.
//   * softmax: online, base 2 (log2 e folded into q); the running maximum only moves when a
//     tile exceeds it by more than 2^8 (the f32 accumulators have the range), so rescaling
//     the accumulators is rare.
//   * values: O[head][col] += P . V over the wave's 256 columns, B = transposing loads.
// Parts write unnormalised partials (acc, m, l) that mla_attend_combine_kernel merges in
// ascending order; the plan is a pure function of the call's shape and of the lengths, so
// equal calls give bit-equal results.
// Launch-only; see include/rivoli_kvcache.h for the contract of every entry point.
#include <type_traits>

#include "attend_common.hpp"

namespace rk {

constexpr int kKvl = 512, kRopeW = 64, kRowW = kKvl + kRopeW;
constexpr int kAttThreads = 512;
constexpr int kAttWaves = kAttThreads / kWave;
constexpr int kTile = 32;                  // tokens per LDS tile
constexpr int kKSteps = kRowW / 32;        // 18 K-steps of the score contraction ...
constexpr int kKStepsHalf = kKSteps / 2;   // ... 9 per wave of a pair
constexpr int kColTilesHalf = kKvl / 16 / 2;  // 16 output column tiles per wave of a pair
constexpr int kKrRowBytes = kRowW * 2 + 16;  // row-major tile: 1152 B of bf16 + 16 B pad
constexpr int kKrBytes = kTile * kKrRowBytes;
constexpr int kBufs = 3;                   // LDS tiles in rotation: tile t is staged while t-2 is consumed
constexpr int kXchBytes = 2 * kAttWaves * kWave * 8 * 4;  // partial scores, 8 f32 per lane, two parities
constexpr int kTableLds = 1024;            // block-table entries staged per workgroup
constexpr int kBlockScaleBytes = kBufs * kTile * 16;  // linear slabs: four block scales per token
constexpr int kAttSmemBytes =
    kBufs * kKrBytes + 2 * kBufs * kTile * 4 + kXchBytes + kTableLds * 4 + kBlockScaleBytes;
static_assert(kAttSmemBytes + (1024 + 8 + 8) * 4 <= 160 * 1024, "one workgroup per CU must fit the 160 KiB of LDS");

// Work plan. `n_splits` is a pure function of the call's shape; with more than one split the
// attended rows of ALL sequences, in tiles, are dealt evenly to n_seqs * n_splits work items
// from the device-side lengths (a work item may cover parts of several sequences, a sequence
// several work items), so ragged batches keep every CU busy.
constexpr int kAttTargetGroups = 256;      // one workgroup per CU of a 256-CU part
constexpr int kAttMinTilesPerSplit = 8;    // below 256 rows a split costs more than it buys
constexpr int kAttMaxSplits = 64;
constexpr int kDealMaxSeqs = 1024;         // dealing keeps a prefix sum over the sequences in LDS

struct AttendPlan {
    int n_splits;
    int n_items;    // work items per head block when dealing (0 = one workgroup per sequence)
    int n_records;  // partial records when dealing: a (work item, sequence) pair is item + seq
};

static inline AttendPlan attend_plan(int n_seqs, int H, int max_rows) {
    const int head_blocks = (H + 63) / 64;
    const int tiles = (max_rows + kTile - 1) / kTile;
    const long long per_split = (long long)n_seqs * head_blocks;
    int by_grid = (int)((kAttTargetGroups + per_split - 1) / per_split);
    int by_work = tiles / kAttMinTilesPerSplit;
    int n = by_grid < by_work ? by_grid : by_work;
    if (n > kAttMaxSplits) n = kAttMaxSplits;
    if (n < 1 || n_seqs > kDealMaxSeqs) n = 1;
    AttendPlan p;
    p.n_splits = n;
    p.n_items = n > 1 ? n * n_seqs : 0;
    p.n_records = n > 1 ? p.n_items + n_seqs : 0;
    return p;
}

// The tiles of work item `item` of `n_items` over `total` tiles: [lo, hi).
__host__ __device__ __forceinline__ long long deal_lo(long long item, long long n_items, long long total) {
    return item * total / n_items;
}
// The work item that holds tile `t` (the largest item whose first tile is <= t).
__device__ __forceinline__ int deal_item_of(long long t, long long n_items, long long total) {
    return (int)(((t + 1) * n_items - 1) / total);
}

// e4m3 codes -> bf16, exact: four codes (one dword) -> two dwords
__device__ __forceinline__ void e4m3x4_to_bf16(uint32_t c, uint32_t& lo, uint32_t& hi) {
    lo = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(c, 1.0f, false));
    hi = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(c, 1.0f, true));
}

struct AttendArgs {
    const float* qabs;            // [n_seqs][H][512]
    const float* qrope;           // [n_seqs][H][64]
    const uint8_t* pool;
    const int* block_table;       // [n_seqs][max_blocks]
    const int* seq_lens;          // dense: attended rows per sequence
    const unsigned int* rows;     // sparse: [n_seqs][k] token indices (null = dense)
    const int* n_rows;            // sparse: rows per sequence (null = k)
    int k;
    int H, max_blocks, page_tokens, n_pages;
    int kvl, rope, row_w;         // widths of a cache row: latent, rope, and their sum (512 / 64 / 576 on the fast path)
    // MODE == kLinear, the reference's slabs: e4m3 latent codes [t][kvl] with one f32 scale per
    // 128 of them [t][n_blocks], and the roped key as bf16 [t][rope]
    const uint8_t* lc8;
    const float* lscale;
    const uint16_t* rc;
    int n_blocks;
    int page_shift;               // log2(page_tokens) when that is a power of two, else -1
    size_t page_bytes;
    float qscale;                 // softmax scale * log2(e)
    int n_seqs, n_items;          // n_items > 0: tiles are dealt to that many work items
    float* clat;                  // [n_seqs][H][512]
    float* part_acc;              // [n_records][H][512]
    float* part_ml;               // [n_records][H][2]
    unsigned int* bad_rows;
};

// MODE: how a tile's tokens are found.
enum : int {
    kDense = 0,      // token = row position, any page size: one table lookup per token
    kSparse = 1,     // token = rows[position]: one list entry and one table lookup per token
    kDensePaged = 2, // token = row position and page_tokens is a power of two >= the tile: a
                     // tile lies inside ONE page, so a tile costs one (scalar) table lookup
    kLinear = 3      // the reference's linear slabs (one sequence): token = rows ? rows[position]
                     // : position, addressed by the token index, block scales, bf16 rope
};
// ANY: the row widths are runtime values (kvl a multiple of 128 up to 512, rope up to 64): the
// tile keeps its 512 + 64 layout and the dims a cache does not have are staged as zeros, so a
// narrower cache costs the matrix cores the same as the full one. The fast path (ANY = false)
// is the shipped 512 + 64 row.

// One part of a workgroup's work: rows [r_begin, r_end) of sequence `seq`, heads 64*hb ..+63.
// `whole`: the part is the whole sequence, so the normalised result goes straight to clat;
// otherwise the unnormalised accumulators and (m, l) go to the partial record pa / pml.
template <int QSPLIT, int PSPLIT, int MODE, bool ANY>
__device__ __forceinline__ void attend_part(const AttendArgs& a, int seq, int hb, int r_begin,
                                                      int r_end, bool whole, float* pa, float* pml) {
    constexpr bool SPARSE = MODE == kSparse;
    constexpr bool LINEAR = MODE == kLinear;
    static_assert(!LINEAR || (ANY && QSPLIT == 2 && PSPLIT == 2), "the linear slabs run in the parity mode");
    const int kvl = ANY ? a.kvl : kKvl, ropew = ANY ? a.rope : kRopeW, row_w = ANY ? a.row_w : kRowW;
    // operand fragments requested together ahead of the MFMAs that consume them: as many
    // as the register budget of two waves per SIMD (256) leaves room for
    constexpr int kFragBlock = QSPLIT == 2 ? 3 : 9;   // score side, K-steps (2 fragments each)
    constexpr int kValueAhead = QSPLIT == 2 ? 4 : 8;  // value side, fragments
    __shared__ __attribute__((aligned(16))) uint8_t smem[kAttSmemBytes];
    // Every LDS pointer below is typed as such. Left generic, the pointers become loop-carried
    // once this body sits in the dealing kernel's loop over parts, the compiler can no longer
    // prove they are LDS, and its fallback (flat addressing) fails in instruction selection.
    const lds_ptr<uint8_t> kr = (lds_ptr<uint8_t>)smem;  // [kBufs] row-major tiles
    // per token of a tile, by contraction index: its scale (0 when the token is not there)
    // and a score bias (0, or -inf when it is not there): score = s * scale + bias
    const lds_ptr<float> sc = (lds_ptr<float>)(kr + kBufs * kKrBytes);    // [kBufs][32]
    const lds_ptr<float> sbias = sc + kBufs * kTile;                       // [kBufs][32]
    const lds_ptr<f32x4> xch = (lds_ptr<f32x4>)(sbias + kBufs * kTile);    // [2 parities][8 waves][64 lanes][2]
    const lds_ptr<int> tbl = (lds_ptr<int>)(xch + 2 * kAttWaves * kWave * 2);
    const lds_ptr<f32x4> sc4 = (lds_ptr<f32x4>)(tbl + kTableLds);  // [kBufs][32], linear slabs only


    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hw = wave & 3;    // which 16 heads of the block
    const int half = wave >> 2; // which half of the contraction dims / of the output columns
    const int g = lane >> 4, n16 = lane & 15;

    const int n_tiles = (r_end - r_begin + kTile - 1) / kTile;

    // ---- block-table slice into LDS -----------------------------------------------------
    const int* const table_g = LINEAR ? nullptr : a.block_table + (size_t)seq * a.max_blocks;
    const int tbl_first = (SPARSE || LINEAR) ? 0 : r_begin / a.page_tokens;
    const int tbl_last = SPARSE ? a.max_blocks - 1 : min(a.max_blocks - 1, (r_end - 1) / a.page_tokens);
    const int tbl_count = LINEAR ? 0 : min(kTableLds, tbl_last - tbl_first + 1);
    for (int i = tid; i < tbl_count; i += kAttThreads) tbl[i] = table_g[tbl_first + i];

    // ---- this wave's half of its 16 query heads as the B operand, for the whole kernel ---
    bf16x8 qh[kKStepsHalf], ql[QSPLIT == 2 ? kKStepsHalf : 1];
    {
        const int head = hb * 64 + 16 * hw + n16;
        const bool live = head < a.H;
        const size_t qrow = (size_t)seq * a.H + (live ? head : 0);
        const float* qa = a.qabs + qrow * kvl + 8 * g;
        const float* qr = a.qrope + qrow * ropew + 8 * g;
#pragma unroll
        for (int j = 0; j < kKStepsHalf; ++j) {
            const int ks = half * kKStepsHalf + j;  // uniform: 0..8 or 9..17 (16, 17 are the rope)
            float v[8];
            if constexpr (!ANY) {
                const float4* src = reinterpret_cast<const float4*>(ks < 16 ? qa + 32 * ks : qr + 32 * (ks - 16));
                float4 v0 = {0, 0, 0, 0}, v1 = {0, 0, 0, 0};
                if (live) v0 = src[0], v1 = src[1];
                v[0] = v0.x, v[1] = v0.y, v[2] = v0.z, v[3] = v0.w, v[4] = v1.x, v[5] = v1.y, v[6] = v1.z, v[7] = v1.w;
            } else {  // a dim this cache does not have multiplies a staged zero: its q is zero too
                const float* src = ks < 16 ? qa + 32 * ks : qr + 32 * (ks - 16);
                const int left = (ks < 16 ? kvl - 32 * ks : ropew - 32 * (ks - 16)) - 8 * g;
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = (live && i < left) ? src[i] : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float x = v[i] * a.qscale;
                const __bf16 hi = (__bf16)x;
                qh[j][i] = hi;
                if (QSPLIT == 2) ql[j][i] = (__bf16)(x - (float)hi);
            }
        }
    }
    __syncthreads();  // table slice visible

    auto table_at = [&](int blk) -> int {
        const int rel = blk - tbl_first;
        return (rel >= 0 && rel < tbl_count) ? tbl[rel] : table_g[blk];
    };

    // ---- where a tile's tokens are ------------------------------------------------------
    // General form (kDense, kSparse): lanes 0..3 resolve the wave's 4 tokens: row position ->
    // token -> page -> byte offsets of the code row and of the scale; offset ~0 marks a
    // token that is not there (past the end of the split, or its page id outside the pool).
    // kDensePaged: the whole tile is `n_here` consecutive rows of one page starting at
    // `tile_off`, all wave-uniform.
    constexpr unsigned long long kNone = ~0ull;
    struct Where {
        unsigned long long code_off, scale_off;  // per lane (lanes 0..3), general form
        unsigned long long tile_off, tile_scale_off;  // uniform, kDensePaged
        int n_here;                                    // uniform, kDensePaged: valid rows in the tile
    };
    const unsigned int* const rows_g = SPARSE ? a.rows + (size_t)seq * a.k : (LINEAR ? a.rows : nullptr);
    auto row_token = [&](int tile) -> unsigned int {  // sparse: the row list entry, else the position
        if (MODE == kDensePaged) return 0;
        const int pos = r_begin + tile * kTile + tile_pos_of(wave, lane & 3);
        if (lane >= 4 || pos >= r_end) return 0xffffffffu;
        if (LINEAR) return rows_g ? rows_g[pos] : (unsigned)pos;
        return SPARSE ? rows_g[pos] : (unsigned)pos;
    };
    auto resolve = [&](int tile, unsigned int tok, Where& w) {
        if (MODE == kDensePaged) {
            const int pos0 = r_begin + tile * kTile;  // uniform; the split starts on a tile boundary
            w.n_here = 0, w.tile_off = 0, w.tile_scale_off = 0;
            if (pos0 >= r_end) return;
            const int blk = pos0 >> a.page_shift, off = pos0 & (a.page_tokens - 1);
            // a position the block table has no entry for is skipped and counted, like a page
            // id outside the pool: the table row of the next sequence is never read
            const int page = blk < a.max_blocks ? __builtin_amdgcn_readfirstlane(table_at(blk)) : -1;
            const int n = min(kTile, r_end - pos0);
            if ((unsigned)page < (unsigned)a.n_pages) {
                w.n_here = n;
                w.tile_off = (unsigned long long)page * a.page_bytes + (unsigned long long)off * row_w;
                w.tile_scale_off = (unsigned long long)page * a.page_bytes +
                                   (unsigned long long)a.page_tokens * row_w + (unsigned long long)off * 4;
            } else if (a.bad_rows && hb == 0 && tid == 0) {
                atomicAdd(a.bad_rows, (unsigned)n);
            }
            return;
        }
        w.code_off = kNone, w.scale_off = 0;
        if (tok == 0xffffffffu) return;
        if (LINEAR) {  // addressed by the token index itself
            w.code_off = tok;
            return;
        }
        unsigned int blk, off;
        if (a.page_shift >= 0) blk = tok >> a.page_shift, off = tok & (unsigned)(a.page_tokens - 1);
        else blk = tok / (unsigned)a.page_tokens, off = tok - blk * (unsigned)a.page_tokens;
        const int page = blk < (unsigned)a.max_blocks ? table_at((int)blk) : -1;
        if ((unsigned)page < (unsigned)a.n_pages) {
            const unsigned long long pbase = (unsigned long long)page * a.page_bytes;
            w.code_off = pbase + (unsigned long long)off * row_w;
            w.scale_off = pbase + (unsigned long long)a.page_tokens * row_w + (unsigned long long)off * 4;
        } else if (a.bad_rows && hb == 0) {
            atomicAdd(a.bad_rows, 1u);
        }
    };

    u32x2 raw[4];
    uint32_t raw_rope;          // four rope codes; linear slabs: raw_rope / raw_rope_hi hold four bf16
    uint32_t raw_rope_hi = 0;
    float raw_scale, raw_bias;  // lanes 0..3
    f32x4 raw_scale4 = {0, 0, 0, 0};  // linear slabs, lanes 0..3: the token's block scales
    const int my_pos0 = tile_pos_of(wave, 0);  // the wave's 4 tokens are consecutive tile positions
    // ANY: a lane whose chunk lies past the row's latent (rope) width loads the row's first
    // chunk instead and discards it: no branch sits between the loads of a tile
    const bool lat_ok = !ANY || 8 * lane < kvl;
    const bool rope_ok = !ANY || 4 * (lane & 15) < ropew;
    const int lat_at = lat_ok ? 8 * lane : 0, rope_at = kvl + (rope_ok ? 4 * (lane & 15) : 0);
    auto issue_loads = [&](const Where& w) {
        if (MODE == kDensePaged) {
            const uint8_t* const base = a.pool + w.tile_off + (size_t)my_pos0 * row_w;
            if (my_pos0 + 3 < w.n_here) {  // the common case: all four rows are there
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    raw[i] = *reinterpret_cast<const u32x2*>(base + i * row_w + lat_at);
                raw_rope = *reinterpret_cast<const uint32_t*>(base + (lane >> 4) * row_w + rope_at);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    raw[i] = u32x2{0, 0};
                    if (my_pos0 + i < w.n_here) raw[i] = *reinterpret_cast<const u32x2*>(base + i * row_w + lat_at);
                }
                raw_rope = 0;
                if (my_pos0 + (lane >> 4) < w.n_here)
                    raw_rope = *reinterpret_cast<const uint32_t*>(base + (lane >> 4) * row_w + rope_at);
            }
            if (ANY) {
#pragma unroll
                for (int i = 0; i < 4; ++i) raw[i] = lat_ok ? raw[i] : u32x2{0, 0};
                raw_rope = rope_ok ? raw_rope : 0u;
            }
            raw_scale = 0.0f, raw_bias = -INFINITY;
            if (lane < 4 && my_pos0 + lane < w.n_here) {
                raw_scale = *reinterpret_cast<const float*>(a.pool + w.tile_scale_off + (size_t)(my_pos0 + lane) * 4);
                raw_bias = 0.0f;
            }
            return;
        }
        const uint32_t lo = (uint32_t)w.code_off, hi = (uint32_t)(w.code_off >> 32);
        if constexpr (LINEAR) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t blo = __builtin_amdgcn_readlane(lo, i), bhi = __builtin_amdgcn_readlane(hi, i);
                const unsigned long long t = ((unsigned long long)bhi << 32) | blo;
                raw[i] = u32x2{0, 0};
                if (t != kNone && lat_ok) raw[i] = *reinterpret_cast<const u32x2*>(a.lc8 + t * kvl + 8 * lane);
            }
            // the roped key is bf16 already: four values per lane, read one by one (any width, any alignment)
            const unsigned long long tr = __shfl(w.code_off, lane >> 4, kWave);
            uint32_t r4[4] = {0, 0, 0, 0};
            if (tr != kNone) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int d = 4 * (lane & 15) + e;
                    if (d < ropew) r4[e] = a.rc[tr * ropew + d];
                }
            }
            raw_rope = r4[0] | (r4[1] << 16), raw_rope_hi = r4[2] | (r4[3] << 16);
            raw_scale = 0.0f, raw_bias = -INFINITY, raw_scale4 = f32x4{0, 0, 0, 0};
            if (lane < 4 && w.code_off != kNone) {
                const float* sp = a.lscale + w.code_off * a.n_blocks;
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    if (128 * b < kvl) raw_scale4[b] = sp[b];
                raw_scale = 1.0f, raw_bias = 0.0f;
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t blo = __builtin_amdgcn_readlane(lo, i), bhi = __builtin_amdgcn_readlane(hi, i);
            const unsigned long long b = ((unsigned long long)bhi << 32) | blo;
            raw[i] = u32x2{0, 0};
            if (b != kNone && lat_ok) raw[i] = *reinterpret_cast<const u32x2*>(a.pool + b + 8 * lane);
        }
        const unsigned long long br = __shfl(w.code_off, lane >> 4, kWave);
        raw_rope = 0;
        if (br != kNone && rope_ok) raw_rope = *reinterpret_cast<const uint32_t*>(a.pool + br + kvl + 4 * (lane & 15));
        raw_scale = 0.0f, raw_bias = -INFINITY;
        if (lane < 4 && w.code_off != kNone) {
            raw_scale = *reinterpret_cast<const float*>(a.pool + w.scale_off);
            raw_bias = 0.0f;
        }
    };
    auto stage = [&](int buf) {
        const lds_ptr<uint8_t> krb = kr + buf * kKrBytes;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t r[4];
            e4m3x4_to_bf16(raw[i].x, r[0], r[1]);
            e4m3x4_to_bf16(raw[i].y, r[2], r[3]);
            *(lds_ptr<u32x4>)(krb + (my_pos0 + i) * kKrRowBytes + 16 * lane) = u32x4{r[0], r[1], r[2], r[3]};
        }
        uint32_t rr0, rr1;
        if constexpr (LINEAR) rr0 = raw_rope, rr1 = raw_rope_hi;
        else e4m3x4_to_bf16(raw_rope, rr0, rr1);
        *(lds_ptr<u32x2>)(krb + (my_pos0 + (lane >> 4)) * kKrRowBytes + kKvl * 2 + 8 * (lane & 15)) =
            u32x2{rr0, rr1};
        if (LINEAR && lane < 4) sc4[buf * kTile + 4 * wave + lane] = raw_scale4;
        if (lane < 4) {
            // a scale that is not a positive number cannot come from the append: such a
            // token is left out like one that is not there
            const bool ok = raw_scale > 0.0f;
            sc[buf * kTile + 4 * wave + lane] = ok ? raw_scale : 0.0f;
            sbias[buf * kTile + 4 * wave + lane] = ok ? raw_bias : -INFINITY;
        }
    };

    // ---- prologue: tiles 0 and 1 staged, tile 2 in registers, tile 3 resolved ------------
    Where where;
    resolve(0, row_token(0), where);
    issue_loads(where);
    stage(0);
    resolve(1, n_tiles > 1 ? row_token(1) : 0xffffffffu, where);
    if (n_tiles > 1) {
        issue_loads(where);
        stage(1);
    }
    resolve(2, n_tiles > 2 ? row_token(2) : 0xffffffffu, where);
    if (n_tiles > 2) issue_loads(where);
    resolve(3, n_tiles > 3 ? row_token(3) : 0xffffffffu, where);
    __syncthreads();

    f32x4 o[kColTilesHalf];
#pragma unroll
    for (int nt = 0; nt < kColTilesHalf; ++nt) o[nt] = f32x4{0, 0, 0, 0};
    float m_ref = -INFINITY, l_sum = 0.0f;

    // Iteration t: scores of tile t -> exchange -> BARRIER -> softmax, values of tile t ->
    // stage tile t+2 (in registers since iteration t-1) -> request tile t+3 from memory.
    // The barrier orders everything that needs ordering: a wave past it knows that every
    // wave has finished tile t-1 (so its LDS tile, (t+2) mod 3, may be overwritten) and has
    // staged tile t+1 (which it did before its scores of tile t).
    int buf = 0;  // t mod 3
    for (int tile = 0; tile < n_tiles; ++tile) {
        const unsigned int tok_ahead = tile + 4 < n_tiles ? row_token(tile + 4) : 0xffffffffu;
        const lds_ptr<f32x4> xch_mine = xch + (((tile & 1) * kAttWaves + wave) * kWave + lane) * 2;
        const lds_ptr<f32x4> xch_peer = xch + (((tile & 1) * kAttWaves + (wave ^ 4)) * kWave + lane) * 2;

        // ---- scores: this wave's half of the dims, S^T[token][head], two 16-token halves --
        const lds_ptr<uint8_t> krb = kr + buf * kKrBytes + half * (kKStepsHalf * 64);
        const lds_ptr<bf16x8> a0p = (lds_ptr<bf16x8>)(krb + n16 * kKrRowBytes + 16 * g);
        const lds_ptr<bf16x8> a1p = (lds_ptr<bf16x8>)(krb + (16 + n16) * kKrRowBytes + 16 * g);
        f32x4 s0 = {0, 0, 0, 0}, s1 = {0, 0, 0, 0};
        if constexpr (LINEAR) {
            // One scale per token AND per 128 latent dims: each block's dots are folded into the
            // running score with that block's scales before the next block starts; the roped
            // dims (K-steps 16, 17) carry no scale. Which K-steps close a block depends on the
            // half of the dims this wave owns, so the loop is written once per half.
            f32x4 t0 = {0, 0, 0, 0}, t1 = {0, 0, 0, 0};
            auto run = [&](auto half_c) {
                constexpr int HF = decltype(half_c)::value;
#pragma unroll
                for (int j = 0; j < kKStepsHalf; ++j) {
                    const bf16x8 f0 = a0p[j * 4], f1 = a1p[j * 4];
                    s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f0, qh[j], s0, 0, 0, 0);
                    s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f1, qh[j], s1, 0, 0, 0);
                    s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f0, ql[j], s0, 0, 0, 0);
                    s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f1, ql[j], s1, 0, 0, 0);
                    const int ks = HF * kKStepsHalf + j;
                    const int blk = ks < 16 ? ks / 4 : 4;
                    const int blk_next = j + 1 == kKStepsHalf ? -1 : (ks + 1 < 16 ? (ks + 1) / 4 : 4);
                    if (blk_next != blk) {
                        if (blk < 4) {
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                t0[i] += s0[i] * sc4[buf * kTile + 8 * g + i][blk];
                                t1[i] += s1[i] * sc4[buf * kTile + 8 * g + 4 + i][blk];
                            }
                        } else {
                            t0 += s0, t1 += s1;
                        }
                        s0 = f32x4{0, 0, 0, 0}, s1 = f32x4{0, 0, 0, 0};
                    }
                }
            };
            if (half == 0) run(std::integral_constant<int, 0>{});
            else run(std::integral_constant<int, 1>{});
            s0 = t0, s1 = t1;
        }
        // The operand fragments of a block of K-steps are all requested before the first MFMA
        // of the block; left alone the compiler keeps two reads in flight and every pair of
        // MFMAs then waits out a full LDS round trip.
#pragma unroll
        for (int j0 = 0; j0 < (LINEAR ? 0 : kKStepsHalf); j0 += kFragBlock) {
            bf16x8 fa0[kFragBlock], fa1[kFragBlock];
#pragma unroll
            for (int i = 0; i < kFragBlock; ++i) fa0[i] = a0p[(j0 + i) * 4], fa1[i] = a1p[(j0 + i) * 4];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < kFragBlock; ++i) {
                const int j = j0 + i;
                s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa0[i], qh[j], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa1[i], qh[j], s1, 0, 0, 0);
                if (QSPLIT == 2) {
                    s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa0[i], ql[j], s0, 0, 0, 0);
                    s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa1[i], ql[j], s1, 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        xch_mine[0] = s0, xch_mine[1] = s1;
        // what does not depend on the other half of the scores is fetched under the barrier:
        // the first value-side fragments, the tokens' scales and biases
        // value-side operand of column tile nt: for each of the lane's 8 contraction indices
        // (tokens 4g..4g+3 of both 16-token halves) the value of column 16*nt' + n16. One
        // transposing load hands a lane element e of the 8-byte chunk that lane
        // 4e + (n16 >> 2) of its 16-lane row addressed, position n16 & 3 — so lane i
        // addresses token 4g + (i >> 2), columns 16*nt' + 4*(i & 3) .. +3.
        const lds_ptr<uint8_t> vrow = kr + buf * kKrBytes + (4 * g + (n16 >> 2)) * kKrRowBytes +
                                      (half * (kKvl / 2) + 4 * (n16 & 3)) * 2;
        auto vt_frag = [&](int nt) -> bf16x8 {
            typedef short s16x4 __attribute__((ext_vector_type(4)));
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr<s16x4>)(vrow + nt * 32));
            const s16x4 hi =
                __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr<s16x4>)(vrow + 16 * kKrRowBytes + nt * 32));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const s16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            return __builtin_bit_cast(bf16x8, both);
        };
        bf16x8 fb[kValueAhead];
#pragma unroll
        for (int i = 0; i < kValueAhead; ++i) fb[i] = vt_frag(i);
        __builtin_amdgcn_sched_barrier(0);
        const f32x4 sa = *(lds_ptr<f32x4>)(sc + buf * kTile + 8 * g);
        const f32x4 sb = *(lds_ptr<f32x4>)(sc + buf * kTile + 8 * g + 4);
        const f32x4 ba = *(lds_ptr<f32x4>)(sbias + buf * kTile + 8 * g);
        const f32x4 bb = *(lds_ptr<f32x4>)(sbias + buf * kTile + 8 * g + 4);
        __syncthreads();  // both halves of every score are in LDS
        {
            const f32x4 p0 = xch_peer[0], p1 = xch_peer[1];
            s0 += p0, s1 += p1;  // a + b == b + a: the pair works on identical numbers
        }

        // ---- online softmax over the lane's 8 tokens of head n16 --------------------------
        const float scl[8] = {sa.x, sa.y, sa.z, sa.w, sb.x, sb.y, sb.z, sb.w};
        const float bias[8] = {ba.x, ba.y, ba.z, ba.w, bb.x, bb.y, bb.z, bb.w};
        float v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = __builtin_fmaf(s0[i], scl[i], bias[i]);              // -inf where the token is not there
            v[4 + i] = __builtin_fmaf(s1[i], scl[4 + i], bias[4 + i]);
        }
        float tmax = fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7])));
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
            for (int nt = 0; nt < kColTilesHalf; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) o[nt][i] *= c[i];
        }
        const float mu = m_ref == -INFINITY ? 0.0f : m_ref;
        // The value MFMA sees a_t = bf16(p_t * s_t), as hi + lo when PSPLIT == 2. Carried
        // once, the denominator sums a_t / s_t — the weights the numerator really holds — so
        // the result is an exactly normalised average under weights perturbed by one bf16
        // rounding each: the error scales with the spread of the attended rows, not their
        // magnitude, and vanishes when one token holds the whole softmax. Carried as
        // hi + lo the weights are good to 2^-17 and the denominator sums p_t itself.
        bf16x8 p, p_lo;
        bf16x8 p2, p2_lo;  // linear slabs: the weights under the scales of the wave's second column block
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float e = __builtin_amdgcn_exp2f(v[i] - mu);  // not there -> 0
            float x = e * scl[i];
            if constexpr (LINEAR) {  // columns 256*half .. +127 and +128 .. +255 are blocks 2*half, 2*half + 1
                const f32x4 s4 = sc4[buf * kTile + 8 * g + i];
                x = e * (half ? s4[2] : s4[0]);
                const float x2 = e * (half ? s4[3] : s4[1]);
                const __bf16 w2 = (__bf16)x2;
                p2[i] = w2;
                p2_lo[i] = (__bf16)(x2 - (float)w2);
            }
            const __bf16 w = (__bf16)x;
            p[i] = w;
            if (PSPLIT == 2) {
                p_lo[i] = (__bf16)(x - (float)w);
                l_sum += e;
            } else {
                l_sum += (float)w * (scl[i] > 0.0f ? __builtin_amdgcn_rcpf(scl[i]) : 0.0f);
            }
        }

        // ---- values: O[head][col] += P . V over this wave's 256 columns -------------------
#pragma unroll
        for (int n0 = 0; n0 < kColTilesHalf; n0 += kValueAhead) {
            if (n0 > 0) {
#pragma unroll
                for (int i = 0; i < kValueAhead; ++i) fb[i] = vt_frag(n0 + i);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < kValueAhead; ++i) {
                const bool second = LINEAR && n0 + i >= kColTilesHalf / 2;  // known when unrolled
                o[n0 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(second ? p2 : p, fb[i], o[n0 + i], 0, 0, 0);
                if (PSPLIT == 2)
                    o[n0 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(second ? p2_lo : p_lo, fb[i], o[n0 + i], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        // ---- stage tile + 2, request tile + 3, resolve tile + 4 ---------------------------
        // (the request goes out LAST: resolving reads the block table, and the wait that
        // read needs would otherwise also wait for the bytes just requested)
        if (tile + 2 < n_tiles) stage(buf == 0 ? 2 : buf - 1);
        Where next;
        resolve(tile + 4, tok_ahead, next);
        if (tile + 3 < n_tiles) issue_loads(where);
        where = next;
        buf = buf == 2 ? 0 : buf + 1;
    }

    // ---- epilogue -----------------------------------------------------------------------
    l_sum = rows_sum(l_sum);
    // the lane's accumulators are heads 4g+i; their (m, l) live in lanes with n16 == 4g+i
    float l_h[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) l_h[i] = __shfl(l_sum, 4 * g + i, kWave);
    const int head0 = hb * 64 + 16 * hw;
    const int col0 = half * (kKvl / 2) + n16;
    if (!whole) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int head = head0 + 4 * g + i;
            if (head < a.H) {
#pragma unroll
                for (int nt = 0; nt < kColTilesHalf; ++nt) pa[(size_t)head * kKvl + col0 + 16 * nt] = o[nt][i];
            }
        }
        if (half == 0 && g == 0 && head0 + n16 < a.H) {
            pml[(head0 + n16) * 2] = m_ref;
            pml[(head0 + n16) * 2 + 1] = l_sum;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int head = head0 + 4 * g + i;
            const float inv = l_h[i] > 0.0f ? 1.0f / l_h[i] : 0.0f;
            if (head < a.H) {
                float* const dst = a.clat + ((size_t)seq * a.H + head) * kvl;
#pragma unroll
                for (int nt = 0; nt < kColTilesHalf; ++nt)
                    if (!ANY || col0 + 16 * nt < kvl) dst[col0 + 16 * nt] = o[nt][i] * inv;
            }
        }
    }
}

}  // namespace rk
#include "mla_attend_f8.hpp"
namespace rk {

// F8: the contractions run on the 8-bit matrix instructions with QSPLIT / PSPLIT e4m3 terms for
// q / the softmax weights (mla_attend_f8.hpp); else on the bf16 ones.
template <int QSPLIT, int PSPLIT, int MODE, bool ANY, bool F8 = false>
__global__ __launch_bounds__(F8 ? kF8Threads : kAttThreads) void mla_attend_paged_kernel(const AttendArgs a) {
    constexpr int THREADS = F8 ? kF8Threads : kAttThreads;
    constexpr int PER = kDealMaxSeqs / THREADS;  // sequences per thread in the prefix below
    __shared__ int pre[kDealMaxSeqs + 8];  // tiles before each sequence, when dealing
    __shared__ int wave_total[THREADS / kWave];
    constexpr bool SPARSE = MODE == kSparse;
    const int hb = blockIdx.z;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    auto attended = [&](int s) -> int {
        if (MODE == kLinear) return a.k;
        if (SPARSE) return a.n_rows ? max(min(a.n_rows[s], a.k), 0) : a.k;
        return max(min(a.seq_lens[s], a.k), 0);
    };

    // ---- which rows of which sequences this workgroup attends ------------------------------
    // One sequence, all of it, when nothing is dealt. Otherwise the tiles [t_lo, t_hi) of the
    // batch-wide tile sequence: the workgroup walks the sequences that range touches.
    long long t_lo = 0, t_hi = 0;
    int seq = blockIdx.y;
    if (a.n_items > 0) {
        // inclusive prefix of tiles per sequence, PER consecutive sequences per thread
        // (the lengths are read unconditionally, a sequence past the last re-reading the last
        // one: under `s < n_seqs` each read would be a branch with a wait of its own)
        int c[PER], run = 0;
        const int* const lens = MODE == kLinear ? nullptr : (SPARSE ? a.n_rows : a.seq_lens);
        if (lens) {
#pragma unroll
            for (int j = 0; j < PER; ++j) c[j] = lens[min(PER * tid + j, a.n_seqs - 1)];
#pragma unroll
            for (int j = 0; j < PER; ++j) c[j] = max(min(c[j], a.k), 0);
        } else {
#pragma unroll
            for (int j = 0; j < PER; ++j) c[j] = a.k;
        }
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            c[j] = PER * tid + j < a.n_seqs ? (c[j] + kTile - 1) / kTile : 0;
            run += c[j];
        }
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const int up = __shfl_up(run, off, kWave);
            if (lane >= off) run += up;
        }
        if (lane == kWave - 1) wave_total[wave] = run;
        __syncthreads();
        int before = 0;
        for (int w = 0; w < wave; ++w) before += wave_total[w];
        run += before;  // tiles of sequence 0 .. the thread's last one
        if (tid == 0) pre[0] = 0;
#pragma unroll
        for (int j = PER - 1; j >= 0; --j) {
            const int s = PER * tid + j;
            if (s < a.n_seqs) pre[s + 1] = run;
            run -= c[j];
        }
        __syncthreads();
        const long long total = pre[a.n_seqs];
        t_lo = deal_lo(blockIdx.x, a.n_items, total);
        t_hi = deal_lo(blockIdx.x + 1, a.n_items, total);
        if (t_lo >= t_hi) return;
        // the sequence holding tile t_lo: the last one that starts at or before it
        int lo = 0, hi = a.n_seqs;  // pre[lo] <= t_lo < pre[hi]
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (pre[mid] <= t_lo) lo = mid;
            else hi = mid;
        }
        seq = lo;
    }

  for (;; ++seq) {
    int r_begin = 0, r_end;
    bool whole = true;                 // the whole sequence is this part: write clat directly
    float *pa = a.part_acc, *pml = a.part_ml;  // else this part's partial record
    if (a.n_items > 0) {
        if (t_lo >= t_hi || seq >= a.n_seqs) break;
        const long long p0 = pre[seq], p1 = pre[seq + 1];
        const long long e = t_hi < p1 ? t_hi : p1;
        if (e <= t_lo) continue;  // a sequence with nothing to attend
        r_begin = (int)(t_lo - p0) * kTile;
        r_end = min(attended(seq), (int)(e - p0) * kTile);
        whole = t_lo == p0 && e == p1;
        const size_t rec = (size_t)blockIdx.x + seq;  // unique: both only grow along the walk
        pa = a.part_acc + rec * a.H * kKvl;
        pml = a.part_ml + rec * a.H * 2;
        t_lo = e;
        __syncthreads();  // the previous part is done with the LDS tiles and the prefix reads above
    } else {
        r_end = attended(seq);
        if (r_end <= 0) {
            // a sequence with nothing to attend gets zeros, like the reference's `l > 0 ? 1/l : 0`
            const int kvl = ANY ? a.kvl : kKvl;
            for (int i = tid; i < 64 * kvl; i += THREADS) {
                const int h = hb * 64 + i / kvl;
                if (h < a.H) a.clat[((size_t)seq * a.H + h) * kvl + (i % kvl)] = 0.0f;
            }
            return;
        }
    }
    if constexpr (F8) attend_part_f8<QSPLIT, PSPLIT, MODE == kSparse, MODE == kSparse ? 64 : 128>(a, seq, hb, r_begin, r_end, whole, pa, pml);
    else attend_part<QSPLIT, PSPLIT, MODE, ANY>(a, seq, hb, r_begin, r_end, whole, pa, pml);
    if (a.n_items == 0) break;
  }  // parts of this workgroup
}

// Dealt plan: clat[seq][head] = sum_r w_r acc_r / sum_r w_r l_r over the sequence's partial
// records, w_r = 2^(m_r - max m), in ascending work-item order (the reference's combine,
// crates/backend/kernels/attn.hip:235-277, in base 2). A sequence that one work item covered
// whole was written by it directly; one with nothing to attend gets zeros.
__global__ __launch_bounds__(128) void mla_attend_combine_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml, const int* __restrict__ seq_lens,
    const int* __restrict__ n_rows, int sparse, int k, int n_seqs, int n_items, int H, int kvl,
    float* __restrict__ clat) {
    __shared__ long long s_sum[3][2];  // per wave: tiles before seq, tiles of seq .. end
    const int head = blockIdx.x, seq = blockIdx.y;
    // tiles before this sequence, of this sequence, and in all
    long long before = 0, mine = 0, total = 0;
    for (int s = threadIdx.x; s < n_seqs; s += 128) {
        int n = (sparse || !seq_lens) ? (n_rows ? min(n_rows[s], k) : k) : min(seq_lens[s], k);
        n = max(n, 0);
        const long long t = (n + kTile - 1) / kTile;
        total += t;
        if (s < seq) before += t;
        if (s == seq) mine = t;
    }
    for (int off = 32; off > 0; off >>= 1) {
        before += __shfl_xor(before, off, kWave);
        mine += __shfl_xor(mine, off, kWave);
        total += __shfl_xor(total, off, kWave);
    }
    if ((threadIdx.x & 63) == 0) {
        s_sum[0][threadIdx.x >> 6] = before;
        s_sum[1][threadIdx.x >> 6] = mine;
        s_sum[2][threadIdx.x >> 6] = total;
    }
    __syncthreads();
    before = s_sum[0][0] + s_sum[0][1], mine = s_sum[1][0] + s_sum[1][1], total = s_sum[2][0] + s_sum[2][1];
    if (4 * (int)threadIdx.x >= kvl) return;  // the records are 512 wide whatever the cache's width
    float4* const dst = reinterpret_cast<float4*>(clat + ((size_t)seq * H + head) * kvl) + threadIdx.x;
    if (mine == 0) {
        *dst = float4{0, 0, 0, 0};
        return;
    }
    const int first = deal_item_of(before, n_items, total);
    const int last = deal_item_of(before + mine - 1, n_items, total);
    if (first == last) return;  // one work item had the whole sequence and wrote it
    // Records are fetched eight at a time, every load of a batch issued before the first use
    // (a record past the last re-reads the last and is left out): one round trip per batch
    // instead of one per record. The sums run in ascending record order as before.
    constexpr int kBatch = 8;
    float m_g = -INFINITY;
    for (int b0 = first; b0 <= last; b0 += kBatch) {
        float m_r[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u)
            m_r[u] = part_ml[((size_t)(min(b0 + u, last) + seq) * H + head) * 2];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) m_g = fmaxf(m_g, m_r[u]);
    }
    float4 sum = {0, 0, 0, 0};
    float l_g = 0.0f;
    if (m_g != -INFINITY) {
        for (int b0 = first; b0 <= last; b0 += kBatch) {
            float m_r[kBatch], l_r[kBatch];
            float4 v[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const size_t rec = (size_t)min(b0 + u, last) + seq;
                m_r[u] = part_ml[(rec * H + head) * 2];
                l_r[u] = part_ml[(rec * H + head) * 2 + 1];
                v[u] = reinterpret_cast<const float4*>(part_acc + (rec * H + head) * kKvl)[threadIdx.x];
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                if (b0 + u > last || m_r[u] == -INFINITY) continue;
                const float w = exp2f(m_r[u] - m_g);
                l_g += l_r[u] * w;
                sum.x += v[u].x * w, sum.y += v[u].y * w, sum.z += v[u].z * w, sum.w += v[u].w * w;
            }
        }
    }
    const float inv = l_g > 0.0f ? 1.0f / l_g : 0.0f;
    *dst = float4{sum.x * inv, sum.y * inv, sum.z * inv, sum.w * inv};
}

// What both launchers share once the arguments are in place: the attention kernel of the right
// mode, then the merge of the partial records when the plan has any.
template <int MODE>
static int attend_launch(const AttendArgs& a, const AttendPlan& plan, int n_seqs, int max_rows, bool any,
                         int precise, const int* seq_lens, const int* n_rows, bool listed, hipStream_t st) {
    const dim3 grid(plan.n_items ? (unsigned)plan.n_items : 1u, plan.n_items ? 1u : (unsigned)n_seqs,
                    (unsigned)((a.H + 63) / 64));
    (void)hipGetLastError();
    // A cache of other widths than 512 + 64 always runs in the parity mode.
    if (any || MODE == kLinear)
        hipLaunchKernelGGL((mla_attend_paged_kernel<2, 2, MODE, true>), grid, dim3(kAttThreads), 0, st, a);
    else if constexpr (MODE != kLinear) {
        if (precise == 3)
            hipLaunchKernelGGL((mla_attend_paged_kernel<2, 2, MODE == kSparse ? kSparse : kDense, false, true>), grid,
                               dim3(kF8Threads), 0, st, a);
        else if (precise == 4)
            hipLaunchKernelGGL((mla_attend_paged_kernel<3, 2, MODE == kSparse ? kSparse : kDense, false, true>), grid,
                               dim3(kF8Threads), 0, st, a);
        else if (precise >= 2)
            hipLaunchKernelGGL((mla_attend_paged_kernel<2, 2, MODE, false>), grid, dim3(kAttThreads), 0, st, a);
        else if (precise == 1)
            hipLaunchKernelGGL((mla_attend_paged_kernel<2, 1, MODE, false>), grid, dim3(kAttThreads), 0, st, a);
        else
            hipLaunchKernelGGL((mla_attend_paged_kernel<1, 1, MODE, false>), grid, dim3(kAttThreads), 0, st, a);
    }
    const int rc = launch_status();
    if (rc != 0 || plan.n_splits <= 1) return rc;
    hipLaunchKernelGGL(mla_attend_combine_kernel, dim3((unsigned)a.H, (unsigned)n_seqs), dim3(128), 0, st,
                       a.part_acc, a.part_ml, seq_lens, n_rows, listed ? 1 : 0, max_rows, n_seqs, plan.n_items,
                       a.H, a.kvl, a.clat);
    return launch_status();
}

}  // namespace rk


extern "C" size_t rivoli_mla_attend_paged_scratch_floats(int n_seqs, int H, int max_rows) {
    if (n_seqs <= 0 || H <= 0 || max_rows <= 0) return 0;
    const rk::AttendPlan p = rk::attend_plan(n_seqs, H, max_rows);
    return (size_t)p.n_records * H * (rk::kKvl + 2);
}

extern "C" int rivoli_mla_attend_paged(const float* qabs, const float* qrope,
                                       const unsigned char* pool, const int* block_table,
                                       const int* seq_lens, const unsigned int* rows,
                                       const int* n_rows, int n_seqs, int H, int max_rows,
                                       int max_blocks_per_seq, int kvl, int rope, int page_tokens,
                                       int n_pages, float scale, int precise, float* clat,
                                       float* partial, unsigned int* bad_rows, void* stream) {
    using namespace rk;
    if (!qabs || !qrope || !pool || !block_table || !clat) return 1001;
    if (!rows && !seq_lens) return 1001;
    if (n_seqs <= 0 || H <= 0 || max_rows <= 0 || max_blocks_per_seq <= 0 || kvl <= 0 || rope <= 0 ||
        page_tokens <= 0 || n_pages <= 0)
        return 1001;
    if (n_seqs > 65535 || H > 64 * 65535) return 1002;
    // the latent width as the reference's launcher has it (crates/backend/kernels/attn.hip:
    // 284-293: a multiple of 128 up to 512); the rope codes fill at most two 32-wide steps
    if (kvl > kKvl || (kvl % 128) != 0 || rope > kRopeW || (rope % 8) != 0) return 1004;
    if (!aligned16(qabs) || !aligned16(qrope) || !aligned16(pool) || !aligned16(clat) || !aligned16(partial))
        return 1004;
    const AttendPlan plan = attend_plan(n_seqs, H, max_rows);
    if (plan.n_splits > 1 && !partial) return 1001;
    AttendArgs a = {};
    a.qabs = qabs, a.qrope = qrope, a.pool = pool, a.block_table = block_table;
    a.seq_lens = seq_lens, a.rows = rows, a.n_rows = n_rows, a.k = max_rows;
    a.H = H, a.max_blocks = max_blocks_per_seq, a.page_tokens = page_tokens, a.n_pages = n_pages;
    a.kvl = kvl, a.rope = rope, a.row_w = kvl + rope;
    a.page_shift = (page_tokens & (page_tokens - 1)) == 0 ? __builtin_ctz((unsigned)page_tokens) : -1;
    a.page_bytes = (size_t)page_tokens * a.row_w + (size_t)page_tokens * 4;
    a.qscale = scale * kLog2e;
    a.n_seqs = n_seqs, a.n_items = plan.n_items;
    a.clat = clat, a.bad_rows = bad_rows;
    a.part_acc = plan.n_items ? partial : nullptr;
    a.part_ml = plan.n_items ? partial + (size_t)plan.n_records * H * kKvl : nullptr;
    const bool any = kvl != kKvl || rope != kRopeW;
    hipStream_t st = (hipStream_t)stream;
    if (rows) return attend_launch<kSparse>(a, plan, n_seqs, max_rows, any, precise, seq_lens, n_rows, true, st);
    if (a.page_shift >= 0 && page_tokens >= kTile)
        return attend_launch<kDensePaged>(a, plan, n_seqs, max_rows, any, precise, seq_lens, n_rows, false, st);
    return attend_launch<kDense>(a, plan, n_seqs, max_rows, any, precise, seq_lens, n_rows, false, st);
}

// ---------------------------------------------------------------------------------------------
// The reference's single-token launcher over its linear slabs, signature and guards kept
// (crates/backend/kernels/attn.hip:95-103,279-308): latent e4m3 codes with one f32 scale per
// 128 values, the roped key as bf16, token = rows ? rows[j] : j for j < nr. The same kernel as
// above with a third address mode: the caller's scratch (sized by the reference's rule,
// 16 * H * (kvl + 2) floats) holds as many 512-wide partial records as fit it.
// ---------------------------------------------------------------------------------------------
namespace rk {
constexpr int kRefMaxSplits = 16;  // what rivoli_mla_attend_scratch_floats prices (attn.hip:66,98-103)

// Shapes the tile kernel does not take (a roped key wider than 64, slabs that are not 8-byte
// aligned): a wave per head walks the rows one at a time, lanes over the dims, online softmax.
__global__ __launch_bounds__(256) void mla_attend_rowwise_kernel(
    const float* __restrict__ qabs, const float* __restrict__ qrope, const uint8_t* __restrict__ lc8,
    const float* __restrict__ lscale, const uint16_t* __restrict__ rc, const unsigned int* __restrict__ rows,
    int H, int nr, int kvl, int rope, int n_blocks, float qscale, float* __restrict__ clat) {
    const int lane = threadIdx.x & (kWave - 1);
    const int head = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (head >= H) return;
    const float* qa = qabs + (size_t)head * kvl;
    const float* qr = qrope + (size_t)head * rope;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};  // columns lane, lane + 64, ... (kvl <= 512)
    float m = -INFINITY, l = 0.0f;
    for (int j = 0; j < nr; ++j) {
        const size_t t = rows ? rows[j] : (unsigned)j;
        float lat[8], dot = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int i = lane + c * kWave;
            lat[c] = 0.0f;
            if (i < kvl)
                lat[c] = __builtin_amdgcn_cvt_pk_f32_fp8((uint32_t)lc8[t * kvl + i], false)[0] * lscale[t * n_blocks + i / 128];
            if (i < kvl) dot += qa[i] * lat[c];
        }
        for (int i = lane; i < rope; i += kWave) dot += qr[i] * bf16_lo_to_f32((uint32_t)rc[t * rope + i]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, kWave);
        const float sv = dot * qscale;  // log2 units
        const float m_new = fmaxf(m, sv);
        const float corr = exp2f(m - m_new), pw = exp2f(sv - m_new);
        l = l * corr + pw;
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[c] = acc[c] * corr + pw * lat[c];
        m = m_new;
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int i = lane + c * kWave;
        if (i < kvl) clat[(size_t)head * kvl + i] = acc[c] * inv;
    }
}
}  // namespace rk

extern "C" size_t rivoli_mla_attend_scratch_floats(int H, int kvl) {
    if (H <= 0 || kvl <= 0) return 0;
    return (size_t)rk::kRefMaxSplits * (size_t)H * ((size_t)kvl + 2);
}

extern "C" int rivoli_mla_attend(const float* qabs, const float* qrope, const unsigned char* Lc8,
                                 const float* Lscale, const unsigned short* Rc,
                                 const unsigned int* rows, int H, int nr, int kvl, int rope,
                                 int n_blocks, float scale, float* clat, float* partial) {
    using namespace rk;
    if (H <= 0 || nr <= 0 || kvl <= 0 || rope <= 0 || n_blocks <= 0) return 1001;
    if (((size_t)kvl + rope) * 16 * sizeof(float) > 65536) return 1002;  // the reference's LDS bound
    if (kvl > kKvl || kvl % 128) return 1004;
    if (!qabs || !qrope || !Lc8 || !Lscale || !Rc || !clat) return 1001;
    (void)hipGetLastError();
    if (rope > kRopeW || (reinterpret_cast<uintptr_t>(Lc8) & 7u) != 0 || H > 64 * 65535) {
        hipLaunchKernelGGL(mla_attend_rowwise_kernel, dim3((unsigned)((H + 3) / 4)), dim3(256), 0, nullptr, qabs,
                           qrope, Lc8, Lscale, Rc, rows, H, nr, kvl, rope, n_blocks, scale * kLog2e, clat);
        return launch_status();
    }
    // split plan: as the batched launcher's for one sequence, capped by what the scratch holds
    AttendPlan plan = attend_plan(1, H, nr);
    const int fit = (int)((size_t)kRefMaxSplits * ((size_t)kvl + 2) / (kKvl + 2)) - 1;  // records - 1
    if (plan.n_splits > fit) plan.n_splits = fit;
    if (!partial || plan.n_splits < 2) plan.n_splits = 1;
    plan.n_items = plan.n_splits > 1 ? plan.n_splits : 0;
    plan.n_records = plan.n_items ? plan.n_items + 1 : 0;
    AttendArgs a = {};
    a.qabs = qabs, a.qrope = qrope, a.rows = rows, a.k = nr, a.H = H;
    a.lc8 = Lc8, a.lscale = Lscale, a.rc = Rc, a.n_blocks = n_blocks;
    a.kvl = kvl, a.rope = rope, a.row_w = kvl + rope;
    a.max_blocks = 1, a.page_tokens = 1, a.n_pages = 1, a.page_shift = 0, a.page_bytes = 0;
    a.qscale = scale * kLog2e;
    a.n_seqs = 1, a.n_items = plan.n_items;
    a.clat = clat;
    a.part_acc = plan.n_items ? partial : nullptr;
    a.part_ml = plan.n_items ? partial + (size_t)plan.n_records * H * kKvl : nullptr;
    return attend_launch<kLinear>(a, plan, 1, nr, true, 2, nullptr, nullptr, rows != nullptr, nullptr);
}
