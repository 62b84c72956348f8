// MLA decode attention over the paged fp8 cache on gfx950's 8-bit matrix instructions
// (v_mfma_scale_f32_16x16x128_f8f6f4), included by mla_attend.hip.
//
// The cache rows ARE e4m3 codes, so they go from memory into LDS (global_load_lds: no registers
// on the way) and from LDS into the matrix cores untouched: no conversion, half the LDS bytes of
// the bf16 kernel, a quarter of its matrix instructions. What is not e4m3 is carried as a short
// sum of e4m3 terms under power-of-two block scales (the instruction's own E8M0 scale operands):
//   q      = sum_t 2^(e - 4t) * q_t,  e from the largest |q| of the (head, 128-dim step)
//   p * s  = sum_t 2^(e - 4t) * p_t,  e from the largest weight of the (head, tile)
// Each term adds four significant bits (term t quantizes what the terms before it left over): two
// terms are bf16-class; three of q and two of the weights stay inside the reference's bar.
//
// Mapping: a 256-thread workgroup — one wave per SIMD, each with the whole register file — owns
// 64 heads and a run of rows; wave w owns heads 16 w .. +15 and all 512 output columns (128
// accumulators). The q terms live in the accumulation half of the register file, which the
// matrix instructions read directly. Two buffers of raw code rows in LDS; tiles are 128 tokens
// for dense rows, 64 for listed rows (whose calls are a tile or two long; there a third q term
// lives in LDS). Per tile a wave
//   requests the next tile into the other buffer (dense rows: two requests behind each of the
//     first score units; else all of them first);
//   scores: S^T[token][head] = rows x q, row blocks of 16 tokens x 5 K-steps (128 dims; the
//     rope's 64 fill half a step) x TQ terms, A = 32 contiguous bytes of a row per lane;
//   online softmax in base 2 with a lazily moved reference, the weights to two e4m3 terms in
//     registers: a lane's weights per term are exactly its share of the next operand;
//   values: O[head][col] += P V on the same tile, read through the transposing byte load
//     (ds_read_b64_tr_b8). 128-token tiles: the contraction's K = 128 is the tile's tokens, one
//     matrix instruction per weight term. 64-token tiles: K is the 64 tokens once per term —
//     bytes 0..15 of a lane's weight operand hold the first term of its 16 tokens, bytes 16..31
//     the second (the instruction takes K block b's scale from lane 16 b + row, so lane groups
//     2 and 3 carry the finer scale) and the value operand repeats its 16 bytes;
//   waits for its part of the next tile and meets the other waves at the one barrier of the step.
// Operand fragments are requested one unit ahead of the matrix instructions that use them.
// The file must be compiled with -mllvm -amdgpu-mfma-vgpr-form (the build does): the kernel's
// register budget assumes the output tiles in ordinary registers and the q terms in the
// accumulation registers, and without the switch the compiler moves all 128 accumulators
// between the two halves every tile.
#pragma once

namespace rk {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x2 __attribute__((ext_vector_type(2)));

constexpr int kF8Threads = 256;              // four waves, one per SIMD, each with the full register file
constexpr int kF8Waves = kF8Threads / kWave;
constexpr int kF8Bufs = 2;
constexpr int kF8RowBytes = 592;             // 576 codes + 16 of padding
constexpr int kF8ZeroBytes = 64;
constexpr int kF8Steps = 5;                  // K-steps of the scores: four of 128 latent dims, one for the rope
constexpr int kF8ColTiles = kKvl / 16;       // 32 output column tiles per wave
constexpr int kF8RowGranules = kF8RowBytes / 16;  // 37: 36 of codes, one of padding
// What follows from the tile size. TILE = 128 (dense rows): the value contraction's K is the
// tile's 128 tokens, one matrix instruction per weight term, and every q term lives in
// registers. TILE = 64 (listed rows, whose calls are a tile or two long): K is the 64 tokens
// once per weight term, the value operand repeats its 16 bytes, a third q term lives in LDS.
template <int TILE>
struct F8Shape {
    static_assert(TILE == 64 || TILE == 128, "the value contraction is written for these two");
    static constexpr int kTileBytes = TILE * kF8RowBytes;
    static constexpr int kRowBlocks = TILE / 16;        // score row blocks per tile
    static constexpr int kWaveRows = TILE / kF8Waves;   // rows of a tile one wave brings in
    static constexpr int kRequests = (kWaveRows * kF8RowGranules + kWave - 1) / kWave;
    static constexpr int kTable = TILE == 128 ? 512 : kTableLds;  // block-table entries staged in LDS
    static constexpr int kQTermsInRegs(int tq) { return TILE == 128 ? tq : (tq > 2 ? 2 : tq); }
    // q terms that do not live in registers: the block's 64 heads, rows padded like the tiles'
    static constexpr int kQBytes(int tq) { return tq > kQTermsInRegs(tq) ? (tq - kQTermsInRegs(tq)) * 64 * kF8RowBytes : 16; }
    static constexpr int kSmemBytes =
        kF8Bufs * kTileBytes + kF8ZeroBytes + 3 * kF8Bufs * TILE * 4 + kTable * 4;
};
static_assert(F8Shape<64>::kSmemBytes + F8Shape<64>::kQBytes(3) + (1024 + 8 + 8) * 4 <= 160 * 1024 &&
              F8Shape<128>::kSmemBytes + F8Shape<128>::kQBytes(3) + (1024 + 8 + 8) * 4 <= 160 * 1024,
              "one workgroup per CU must fit the 160 KiB of LDS");
constexpr int kWaitLds0 = 0xC07F;           // s_waitcnt lgkmcnt(0), the other counters left alone
constexpr int kScaleOne = 0x7f7f7f7f;        // E8M0 1.0 in every byte

// 2^e as a float, e in [-126, 127].
__device__ __forceinline__ float pow2i(int e) { return __uint_as_float((uint32_t)(e + 127) << 23); }
// The block exponent for a largest magnitude `amax`: values / 2^e land below 256 (e4m3 holds 448).
__device__ __forceinline__ int block_exp(float amax) {
    const int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 127 - 7;
    return amax > 0.0f ? max(min(e, 100), -100) : 0;  // (a tile of vanishing weights keeps a scale whose finer terms still exist)
}
// x[0..3] (already divided by the block scale) -> four e4m3 codes of x * 16^T, the T-th term of
// a sum whose terms are 16 times finer each; val[i] = what the codes stand for (their values /
// 16^T) and x -= val. Terms past the first use the scaled conversions (the instruction divides
// by a power of two on the way in and multiplies on the way out: no multiplies of our own).
typedef short i16x2 __attribute__((ext_vector_type(2)));
template <int T>
__device__ __forceinline__ uint32_t e4m3x4_term(float (&x)[4], float (&val)[4]) {
    uint32_t u;
    if constexpr (T == 0) {
        int w = 0;
        w = __builtin_amdgcn_cvt_pk_fp8_f32(x[0], x[1], w, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(x[2], x[3], w, true);
        const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(w, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
        val[0] = lo[0], val[1] = lo[1], val[2] = hi[0], val[3] = hi[1];
        u = (uint32_t)w;
    } else {
        constexpr float kFiner = T == 1 ? 0.0625f : T == 2 ? 0.00390625f : 0.000244140625f;
        static_assert(T <= 3, "up to four terms");
        i16x2 w = {0, 0};
        w = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(w, x[0], x[1], kFiner, false);
        w = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(w, x[2], x[3], kFiner, true);
        u = ((uint32_t)(uint16_t)w[1] << 16) | (uint16_t)w[0];
        const auto lo = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(u, kFiner, false), hi = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(u, kFiner, true);
        val[0] = lo[0], val[1] = lo[1], val[2] = hi[0], val[3] = hi[1];
    }
    x[0] -= val[0], x[1] -= val[1], x[2] -= val[2], x[3] -= val[3];
    return u;
}

// Sixteen bytes per lane from memory straight into LDS: lane L's land at dst + 16 L (dst is
// wave-uniform). Issued as text: through the builtin the compiler makes every later LDS read wait
// for the transfer, whichever buffer it reads. The caller waits (vmcnt) before the data is used.
__device__ __forceinline__ void dma16(const uint8_t* src, lds_ptr<uint8_t> dst) {
    const uint32_t base = (uint32_t)(uintptr_t)dst;
    uint32_t keep;  // m0 is the instruction's LDS base; the compiler's own value of it is put back
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(src), "s"(base)
                 : "memory");
}

// The same from a wave-uniform address plus a 32-bit offset per lane (the instruction's scalar
// base form: no 64-bit add, and offsets kept across a loop cost one register each). The base is
// made scalar here: an operand that reaches the statement through a loop-carried value may
// otherwise sit in vector registers, which the assembler accepts and the instruction misreads.
__device__ __forceinline__ void dma16_from(const uint8_t* base_uniform, uint32_t off, lds_ptr<uint8_t> dst) {
    const uint32_t lds_base = (uint32_t)(uintptr_t)dst;
    const uint64_t b = (uint64_t)(uintptr_t)base_uniform;
    const uint64_t sb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(b >> 32)) << 32) |
                        (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    uint32_t keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(off), "s"(sb), "s"(lds_base)
                 : "memory");
}

template <int TQ, int TP, bool SPARSE, int TILE>
__device__ __forceinline__ void attend_part_f8(const AttendArgs& a, int seq, int hb, int r_begin, int r_end,
                                               bool whole, float* pa, float* pml) {
    using Sh = F8Shape<TILE>;
    constexpr int kTileBytes = Sh::kTileBytes, kRowBlocks = Sh::kRowBlocks, kWaveRows = Sh::kWaveRows;
    constexpr int kRequests = Sh::kRequests, kTable = Sh::kTable;
    __shared__ __attribute__((aligned(16))) uint8_t smem8[Sh::kSmemBytes + Sh::kQBytes(TQ)];
    const lds_ptr<uint8_t> tiles = (lds_ptr<uint8_t>)smem8;               // [2][TILE] rows of codes
    const lds_ptr<uint8_t> zeros = tiles + kF8Bufs * kTileBytes;
    const lds_ptr<float> sc = (lds_ptr<float>)(zeros + kF8ZeroBytes);     // [2][TILE] token scales (0 = not there)
    const lds_ptr<float> sbias = sc + kF8Bufs * TILE;                        // [2][TILE] log2 scale, or -inf
    const lds_ptr<float> rsc = sbias + kF8Bufs * TILE;                       // [2][TILE] 1 / scale (0 = not there)
    const lds_ptr<int> tbl = (lds_ptr<int>)(rsc + kF8Bufs * TILE);
    const lds_ptr<uint8_t> qlds = (lds_ptr<uint8_t>)(tbl + kTable);  // [TQ - TQR][64 heads] rows of q codes

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // = which 16 heads of the block
    const int g = lane >> 4, n16 = lane & 15;
    const int n_tiles = (r_end - r_begin + TILE - 1) / TILE;

    // ---- listed rows: a tile's list entries are asked for a tile ahead (the first two tiles'
    // here, in front of everything), so that their way from memory is not waited for in front of
    // the tile's requests. Lanes 0..kWaveRows-1 hold one entry each; the address always exists.
    const unsigned int* const rows_g = SPARSE ? a.rows + (size_t)seq * a.k : nullptr;
    auto list_entry = [&](int t) -> unsigned int {
        if constexpr (!SPARSE) return 0u;
        const int pos = r_begin + t * TILE + kWaveRows * wave + (lane & (kWaveRows - 1));
        return rows_g[min(pos, r_end - 1)];
    };
    unsigned int entry_now = list_entry(0), entry_next = list_entry(1);

    // ---- block-table slice, zero area -------------------------------------------------------
    const int* const table_g = a.block_table + (size_t)seq * a.max_blocks;
    const int tbl_first = SPARSE ? 0 : r_begin / a.page_tokens;
    const int tbl_last = SPARSE ? a.max_blocks - 1 : min(a.max_blocks - 1, (r_end - 1) / a.page_tokens);
    const int tbl_count = min(kTable, tbl_last - tbl_first + 1);
    for (int i = tid; i < tbl_count; i += kF8Threads) tbl[i] = table_g[tbl_first + i];
    if (tid < kF8ZeroBytes / 4) ((lds_ptr<int>)zeros)[tid] = 0;

    // ---- this wave's 16 query heads as e4m3 terms, for the whole kernel ----------------------
    // step s < 4: latent dims 128 s .. +127. Step 4, the rope, has 64 dims for a K of 128: its
    // operand holds the rope's FIRST TWO TERMS side by side, term 0 in lane groups 0 and 1, term 1
    // in lane groups 2 and 3 (qt[0][4]; the key rows' rope bytes are read by both pairs of lane
    // groups), so one matrix instruction does what two half-empty ones would. An element of
    // lane group g, byte b belongs to K block (g >> 1) + 2 (b / 16) and block k takes its scale
    // from lane group k: term 0 sits in blocks 0 and 2, term 1 in blocks 1 and 3, hence a scale
    // register that alternates between the two terms' scales by lane group (qscale_rope). A
    // third term keeps the half-empty form (zeros in lane groups 2 and 3).
    constexpr int TQR = Sh::kQTermsInRegs(TQ);  // terms in (accumulation) registers; one past them lives in LDS
    static_assert(TQR >= 2, "the rope step pairs the first two terms");
    i32x8 qt[TQR][kF8Steps];  // qt[1][4] is not used
    int qscale_lo[TQ], qscale_hi[TQ];  // E8M0 scales: bytes 0..3 = steps 0..3, byte 0 of _hi = step 4
    int qscale_rope = kScaleOne;
    {
        const int head = hb * 64 + 16 * wave + n16;
        const bool live = head < a.H;
        const size_t qrow = (size_t)seq * a.H + (live ? head : 0);
#pragma unroll
        for (int t = 0; t < TQ; ++t) qscale_lo[t] = qscale_hi[t] = kScaleOne;
        // every load of q is requested before the first is used, from addresses that always
        // exist (a head past H reads head 0, lane groups 2 and 3 re-read the rope's halves) and
        // dropped afterwards: a load under a condition is a branch with a wait of its own
        float4 raw[kF8Steps][8];
#pragma unroll
        for (int s = 0; s < kF8Steps; ++s) {
            const float* src =
                s == 4 ? a.qrope + qrow * kRopeW + 32 * (g & 1) : a.qabs + qrow * kKvl + 128 * s + 32 * g;
#pragma unroll
            for (int c = 0; c < 8; ++c) raw[s][c] = reinterpret_cast<const float4*>(src)[c];
        }
#pragma unroll
        for (int s = 0; s < kF8Steps; ++s) {
            // x = q * qscale / 2^e in one multiply per value (2^e is exact, so the product rounds
            // as the two multiplies would); a head past H keeps its loaded values times zero
            // (the rope step: lane groups 2, 3 hold what 0, 1 hold)
            float x[32];
            const float keep = live ? a.qscale : 0.0f;
            float amax = 0.0f;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const float4 v = raw[s][c];
                x[4 * c] = v.x, x[4 * c + 1] = v.y, x[4 * c + 2] = v.z, x[4 * c + 3] = v.w;
            }
#pragma unroll
            for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(x[i]));
            amax = rows_max(amax * keep);  // over the head's four lanes: one scale per (head, step)
            const int e = block_exp(amax);
            const float inv = keep * pow2i(-e);
#pragma unroll
            for (int i = 0; i < 32; ++i) x[i] *= inv;
            uint32_t first_term[8];  // the rope step: term 0's codes, until term 1's join them
#pragma unroll
            for (int t = 0; t < TQ; ++t) {
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    float y[4] = {x[4 * c], x[4 * c + 1], x[4 * c + 2], x[4 * c + 3]}, val[4];
                    uint32_t w4 = t == 0 ? e4m3x4_term<0>(y, val) : t == 1 ? e4m3x4_term<1>(y, val) : e4m3x4_term<2>(y, val);
                    if (s == 4 && t == 0) first_term[c] = w4;
                    if (s == 4 && t == 1) w4 = g < 2 ? first_term[c] : w4;
                    if (s == 4 && t >= 2 && t < TQR) w4 = g < 2 ? w4 : 0u;  // half-empty: zeros in lane groups 2 and 3
                    if (t < TQR && !(s == 4 && t == 0)) {
                        int qa;
                        asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(qa) : "v"(w4));
                        qt[s == 4 && t == 1 ? 0 : t][s][c] = qa;
                    } else if (t >= TQR && (s < 4 || g < 2))
                        *(lds_ptr<uint32_t>)(qlds + ((t - TQR) * 64 + 16 * wave + n16) * kF8RowBytes + 128 * s + 32 * g + 4 * c) = w4;
                    // what is left over, for the next term
                    x[4 * c] = y[0], x[4 * c + 1] = y[1], x[4 * c + 2] = y[2], x[4 * c + 3] = y[3];
                }
                const int byte = max(e - 4 * t + 127, 1);
                if (s < 4) qscale_lo[t] = (qscale_lo[t] & ~(0xff << (8 * s))) | (byte << (8 * s));
                else qscale_hi[t] = (qscale_hi[t] & ~0xff) | byte;
                if (s == 4 && t < 2 && (g & 1) == t) qscale_rope = (qscale_rope & ~0xff) | byte;
            }
        }
    }
    __syncthreads();  // table slice and zero area visible

    auto table_at = [&](int blk) -> int {
        const int rel = blk - tbl_first;
        return (rel >= 0 && rel < tbl_count) ? tbl[rel] : table_g[blk];
    };

    // ---- where the wave's rows of a tile are: lanes 0..kWaveRows-1 resolve one each -------------
    constexpr unsigned long long kNone = ~0ull;
    auto resolve = [&](int t, unsigned int entry, unsigned long long& code_off, unsigned long long& scale_off) {
        code_off = kNone, scale_off = 0;
        const int pos = r_begin + t * TILE + kWaveRows * wave + lane;
        if (lane >= kWaveRows || t >= n_tiles || pos >= r_end) return;
        const unsigned int tok = SPARSE ? entry : (unsigned)pos;
        unsigned int blk, off;
        if (a.page_shift >= 0) blk = tok >> a.page_shift, off = tok & (unsigned)(a.page_tokens - 1);
        else blk = tok / (unsigned)a.page_tokens, off = tok - blk * (unsigned)a.page_tokens;
        const int page = blk < (unsigned)a.max_blocks ? table_at((int)blk) : -1;
        if ((unsigned)page < (unsigned)a.n_pages) {
            const unsigned long long pbase = (unsigned long long)page * a.page_bytes;
            code_off = pbase + (unsigned long long)off * kRowW;
            scale_off = pbase + (unsigned long long)a.page_tokens * kRowW + (unsigned long long)off * 4;
        } else if (a.bad_rows && hb == 0) {
            atomicAdd(a.bad_rows, 1u);
        }
    };
    // A tile goes from memory straight into LDS, 16 bytes per lane, a request's lanes filling
    // consecutive LDS. The wave's rows of 37 granules (36 of codes + the padding one) are one
    // consecutive range of the tile. A row that is not there is zero-filled by hand: its codes
    // must be finite, they meet a zero weight and a -inf bias, never a NaN.
    float next_scale = 0.0f;  // lanes 0..kWaveRows-1: the scale of the row this lane resolved
    // Dense fast path: the wave's rows of a tile are consecutive rows of one page (tiles start
    // on multiples of 32 tokens and the page holds a multiple of the wave's share), so lane L of
    // request i fills granule 64 i + L = row (64 i + L) / 37, granule (64 i + L) % 37 of the row,
    // from byte goff[i] past the first row: no lookups, one request per 1 KiB.
    int goff[kRequests];
#pragma unroll
    for (int i = 0; i < kRequests; ++i) {
        const int gi = min(kWave * i + lane, kWaveRows * kF8RowGranules - 1);
        const int row = gi / kF8RowGranules, c = min(gi - row * kF8RowGranules, kRowW / 16 - 1);
        goff[i] = row * kRowW + 16 * c;  // (the padding granule repeats the one before it)
    }
    const bool pages_hold_runs = !SPARSE && a.page_shift >= (TILE == 128 ? 5 : 4);
    // Request i of such a run, from `run` (the first of the wave's rows in its page).
    auto request_of_run = [&](const uint8_t* run, lds_ptr<uint8_t> dst_tile, int i) {
        if (kWave * (i + 1) <= kWaveRows * kF8RowGranules || lane < kWaveRows * kF8RowGranules - kWave * i)
            dma16_from(run, (uint32_t)goff[i], dst_tile + (kWaveRows * wave) * kF8RowBytes + 1024 * i);
    };
    // Tile t on its way into dst_tile. Returns the run's address when the tile is one and
    // `spread` leaves the requests to the caller (who issues them between the score units: a
    // little faster than one burst), nullptr when everything was requested here.
    auto request_tile = [&](int t, unsigned int entry, lds_ptr<uint8_t> dst_tile, bool spread) -> const uint8_t* {
        const lds_ptr<uint8_t> dst_w = dst_tile + (kWaveRows * wave) * kF8RowBytes;
        if (pages_hold_runs) {
            const int pos0 = r_begin + t * TILE + kWaveRows * wave;
            if (pos0 + kWaveRows <= r_end) {
                const int blk = pos0 >> a.page_shift, off = pos0 & (a.page_tokens - 1);
                const int page = blk < a.max_blocks ? __builtin_amdgcn_readfirstlane(table_at(blk)) : -1;
                if ((unsigned)page < (unsigned)a.n_pages) {
                    const uint8_t* const pg = a.pool + (size_t)page * a.page_bytes;
                    const uint8_t* const src = pg + (size_t)off * kRowW;
                    next_scale = 0.0f;
                    if (lane < kWaveRows)
                        next_scale = reinterpret_cast<const float*>(pg + (size_t)a.page_tokens * kRowW)[off + lane];
                    if (spread) return src;
#pragma unroll
                    for (int i = 0; i < kRequests; ++i) request_of_run(src, dst_tile, i);
                    return nullptr;
                }
            }
        }
        // General path: a request per row, 37 lanes of 16 bytes from the row's own address (held by
        // the lane that resolved it, handed over as a scalar: one page per request, no address
        // arithmetic per lane). A row that is not there is zero-filled by hand.
        unsigned long long code_off, scale_off;
        resolve(t, entry, code_off, scale_off);
        next_scale = 0.0f;
        if (code_off != kNone) next_scale = *reinterpret_cast<const float*>(a.pool + scale_off);
        const uint32_t granule = (uint32_t)min(lane, kRowW / 16 - 1) * 16u;  // (the padding granule repeats the one before it)
#pragma unroll
        for (int r = 0; r < kWaveRows; ++r) {
            const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)code_off, r);
            const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(code_off >> 32), r);
            const lds_ptr<uint8_t> dst_r = dst_w + r * kF8RowBytes;
            if ((lo & hi) != 0xffffffffu) {
                if (lane < kF8RowGranules)
                    dma16_from(a.pool + (((unsigned long long)hi << 32) | lo), granule, dst_r);
            } else if (lane < kF8RowGranules) {
                *(lds_ptr<u32x4>)(dst_r + 16 * lane) = u32x4{0, 0, 0, 0};
            }
        }
        return nullptr;
    };
    auto publish_scales = [&](int buf) {  // the scales of the tile request_tile last asked for
        if (lane < kWaveRows) {
            const bool ok = next_scale > 0.0f;  // a token that is not there has scale 0
            sc[buf * TILE + kWaveRows * wave + lane] = ok ? next_scale : 0.0f;
            // the bias added to a token's scores: log2 of its scale (its weights then carry the
            // scale the value contraction needs), -inf for a token that is not there
            sbias[buf * TILE + kWaveRows * wave + lane] = ok ? __builtin_amdgcn_logf(next_scale) : -INFINITY;
            // the denominator divides every held weight by its token's scale: the reciprocal is
            // taken once per token here, not once per (token, head) in the softmax
            rsc[buf * TILE + kWaveRows * wave + lane] = ok ? __builtin_amdgcn_rcpf(next_scale) : 0.0f;
        }
    };

    // ---- per-lane LDS addresses ---------------------------------------------------------------
    // scores: row 16 mb + n16, this lane's 32 bytes of K-step s; the rope step's upper half
    // (lane groups 2 and 3) reads zeros
    const int a_row = n16 * kF8RowBytes + 32 * g;
    const int a_rope = n16 * kF8RowBytes + kKvl + 32 * (g & 1);  // both pairs of lane groups read the rope
    const bool rope_zero = g >= 2;  // a third q term's rope fragment
    const int q_row = (16 * wave + n16) * kF8RowBytes + 32 * g;
    // values: transposing load r hands this lane bytes 8 r .. 8 r + 7 of its operand = the
    // tokens 16 (2 r + e / 4) + 4 g + e % 4, e = 0..7, of column 16 nt + n16; source lane pair e
    // addresses token e's row, its two lanes the two 8-byte halves of the 16 columns.
    constexpr int kReads = TILE / 32;  // transposing loads per column tile: 16 tokens each... 8 bytes a lane
    int v_off[kReads];
    {
        const int e = n16 >> 1;
#pragma unroll
        for (int r = 0; r < kReads; ++r)
            v_off[r] = (16 * (2 * r + (e >> 2)) + 4 * g + (e & 3)) * kF8RowBytes + 8 * (n16 & 1);
    }

    f32x4 o[kF8ColTiles];
#pragma unroll
    for (int nt = 0; nt < kF8ColTiles; ++nt) o[nt] = f32x4{0, 0, 0, 0};
    float m_ref = -INFINITY, l_sum = 0.0f;

    // prologue: tile 0 into LDS
    request_tile(0, entry_now, tiles, false);
    publish_scales(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    for (int t = 0; t < n_tiles; ++t) {
        const int buf = t & 1;
        const lds_ptr<uint8_t> tile = tiles + buf * kTileBytes, next = tiles + (buf ^ 1) * kTileBytes;
        const lds_ptr<float> sc_t = sc + buf * TILE, sbias_t = sbias + buf * TILE, rsc_t = rsc + buf * TILE;

        // ---- scores: S^T[token][head] over the five K-steps ---------------------------------
        // A unit's operand fragments are requested while the matrix instructions of the unit
        // before run; the scheduling fences keep that order.
        f32x4 acc[kRowBlocks];
#pragma unroll
        for (int mb = 0; mb < kRowBlocks; ++mb) acc[mb] = f32x4{0, 0, 0, 0};
        i32x8 af[2][2], qf[2][TQ > TQR ? TQ - TQR : 1];
        f32x4 s4[kRowBlocks], r4[kRowBlocks], b4[kRowBlocks];  // token scales, their reciprocals, biases
        auto read32 = [&](lds_ptr<uint8_t> src) -> i32x8 {
            const u32x4 lo4 = *(lds_ptr<u32x4>)(src), hi4 = *(lds_ptr<u32x4>)(src + 16);
            return i32x8{(int)lo4.x, (int)lo4.y, (int)lo4.z, (int)lo4.w, (int)hi4.x, (int)hi4.y, (int)hi4.z, (int)hi4.w};
        };
        // unit u: K-step u / UPS, row blocks 2 (u % UPS) + {0, 1}; a step's q fragments (those
        // that live in LDS) come with its first unit
        constexpr int UPS = kRowBlocks / 2, kUnits = UPS * kF8Steps;
        auto load_unit = [&](int u) {
            const int s = u / UPS;
            const bool z = s == 4 && rope_zero;
#pragma unroll
            for (int j = 0; j < 2; ++j)
                af[u & 1][j] = read32(tile + (2 * (u % UPS) + j) * 16 * kF8RowBytes + (s == 4 ? a_rope : a_row + 128 * s));
            if ((u % UPS) == 0) {
#pragma unroll
                for (int tq = 0; tq < TQ - TQR; ++tq)
                    qf[s & 1][tq] = read32(z ? zeros : qlds + tq * 64 * kF8RowBytes + q_row + 128 * s);
            }
        };
        load_unit(0);
        __builtin_amdgcn_sched_barrier(0);
        // tile t + 1 starts on its way into the other buffer (which held tile t - 1: every wave
        // left it before the barrier that ended the previous iteration); the address arithmetic of
        // its requests runs while the first fragments above come out of LDS
        constexpr int kPerUnit = 2;  // requests behind each of the first units
        static_assert(kUnits * kPerUnit >= kRequests, "the units take every request");
        const uint8_t* const run = t + 1 < n_tiles ? request_tile(t + 1, entry_next, next, true) : nullptr;
        if constexpr (SPARSE) entry_next = list_entry(t + 2);
#pragma unroll
        for (int u = 0; u < kUnits; ++u) {
            __builtin_amdgcn_s_waitcnt(kWaitLds0);  // this unit's fragments are in
            __builtin_amdgcn_sched_barrier(0);
            if (u + 1 < kUnits) {
                load_unit(u + 1);
            } else {
                // under the last unit's matrix instructions: what the softmax reads first
#pragma unroll
                for (int mb = 0; mb < kRowBlocks; ++mb) {
                    s4[mb] = *(lds_ptr<f32x4>)(sc_t + 16 * mb + 4 * g);
                    b4[mb] = *(lds_ptr<f32x4>)(sbias_t + 16 * mb + 4 * g);
                    if (TILE == 64) r4[mb] = *(lds_ptr<f32x4>)(rsc_t + 16 * mb + 4 * g);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            const int s = u / UPS;
#pragma unroll
            for (int tq = 0; tq < TQ; ++tq)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if (s == 4 && tq == 1) continue;  // the rope's second term rode with the first
                    const i32x8 fa = af[u & 1][j], fq = tq < TQR ? qt[tq < TQR ? tq : 0][s] : qf[s & 1][tq < TQR ? 0 : tq - TQR];
                    const int mb = 2 * (u % UPS) + j;
                    if (s == 0)
                        acc[mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa, fq, acc[mb], 0, 0, 0, kScaleOne, 0, qscale_lo[tq]);
                    else if (s == 1)
                        acc[mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa, fq, acc[mb], 0, 0, 0, kScaleOne, 1, qscale_lo[tq]);
                    else if (s == 2)
                        acc[mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa, fq, acc[mb], 0, 0, 0, kScaleOne, 2, qscale_lo[tq]);
                    else if (s == 3)
                        acc[mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa, fq, acc[mb], 0, 0, 0, kScaleOne, 3, qscale_lo[tq]);
                    else
                        acc[mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa, fq, acc[mb], 0, 0, 0, kScaleOne, 0, tq == 0 ? qscale_rope : qscale_hi[tq]);
                }
            if (kPerUnit * u < kRequests) {
                // (the sums are used here so that the unit's matrix instructions stay in front
                // of the branch: the compiler would sink them past it)
#pragma unroll
                for (int j = 0; j < 2; ++j) asm volatile("" : "+v"(acc[2 * (u % UPS) + j]));
                if (run) {
#pragma unroll
                    for (int i = kPerUnit * u; i < kPerUnit * (u + 1) && i < kRequests; ++i) request_of_run(run, next, i);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        // the value contraction's first operands are requested now: they do not depend on the
        // softmax, whose arithmetic then hides their way out of LDS
        static_assert(TP == 2, "two terms fill the value contraction's K exactly");
        constexpr int CU = TILE == 128 ? 4 : 8;  // column tiles per unit (eight matrix instructions)
        i32x8 vf[2][CU];
        auto load_cols = [&](int n0, i32x8 (&f)[CU]) {
#pragma unroll
            for (int j = 0; j < CU; ++j) {
                i32x2 r[kReads];
#pragma unroll
                for (int k = 0; k < kReads; ++k)
                    r[k] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_ptr<i32x2>)(tile + v_off[k] + 16 * (n0 + j)));
                if constexpr (TILE == 128) f[j] = i32x8{r[0][0], r[0][1], r[1][0], r[1][1], r[2][0], r[2][1], r[3][0], r[3][1]};
                else f[j] = i32x8{r[0][0], r[0][1], r[1][0], r[1][1], r[0][0], r[0][1], r[1][0], r[1][1]};
            }
        };
        load_cols(0, vf[0]);
        __builtin_amdgcn_sched_barrier(0);

        // ---- online softmax over the lane's tokens of head n16: tokens 16 mb + 4 g + i ---------
        float tmax = -INFINITY;
#pragma unroll
        for (int mb = 0; mb < kRowBlocks; ++mb) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[mb][i] = __builtin_fmaf(acc[mb][i], s4[mb][i], b4[mb][i]);  // -inf where the token is not there
                tmax = fmaxf(tmax, acc[mb][i]);
            }
        }
        if constexpr (TILE == 128) {  // (asked for here: the registers of the scales above are free again)
#pragma unroll
            for (int mb = 0; mb < kRowBlocks; ++mb) r4[mb] = *(lds_ptr<f32x4>)(rsc_t + 16 * mb + 4 * g);
        }
        tmax = rows_max(tmax);
        const bool grow = tmax > m_ref + kLazyRescale;  // false while everything is masked
        if (__builtin_amdgcn_ballot_w64(grow) != 0) {
            const float corr = grow ? __builtin_amdgcn_exp2f(m_ref - tmax) : 1.0f;
            if (grow) m_ref = tmax;
            l_sum *= corr;
            float c[4];  // the lane's accumulators are heads 4g+i; corr lives in lanes n16 == head
#pragma unroll
            for (int i = 0; i < 4; ++i) c[i] = __shfl(corr, 4 * g + i, kWave);
#pragma unroll
            for (int nt = 0; nt < kF8ColTiles; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) o[nt][i] *= c[i];
        }
        const float mu = m_ref == -INFINITY ? 0.0f : m_ref;
        // weights w_t = 2^(v_t - mu) * s_t = 2^(v'_t - mu) with v' = v + log2 s_t (the published
        // bias carries log2 s_t, so the token scale costs nothing here), as TP e4m3 terms under
        // one scale 2^pe per (head, tile). The largest weight of the head's tokens is
        // 2^(tmax - mu), exp2 being monotonic: no second maximum is taken. The terms are cut from
        // y = w / 2^pe, computed as one exponential.
        const int pe = block_exp(__builtin_amdgcn_exp2f(tmax - mu));
        const float shift = mu + (float)pe, unit = pow2i(pe);
        // TILE = 64: one operand, bytes 0..15 the first term of the lane's 16 tokens, 16..31 the
        // second (the instruction takes K block b's scale from lane 16 b + row: blocks 0, 1 are
        // the first term of lane groups 0,1 / 2,3, blocks 2, 3 the second term, 16 times finer).
        // TILE = 128: an operand per term, byte b the token 16 (b / 4) + 4 g + b % 4.
        constexpr int kOperands = TILE == 128 ? TP : 1;
        i32x8 pt[kOperands];
        int pscale[kOperands];
#pragma unroll
        for (int k = 0; k < kOperands; ++k)
            pscale[k] = (int)((uint32_t)max(pe - 4 * (TILE == 128 ? k : (g >> 1)) + 127, 1) * 0x01010101u);
        float l_tile = 0.0f;  // in units of 2^pe
#pragma unroll
        for (int mb = 0; mb < kRowBlocks; ++mb) {
            float y[4], val[4], back[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) y[i] = __builtin_amdgcn_exp2f(acc[mb][i] - shift);  // not there -> 0
            const int first = (int)e4m3x4_term<0>(y, val);
            const int second = (int)e4m3x4_term<1>(y, back);
            if constexpr (TILE == 128) pt[0][mb] = first, pt[1][mb] = second;
            else pt[0][mb] = first, pt[0][4 + mb] = second;
            // The denominator sums the weights the numerator really holds (w_t less the last
            // residual), over the token scale: the result is an exactly normalised average under
            // weights perturbed by 2^-8 each.
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float held = val[i] + back[i];  // 0 for a token that is not there
                l_tile = __builtin_fmaf(held, r4[mb][i], l_tile);
            }
        }
        l_sum = __builtin_fmaf(l_tile, unit, l_sum);

        // ---- values: O[head][col] += P . V over all 512 columns (the first unit's operands were
        // requested before the softmax) --------------------------------------------------------
#pragma unroll
        for (int n0 = 0; n0 < kF8ColTiles; n0 += CU) {
            __builtin_amdgcn_s_waitcnt(kWaitLds0);
            __builtin_amdgcn_sched_barrier(0);
            if (n0 + CU < kF8ColTiles) load_cols(n0 + CU, vf[((n0 / CU) + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < CU; ++j)
#pragma unroll
                for (int k = 0; k < kOperands; ++k)
                    o[n0 + j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(pt[k], vf[(n0 / CU) & 1][j], o[n0 + j], 0, 0, 0, pscale[k], 0, kScaleOne);
            // TILE = 128: the products stay here, under the next unit's operands on their way out
            // of LDS. Left free, the compiler sinks them all below the end of the tile (nothing
            // reads the sums before the next tile) and has to hold every unit's operands at once.
            if constexpr (TILE == 128) {
#pragma unroll
                for (int j = 0; j < CU; ++j) asm volatile("" : "+v"(o[n0 + j]));
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        if (t + 1 < n_tiles) publish_scales(buf ^ 1);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's part of tile t + 1 has landed
        __syncthreads();  // tile t + 1 is in LDS; every wave is done with tile t
    }

    // ---- epilogue ---------------------------------------------------------------------------
    l_sum = rows_sum(l_sum);
    float l_h[4];  // the lane's accumulators are heads 4g+i; their (m, l) live in lanes with n16 == 4g+i
#pragma unroll
    for (int i = 0; i < 4; ++i) l_h[i] = __shfl(l_sum, 4 * g + i, kWave);
    const int head0 = hb * 64 + 16 * wave;
    if (!whole) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int head = head0 + 4 * g + i;
            if (head < a.H) {
#pragma unroll
                for (int nt = 0; nt < kF8ColTiles; ++nt) pa[(size_t)head * kKvl + n16 + 16 * nt] = o[nt][i];
            }
        }
        if (g == 0 && head0 + n16 < a.H) {
            pml[(head0 + n16) * 2] = m_ref;
            pml[(head0 + n16) * 2 + 1] = l_sum;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int head = head0 + 4 * g + i;
            const float inv = l_h[i] > 0.0f ? 1.0f / l_h[i] : 0.0f;
            if (head < a.H) {
                float* const dst = a.clat + ((size_t)seq * a.H + head) * kKvl;
#pragma unroll
                for (int nt = 0; nt < kF8ColTiles; ++nt) dst[n16 + 16 * nt] = o[nt][i] * inv;
            }
        }
    }
}

}  // namespace rk
