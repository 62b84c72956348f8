// DSA lightning-indexer scores and the paged indexer key cache.
//
//   scores[t] = sum over active heads h of  w[h] * wscale * max((q_h . k_t) * dscale, 0)
//
// (crates/backend/kernels/indexer.hip:60-93; host restatement crates/engine/tests/
// indexer_kernel.rs:238-250). The key cache holds one hd-wide bf16 row per token; here it is
// addressed by slot (slot = page * page_tokens + offset), so a block table pages it exactly
// like the fp8 latent cache, and `index_append` becomes a many-token scatter.
//
// The reference runs one workgroup per token with a serial dot per head. Here the dots of 32
// tokens x 32 heads are one 32x32 MFMA tile: A = the query heads (rows), B = the tokens' key
// rows (columns), K = hd. The keys are bf16 already and enter the matrix core untouched; the
// f32 query is split into a bf16 head and a bf16 remainder (q = hi + lo to 2^-18 relative),
// two MFMAs per K-step, so the products carry ~17 bits of the query — inside the 1e-5
// (relative to the largest score) bar the reference sets for this kernel, which a single
// bf16 rounding of q would miss. With heads as the tile's ROWS a lane holds 16 heads of one
// token, so ReLU, the head weights and the sum over heads are register arithmetic plus one
// cross-half shuffle; nothing goes through LDS after the query is staged.
// A workgroup stages its query once and walks 2048 tokens (4 waves x 16 blocks of 32). The
// kernel reads hd*2 bytes per token and is bound by that stream, not by the matrix cores.
// Launch-only; see include/rivoli_kvcache.h for the contract of every entry point.
#include "topk_common.hpp"

namespace rk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kScoreThreads = 256;
constexpr int kScoreWaves = kScoreThreads / kWave;
constexpr int kScoreMaxHeads = 64;   // active heads, padded to a multiple of 32
constexpr int kScoreMaxHd = 128;     // head dimension, a multiple of 16
constexpr int kScoreBlocks = 16;     // 32-token blocks per wave
constexpr int kScoreTokensPerGroup = kScoreWaves * kScoreBlocks * 32;
constexpr int kScoreRowPad = 8;      // bf16 of padding per staged query row

// RB = 32-head row blocks (1 or 2). HD = the head dimension at compile time (128, the shipped
// one) or 0 for the runtime value: with it the chunk-to-row divisions are shifts (with a runtime
// width they were two thirds of the kernel's vector instructions), the K loop has a constant
// trip count, and the head halves of the query's operand fragments (the same for every block
// of tokens) are read from LDS once and kept in registers instead of being re-read per block:
// two of every five LDS reads of the runtime form. Keeping the remainder halves as well leaves
// room for one wave per SIMD and is no faster; neither is a second block in flight per wave.
template <int RB, int HD>
__global__ __launch_bounds__(kScoreThreads) void index_score_kernel(
    const float* __restrict__ q, const float* __restrict__ w,
    const uint16_t* __restrict__ kpool, const int* __restrict__ block_table,
    const int* __restrict__ nts, const unsigned int* __restrict__ heads, int max_blocks_per_seq,
    int stride, int nt_all, int nh, int nact, int hd_rt, int page_tokens, int n_pages, float wscale,
    float dscale, float* __restrict__ scores, uint32_t* __restrict__ topk_ws, size_t ws_stride) {
    const int hd = HD ? HD : hd_rt;
    __shared__ __attribute__((aligned(16))) uint16_t s_qh[RB * 32][kScoreMaxHd + kScoreRowPad];
    __shared__ __attribute__((aligned(16))) uint16_t s_ql[RB * 32][kScoreMaxHd + kScoreRowPad];
    __shared__ float s_w[RB * 32];
    __shared__ __attribute__((aligned(16)))
    uint16_t s_k[kScoreWaves][32][kScoreMaxHd + kScoreRowPad];  // one key tile per wave
    // With a top-k workspace: the histogram of this workgroup's scores by the top 12 bits of
    // their selection key, two 16-bit counters per word (a workgroup scores 2048 tokens).
    __shared__ uint32_t s_hist[kTopBins / 2];
    static_assert(kScoreTokensPerGroup < 65536, "16-bit histogram counters");

    const int qi = blockIdx.y;
    const int nt = nts ? min(nts[qi], nt_all) : nt_all;
    const int t0 = (int)blockIdx.x * kScoreTokensPerGroup;
    if (t0 >= nt) return;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (topk_ws)
        for (int i = tid; i < kTopBins / 2; i += kScoreThreads) s_hist[i] = 0u;

    // ---- stage the active heads: q = hi + lo in bf16, and the per-head weight ----
    // eight consecutive query values per step: two 16-byte loads in, two 16-byte LDS stores out
    const int cpr = hd >> 3;
    for (int c = tid; c < RB * 32 * cpr; c += kScoreThreads) {
        const int a = c / cpr, d = (c - a * cpr) * 8;
        float val[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        if (a < nact) {
            const int h = heads ? (int)heads[a] : a;
            if ((unsigned)h < (unsigned)nh) {
                const float4* src =
                    reinterpret_cast<const float4*>(q + ((size_t)qi * nh + h) * hd + d);
                const float4 v0 = src[0], v1 = src[1];
                val[0] = v0.x, val[1] = v0.y, val[2] = v0.z, val[3] = v0.w;
                val[4] = v1.x, val[5] = v1.y, val[6] = v1.z, val[7] = v1.w;
            }
        }
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            hi[i] = pack_bf16x2(val[2 * i], val[2 * i + 1]);
            lo[i] = pack_bf16x2(val[2 * i] - bf16_lo_to_f32(hi[i]),
                                val[2 * i + 1] - bf16_hi_to_f32(hi[i]));
        }
        *reinterpret_cast<u32x4*>(&s_qh[a][d]) = u32x4{hi[0], hi[1], hi[2], hi[3]};
        *reinterpret_cast<u32x4*>(&s_ql[a][d]) = u32x4{lo[0], lo[1], lo[2], lo[3]};
    }
    if (tid < RB * 32) {
        float wv = 0.0f;  // padding heads weigh nothing
        if (tid < nact) {
            const int h = heads ? (int)heads[tid] : tid;
            if ((unsigned)h < (unsigned)nh) wv = w[(size_t)qi * nh + h] * wscale;  // a head id
        }                                              // outside [0, nh) contributes nothing
        s_w[tid] = wv;
    }
    __syncthreads();

    const int col = lane & 31;        // the lane's token within a block / head within a row block
    const int khalf = (lane >> 5) * 8;  // which 8 of each 16-wide K-step this lane carries
    const int ksteps = hd >> 4;
    constexpr int KS = HD ? HD / 16 : 1;
    bf16x8 qh[RB][KS];
    if constexpr (HD != 0) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int s = 0; s < KS; ++s)
                qh[rb][s] = *reinterpret_cast<const bf16x8*>(&s_qh[rb * 32 + col][khalf + 16 * s]);
    }
    // accumulator element v of a lane is head row 8*(v/4) + 4*(lane/32) + v%4, token `col`:
    // the lane's 16 (32) head weights are fixed for the whole kernel, so they sit in registers
    float wv[RB][16];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int v = 0; v < 16; ++v)
            wv[rb][v] = s_w[rb * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)];

    // A block's 32 key rows are one contiguous run (consecutive tokens of one page, or of the
    // linear cache), so the wave fetches it with fully coalesced 16-byte loads, parks it in its
    // own LDS tile and reads it back in the matrix core's operand layout. Fetching each lane's
    // operand straight from memory instead touches 32 different rows per instruction and was
    // measured ~1.6x slower. The next block's fetch is issued before this block's MFMAs.
    constexpr int kChunks = 32 * kScoreMaxHd / 8 / kWave;  // 16-byte chunks per lane per block
    uint16_t(*tile)[kScoreMaxHd + kScoreRowPad] = s_k[wave];
    const int cprk = hd >> 3;                               // 16-byte chunks per key row
    // rows_ok < 0: the block's page is outside the pool, -rows_ok of its tokens are in range
    auto block_base = [&](int tb, int& rows_ok) -> const uint16_t* {
        rows_ok = min(32, nt - tb);
        size_t slot = (size_t)tb;
        if (block_table) {
            const int page = block_table[(size_t)qi * max_blocks_per_seq + tb / page_tokens];
            if ((unsigned)page >= (unsigned)n_pages) {
                rows_ok = -rows_ok;  // nothing of this block is readable
                return kpool;
            }
            slot = (size_t)page * page_tokens + (size_t)(tb % page_tokens);
        }
        return kpool + slot * hd;
    };
    auto fetch = [&](const uint16_t* base, int rows_ok, u32x4 (&raw)[kChunks]) {
#pragma unroll
        for (int j = 0; j < kChunks; ++j) {
            const int c = lane + j * kWave;
            raw[j] = (c < rows_ok * cprk) ? reinterpret_cast<const u32x4*>(base)[c]
                                          : u32x4{0, 0, 0, 0};
        }
    };

    int tb = t0 + wave * 32, rows_ok = 0;
    u32x4 raw[kChunks];
    if (tb < nt) fetch(block_base(tb, rows_ok), rows_ok, raw);
    for (int it = 0; it < kScoreBlocks && tb < nt; ++it) {
        // park this block; the wave's LDS operations execute in order, the fences only keep
        // the compiler from moving the reads above the writes (and the next writes above them)
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
        for (int j = 0; j < kChunks; ++j) {
            const int c = lane + j * kWave;
            if (c < 32 * cprk) {
                const int r = c / cprk, cc = c - r * cprk;
                *reinterpret_cast<u32x4*>(&tile[r][cc * 8]) = raw[j];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        const int token = tb + col;
        const bool valid = col < rows_ok;
        const int tb_next = tb + kScoreWaves * 32;
        int rows_next = 0;
        if (it + 1 < kScoreBlocks && tb_next < nt) fetch(block_base(tb_next, rows_next), rows_next, raw);

        f32x16 acc[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[rb][v] = 0.0f;
#pragma unroll
        for (int s = 0; s < kScoreMaxHd / 16; ++s) {
            if (s < ksteps) {
                const bf16x8 kb = *reinterpret_cast<const bf16x8*>(&tile[col][khalf + 16 * s]);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    bf16x8 ah;
                    if constexpr (HD != 0)
                        ah = qh[rb][s];
                    else
                        ah = *reinterpret_cast<const bf16x8*>(&s_qh[rb * 32 + col][khalf + 16 * s]);
                    const bf16x8 al =
                        *reinterpret_cast<const bf16x8*>(&s_ql[rb * 32 + col][khalf + 16 * s]);
                    acc[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, kb, acc[rb], 0, 0, 0);
                    acc[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, kb, acc[rb], 0, 0, 0);
                }
            }
        }
        float sum = 0.0f;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int v = 0; v < 16; ++v) sum += wv[rb][v] * fmaxf(acc[rb][v] * dscale, 0.0f);
        sum += __shfl_xor(sum, 32, kWave);
        // With the selection's histogram: a token of an unreadable page gets the score -inf and
        // is counted like any other, so that the histogram and the scores the selection reads
        // next agree. Without it such a token is left unwritten, as the plain form documents.
        const bool lost = topk_ws && col < -rows_ok;
        if (lost) sum = -INFINITY;
        if (lane < 32 && (valid || lost)) {
            scores[(size_t)qi * stride + token] = sum;
            if (topk_ws) {
                const uint32_t bin = topk_key(sum) >> kLowBits;
                atomicAdd(&s_hist[bin >> 1], 1u << ((bin & 1u) * 16u));
            }
        }
        tb = tb_next;
        rows_ok = rows_next;
    }
    if (!topk_ws) return;
    // the selection's first launch, done here: one global atomic per non-empty bin
    __syncthreads();
    uint32_t* wq = topk_ws + (size_t)qi * ws_stride;
    for (int i = tid; i < kTopBins / 2; i += kScoreThreads) {
        const uint32_t c = s_hist[i];
        if (c & 0xffffu) atomicAdd(&wq[2 * i], c & 0xffffu);
        if (c >> 16) atomicAdd(&wq[2 * i + 1], c >> 16);
    }
}

// Shapes outside the matrix-core kernel's limits (more than 64 active heads, a head dimension
// above 128 or not a multiple of 16): plain f32 arithmetic, any shape the reference's launcher
// accepts (crates/backend/kernels/indexer.hip:283-289). A wave owns a token: its key row sits
// in registers (lane L holds dims L, L + 64, ...), every active head is one coalesced pass over
// the query row (from LDS when the active heads fit 64 KiB, else from memory), a butterfly sum
// and the ReLU-weighted accumulate. A workgroup of four waves walks 64 tokens.
constexpr int kPlainTokensPerGroup = 64;
constexpr int kPlainMaxRegs = 8;  // key dims held per lane before the row is re-read per head
__global__ __launch_bounds__(kScoreThreads) void index_score_plain_kernel(
    const float* __restrict__ q, const float* __restrict__ w,
    const uint16_t* __restrict__ kpool, const int* __restrict__ block_table,
    const int* __restrict__ nts, const unsigned int* __restrict__ heads, int max_blocks_per_seq,
    int stride, int nt_all, int nh, int nact, int hd, int page_tokens, int n_pages, float wscale,
    float dscale, float* __restrict__ scores, uint32_t* __restrict__ topk_ws, size_t ws_stride,
    int q_in_lds) {
    extern __shared__ float s_q[];  // [nact][hd] when q_in_lds
    const int qi = blockIdx.y;
    const int nt = nts ? min(nts[qi], nt_all) : nt_all;
    const int t0 = (int)blockIdx.x * kPlainTokensPerGroup;
    if (t0 >= nt) return;
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    auto head_of = [&](int a) -> int {
        const int h = heads ? (int)heads[a] : a;
        return (unsigned)h < (unsigned)nh ? h : -1;  // a head id outside [0, nh) contributes nothing
    };
    if (q_in_lds) {
        for (int i = tid; i < nact * hd; i += kScoreThreads) {
            const int a = i / hd, h = head_of(a);
            s_q[i] = h >= 0 ? q[((size_t)qi * nh + h) * hd + (i - a * hd)] : 0.0f;
        }
        __syncthreads();
    }
    const bool in_regs = hd <= kPlainMaxRegs * kWave;
    for (int t = t0 + wave; t < min(t0 + kPlainTokensPerGroup, nt); t += kScoreWaves) {
        size_t slot = (size_t)t;
        if (block_table) {
            const int page = block_table[(size_t)qi * max_blocks_per_seq + t / page_tokens];
            if ((unsigned)page >= (unsigned)n_pages) {
                // not readable: not written — except with the selection's histogram, where the
                // token scores -inf and is counted, so that histogram and scores agree
                if (topk_ws && lane == 0) {
                    scores[(size_t)qi * stride + t] = -INFINITY;
                    atomicAdd(&topk_ws[(size_t)qi * ws_stride + (topk_key(-INFINITY) >> kLowBits)], 1u);
                }
                continue;
            }
            slot = (size_t)page * page_tokens + (size_t)(t % page_tokens);
        }
        const uint16_t* krow = kpool + slot * hd;
        float kreg[kPlainMaxRegs];
#pragma unroll
        for (int j = 0; j < kPlainMaxRegs; ++j) {
            const int d = lane + j * kWave;
            kreg[j] = (in_regs && d < hd) ? bf16_lo_to_f32((uint32_t)krow[d]) : 0.0f;
        }
        float total = 0.0f;
        for (int a = 0; a < nact; ++a) {
            const int h = head_of(a);
            if (h < 0) continue;
            const float* qrow = q_in_lds ? s_q + (size_t)a * hd : q + ((size_t)qi * nh + h) * hd;
            float dot = 0.0f;
            if (in_regs) {
#pragma unroll
                for (int j = 0; j < kPlainMaxRegs; ++j) {
                    const int d = lane + j * kWave;
                    if (d < hd) dot += qrow[d] * kreg[j];
                }
            } else {
                for (int d = lane; d < hd; d += kWave) dot += qrow[d] * bf16_lo_to_f32((uint32_t)krow[d]);
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, kWave);
            total += w[(size_t)qi * nh + h] * wscale * fmaxf(dot * dscale, 0.0f);
        }
        if (lane == 0) {
            scores[(size_t)qi * stride + t] = total;
            if (topk_ws) atomicAdd(&topk_ws[(size_t)qi * ws_stride + (topk_key(total) >> kLowBits)], 1u);
        }
    }
}

// kpool[slot*hd + i] = bf16(k[t*hd + i]); 8 elements per thread.
__global__ __launch_bounds__(256) void index_append_paged_kernel(
    const float* __restrict__ k, const int* __restrict__ slot_mapping,
    uint16_t* __restrict__ kpool, int n_tokens, int hd, long long n_slots,
    unsigned int* __restrict__ bad_slots) {
    const int per_row = hd >> 3;
    const long long g = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= (long long)n_tokens * per_row) return;
    const int t = (int)(g / per_row), c = (int)(g - (long long)t * per_row);
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    if ((long long)slot >= n_slots) {
        if (c == 0 && bad_slots) atomicAdd(bad_slots, 1u);
        return;
    }
    const float* src = k + (size_t)t * hd + c * 8;
    u32x4 out;
    out.x = pack_bf16x2(src[0], src[1]);
    out.y = pack_bf16x2(src[2], src[3]);
    out.z = pack_bf16x2(src[4], src[5]);
    out.w = pack_bf16x2(src[6], src[7]);
    *reinterpret_cast<u32x4*>(kpool + (size_t)slot * hd + c * 8) = out;
}

static int index_score_launch(const float* q, const float* w, const unsigned short* kpool,
                              const int* block_table, const int* nts, const unsigned int* heads,
                              int n_queries, int max_blocks_per_seq, int stride, int nt, int nh,
                              int nact, int hd, int page_tokens, int n_pages, float wscale,
                              float dscale, float* scores, void* topk_workspace,
                              hipStream_t stream) {
    if (!q || !w || !kpool || !scores) return 1001;
    if (n_queries <= 0 || nt <= 0 || nh <= 0 || nact <= 0 || nact > nh || hd <= 0) return 1001;
    if (block_table && (max_blocks_per_seq <= 0 || page_tokens <= 0 || n_pages <= 0)) return 1001;
    if (stride < nt || n_queries > 65535) return 1002;
    {   // what the reference's launcher refuses (crates/backend/kernels/indexer.hip:283-289)
        int bd = 32;
        while (bd < nact) bd <<= 1;
        if (bd > 1024 || ((size_t)hd + bd) * sizeof(float) > 65536) return 1002;
    }
    const bool plain = nact > kScoreMaxHeads || hd > kScoreMaxHd || (hd % 16) != 0 ||
                       (block_table && (page_tokens % 32) != 0) || !aligned16(q) || !aligned16(kpool);
    // every scored token needs an entry in its query's block-table row
    if (block_table && (long long)nt > (long long)max_blocks_per_seq * page_tokens) return 1002;
    // the histogram is only wanted where the selection of this shape runs split over the chip
    if (topk_workspace && !aligned16(topk_workspace)) return 1004;
    uint32_t* ws = topk_runs_split(n_queries, nt) ? (uint32_t*)topk_workspace : nullptr;
    const size_t ws_stride = topk_ws_words(topk_segments(nt));
    dim3 grid((unsigned)((nt + kScoreTokensPerGroup - 1) / kScoreTokensPerGroup),
              (unsigned)n_queries);
    (void)hipGetLastError();
    if (plain) {
        const size_t q_bytes = (size_t)nact * hd * sizeof(float);
        const int q_in_lds = q_bytes <= 65536;
        hipLaunchKernelGGL(index_score_plain_kernel,
                           dim3((unsigned)((nt + kPlainTokensPerGroup - 1) / kPlainTokensPerGroup),
                                (unsigned)n_queries),
                           dim3(kScoreThreads), q_in_lds ? q_bytes : 0, stream, q, w, kpool, block_table,
                           nts, heads, max_blocks_per_seq, stride, nt, nh, nact, hd, page_tokens, n_pages,
                           wscale, dscale, scores, ws, ws_stride, q_in_lds);
        return launch_status();
    }
#define RK_SCORE(RBV, HDV)                                                                      \
    hipLaunchKernelGGL((index_score_kernel<RBV, HDV>), grid, dim3(kScoreThreads), 0, stream, q, w, \
                       kpool, block_table, nts, heads, max_blocks_per_seq, stride, nt, nh, nact,  \
                       hd, page_tokens, n_pages, wscale, dscale, scores, ws, ws_stride)
    if (hd == 128) {
        if (nact <= 32) RK_SCORE(1, 128); else RK_SCORE(2, 128);
    } else {
        if (nact <= 32) RK_SCORE(1, 0); else RK_SCORE(2, 0);
    }
#undef RK_SCORE
    return launch_status();
}

}  // namespace rk

extern "C" int rivoli_index_score(const float* q, const float* w, const unsigned short* kcache,
                                  const unsigned int* heads, int nt, int nh, int nact, int hd,
                                  float wscale, float dscale, float* scores) {
    return rk::index_score_launch(q, w, kcache, nullptr, nullptr, heads, 1, 0, nt, nt, nh, nact, hd,
                                  0, 0, wscale, dscale, scores, nullptr, nullptr);
}

extern "C" int rivoli_index_score_paged(const float* q, const float* w,
                                        const unsigned short* kpool, const int* block_table,
                                        const int* nts, const unsigned int* heads, int n_queries,
                                        int max_blocks_per_seq, int stride, int nt, int nh,
                                        int nact, int hd, int page_tokens, int n_pages,
                                        float wscale, float dscale, float* scores, void* stream) {
    if (!block_table) return 1001;
    return rk::index_score_launch(q, w, kpool, block_table, nts, heads, n_queries,
                                  max_blocks_per_seq, stride, nt, nh, nact, hd, page_tokens,
                                  n_pages, wscale, dscale, scores, nullptr, (hipStream_t)stream);
}

extern "C" int rivoli_index_score_paged_hist(const float* q, const float* w,
                                             const unsigned short* kpool, const int* block_table,
                                             const int* nts, const unsigned int* heads,
                                             int n_queries, int max_blocks_per_seq, int stride,
                                             int nt, int nh, int nact, int hd, int page_tokens,
                                             int n_pages, float wscale, float dscale, float* scores,
                                             void* topk_workspace, void* stream) {
    if (!block_table || !topk_workspace) return 1001;
    return rk::index_score_launch(q, w, kpool, block_table, nts, heads, n_queries,
                                  max_blocks_per_seq, stride, nt, nh, nact, hd, page_tokens,
                                  n_pages, wscale, dscale, scores, topk_workspace,
                                  (hipStream_t)stream);
}

extern "C" int rivoli_index_append_paged(const float* k, const int* slot_mapping,
                                         unsigned short* kpool, int n_tokens, int hd,
                                         int page_tokens, int n_pages, unsigned int* bad_slots,
                                         void* stream) {
    if (!k || !slot_mapping || !kpool) return 1001;
    if (n_tokens <= 0 || hd <= 0 || page_tokens <= 0 || n_pages <= 0) return 1001;
    if ((hd % 8) != 0) return 1004;
    const long long work = (long long)n_tokens * (hd >> 3);
    (void)hipGetLastError();
    hipLaunchKernelGGL(rk::index_append_paged_kernel, dim3((unsigned)((work + 255) / 256)),
                       dim3(256), 0, (hipStream_t)stream, k, slot_mapping, kpool, n_tokens, hd,
                       (long long)n_pages * page_tokens, bad_slots);
    return rk::launch_status();
}
