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
// A workgroup stages its query once and walks 512 tokens (4 waves x 4 blocks of 32). The
// kernel reads hd*2 bytes per token and is bound by that stream, not by the matrix cores.
// Launch-only; see include/rivoli_kvcache.h for the contract of every entry point.
#include "codec.hpp"

namespace rk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kScoreThreads = 256;
constexpr int kScoreWaves = kScoreThreads / kWave;
constexpr int kScoreMaxHeads = 64;   // active heads, padded to a multiple of 32
constexpr int kScoreMaxHd = 128;     // head dimension, a multiple of 16
constexpr int kScoreBlocks = 4;      // 32-token blocks per wave
constexpr int kScoreTokensPerGroup = kScoreWaves * kScoreBlocks * 32;
constexpr int kScoreRowPad = 8;      // bf16 of padding per staged query row

// RB = 32-head row blocks (1 or 2).
template <int RB>
__global__ __launch_bounds__(kScoreThreads) void index_score_kernel(
    const float* __restrict__ q, const float* __restrict__ w,
    const uint16_t* __restrict__ kpool, const int* __restrict__ block_table,
    const int* __restrict__ nts, const unsigned int* __restrict__ heads, int max_blocks_per_seq,
    int stride, int nt_all, int nh, int nact, int hd, int page_tokens, int n_pages, float wscale,
    float dscale, float* __restrict__ scores) {
    __shared__ __attribute__((aligned(16))) uint16_t s_qh[RB * 32][kScoreMaxHd + kScoreRowPad];
    __shared__ __attribute__((aligned(16))) uint16_t s_ql[RB * 32][kScoreMaxHd + kScoreRowPad];
    __shared__ float s_w[RB * 32];

    const int qi = blockIdx.y;
    const int nt = nts ? min(nts[qi], nt_all) : nt_all;
    const int t0 = (int)blockIdx.x * kScoreTokensPerGroup;
    if (t0 >= nt) return;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // ---- stage the active heads: q = hi + lo in bf16, and the per-head weight ----
    for (int idx = tid; idx < RB * 32 * hd; idx += kScoreThreads) {
        const int a = idx / hd, d = idx - a * hd;
        float val = 0.0f;
        if (a < nact) {
            const int h = heads ? (int)heads[a] : a;
            if ((unsigned)h < (unsigned)nh) val = q[((size_t)qi * nh + h) * hd + d];
        }
        const uint16_t hi = f32_to_bf16(val);
        const uint16_t lo = f32_to_bf16(val - __uint_as_float((uint32_t)hi << 16));
        s_qh[a][d] = hi;
        s_ql[a][d] = lo;
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
    for (int it = 0; it < kScoreBlocks; ++it) {
        const int tb = t0 + (it * kScoreWaves + wave) * 32;
        if (tb >= nt) break;  // wave-uniform
        const int token = tb + col;
        bool valid = token < nt;
        const int tc = valid ? token : nt - 1;  // a clamped, always readable token
        size_t slot = (size_t)tc;
        if (block_table) {
            const int page = block_table[(size_t)qi * max_blocks_per_seq + tc / page_tokens];
            const bool ok = (unsigned)page < (unsigned)n_pages;
            valid = valid && ok;
            slot = ok ? (size_t)page * page_tokens + (size_t)(tc % page_tokens) : 0;
        }
        const uint16_t* krow = kpool + slot * hd + khalf;
        bf16x8 kb[kScoreMaxHd / 16];
#pragma unroll
        for (int s = 0; s < kScoreMaxHd / 16; ++s)
            if (s < ksteps) kb[s] = *reinterpret_cast<const bf16x8*>(krow + 16 * s);

        f32x16 acc[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[rb][v] = 0.0f;
#pragma unroll
        for (int s = 0; s < kScoreMaxHd / 16; ++s) {
            if (s < ksteps) {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    const bf16x8 ah =
                        *reinterpret_cast<const bf16x8*>(&s_qh[rb * 32 + col][khalf + 16 * s]);
                    const bf16x8 al =
                        *reinterpret_cast<const bf16x8*>(&s_ql[rb * 32 + col][khalf + 16 * s]);
                    acc[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, kb[s], acc[rb], 0, 0, 0);
                    acc[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, kb[s], acc[rb], 0, 0, 0);
                }
            }
        }
        // accumulator element v of a lane is head row 8*(v/4) + 4*(lane/32) + v%4, token `col`
        float sum = 0.0f;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = rb * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                sum += s_w[row] * fmaxf(acc[rb][v] * dscale, 0.0f);
            }
        sum += __shfl_xor(sum, 32, kWave);
        if (lane < 32 && valid) scores[(size_t)qi * stride + token] = sum;
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
                              float dscale, float* scores, hipStream_t stream) {
    if (!q || !w || !kpool || !scores) return 1001;
    if (n_queries <= 0 || nt <= 0 || nh <= 0 || nact <= 0 || nact > nh || hd <= 0) return 1001;
    if (block_table && (max_blocks_per_seq <= 0 || page_tokens <= 0 || n_pages <= 0)) return 1001;
    if (nact > kScoreMaxHeads || hd > kScoreMaxHd || stride < nt || n_queries > 65535) return 1002;
    if ((hd % 16) != 0) return 1004;
    dim3 grid((unsigned)((nt + kScoreTokensPerGroup - 1) / kScoreTokensPerGroup),
              (unsigned)n_queries);
    (void)hipGetLastError();
    if (nact <= 32)
        hipLaunchKernelGGL(index_score_kernel<1>, grid, dim3(kScoreThreads), 0, stream, q, w, kpool,
                           block_table, nts, heads, max_blocks_per_seq, stride, nt, nh, nact, hd,
                           page_tokens, n_pages, wscale, dscale, scores);
    else
        hipLaunchKernelGGL(index_score_kernel<2>, grid, dim3(kScoreThreads), 0, stream, q, w, kpool,
                           block_table, nts, heads, max_blocks_per_seq, stride, nt, nh, nact, hd,
                           page_tokens, n_pages, wscale, dscale, scores);
    return launch_status();
}

}  // namespace rk

extern "C" int rivoli_index_score(const float* q, const float* w, const unsigned short* kcache,
                                  const unsigned int* heads, int nt, int nh, int nact, int hd,
                                  float wscale, float dscale, float* scores) {
    return rk::index_score_launch(q, w, kcache, nullptr, nullptr, heads, 1, 0, nt, nt, nh, nact, hd,
                                  0, 0, wscale, dscale, scores, nullptr);
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
                                  n_pages, wscale, dscale, scores, (hipStream_t)stream);
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
