// rivoli_mla_attend: MLA decode attention for ONE token over the reference's linear cache
// slabs, signature and guards kept (crates/backend/kernels/attn.hip:119-308):
//
//     clat_h = sum_t softmax_t((qabs_h . L_t + qrope_h . R_t) * scale) * L_t
//
// L_t = e4m3 codes times one f32 scale per 128 values, R_t = the bf16 roped key, token =
// rows ? rows[j] : j for j < nr. This is the single-query latency path of the reference's
// decode loop; the batched throughput path over the paged cache is rivoli_mla_attend_paged.
//
// Mapping for 64-wide waves: a workgroup owns 8 heads (one wave each) and one split of the
// attended rows; a tile of 16 tokens is widened to f32 into LDS once and shared by the 8
// heads (16-byte loads of codes, one scale per 128-block). A lane owns the columns
// i = lane (mod 64): its part of the 16 score dots, then one butterfly per token, then its
// 8 accumulator columns — so the accumulator stays in registers, as in the reference. The
// softmax is the reference's online form with expf; partials of several splits are merged
// by the same max-shifted combine, splits in ascending order. The split plan is a pure
// function of (H, nr): equal calls give bit-equal results.
// Launch-only; see include/rivoli_kvcache.h for the contract.
#include "codec.hpp"

namespace rk {

constexpr int kLinHeads = 8;        // heads (waves) per workgroup
constexpr int kLinTile = 16;        // tokens widened into LDS per step
constexpr int kLinAccRegs = 8;      // kvl <= 512 -> at most 8 columns per lane
constexpr int kLinMaxSplits = 16;   // bounds grid.y and the caller's scratch (attn.hip:66,98-103)
constexpr int kLinTargetBlocks = 512;
constexpr int kLinMinTilesPerSplit = 4;

struct LinPlan {
    int n_splits, tps;
};
static inline LinPlan lin_plan(int H, int nr, bool have_scratch) {
    const int ntiles = (nr + kLinTile - 1) / kLinTile;
    const int hblocks = (H + kLinHeads - 1) / kLinHeads;
    const int by_work = ntiles / kLinMinTilesPerSplit;
    const int by_grid = (kLinTargetBlocks + hblocks - 1) / hblocks;
    int n = by_work < by_grid ? by_work : by_grid;
    if (n > kLinMaxSplits) n = kLinMaxSplits;
    if (n < 1 || !have_scratch) n = 1;
    LinPlan p;
    p.tps = (ntiles + n - 1) / n;
    p.n_splits = (ntiles + p.tps - 1) / p.tps;
    return p;
}

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__global__ __launch_bounds__(kLinHeads* kWave) void mla_attend_linear_kernel(
    const float* __restrict__ qabs, const float* __restrict__ qrope,
    const uint8_t* __restrict__ lc8, const float* __restrict__ lscale,
    const uint16_t* __restrict__ rc, const unsigned int* __restrict__ rows, int H, int nr, int kvl,
    int rope, int n_blocks, float scale, int tps, float* __restrict__ clat,
    float* __restrict__ partial) {
    extern __shared__ float smem[];
    float* const Lt = smem;                    // [kLinTile][kvl]
    float* const Rt = smem + kLinTile * kvl;   // [kLinTile][rope]

    const int tid = threadIdx.x, lane = tid & 63;
    const int head = blockIdx.x * kLinHeads + __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool active = head < H;
    const int nacc = kvl >> 6;  // kvl is a multiple of 128: 2, 4, 6 or 8 columns per lane
    const float* const qa = qabs + (size_t)(active ? head : 0) * kvl;
    const float* const qr = qrope + (size_t)(active ? head : 0) * rope;

    // the lane's slice of the query, kept for the whole kernel
    float qv[kLinAccRegs];
#pragma unroll
    for (int k = 0; k < kLinAccRegs; ++k) qv[k] = (k < nacc && active) ? qa[lane + 64 * k] : 0.0f;

    float acc[kLinAccRegs] = {0, 0, 0, 0, 0, 0, 0, 0};
    float m = -INFINITY, l = 0.0f;
    const int r_begin = (int)blockIdx.y * tps * kLinTile;
    const int r_end = min(nr, r_begin + tps * kLinTile);

    for (int t0 = r_begin; t0 < r_end; t0 += kLinTile) {
        const int tcount = min(kLinTile, r_end - t0);
        // widen the tile: 16 codes per thread per step (one 16-byte load; kvl % 128 == 0
        // keeps a chunk inside one scale block), bf16 keys one by one (rope is any size)
        const int cpr = kvl >> 4;
        for (int c = tid; c < tcount * cpr; c += kLinHeads * kWave) {
            const int tt = c / cpr, i0 = (c - tt * cpr) * 16;
            const size_t t = rows ? (size_t)rows[t0 + tt] : (size_t)(t0 + tt);
            const float s = lscale[t * n_blocks + (i0 >> 7)];
            const uint8_t* src = lc8 + t * kvl + i0;
            uint32_t w[4];
            if ((reinterpret_cast<uintptr_t>(src) & 15) == 0) {
                const u32x4 v = *reinterpret_cast<const u32x4*>(src);
                w[0] = v.x, w[1] = v.y, w[2] = v.z, w[3] = v.w;
            } else {  // the slabs' alignment is whatever the caller has
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    w[j] = src[4 * j] | (src[4 * j + 1] << 8) | (src[4 * j + 2] << 16) | ((uint32_t)src[4 * j + 3] << 24);
            }
            float* dst = Lt + tt * kvl + i0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float f[4];
                e4m3x4_to_f32(w[j], f);
                dst[4 * j] = f[0] * s, dst[4 * j + 1] = f[1] * s, dst[4 * j + 2] = f[2] * s, dst[4 * j + 3] = f[3] * s;
            }
        }
        for (int c = tid; c < tcount * rope; c += kLinHeads * kWave) {
            const int tt = c / rope, d = c - tt * rope;
            const size_t t = rows ? (size_t)rows[t0 + tt] : (size_t)(t0 + tt);
            Rt[c] = __uint_as_float((uint32_t)rc[t * rope + d] << 16);
        }
        __syncthreads();

        if (active) {
            for (int tt = 0; tt < tcount; ++tt) {
                const float* Lrow = Lt + tt * kvl;
                float lat[kLinAccRegs];
                float part = 0.0f;
#pragma unroll
                for (int k = 0; k < kLinAccRegs; ++k) {
                    lat[k] = k < nacc ? Lrow[lane + 64 * k] : 0.0f;
                    part += qv[k] * lat[k];
                }
                for (int d = lane; d < rope; d += kWave) part += qr[d] * Rt[tt * rope + d];
                const float s = wave_sum_f32(part) * scale;
                const float m_new = fmaxf(m, s);
                const float corr = expf(m - m_new);
                const float p = expf(s - m_new);
#pragma unroll
                for (int k = 0; k < kLinAccRegs; ++k) acc[k] = acc[k] * corr + p * lat[k];
                l = l * corr + p;
                m = m_new;
            }
        }
        __syncthreads();
    }

    if (!active) return;
    if (partial) {
        float* pa = partial + ((size_t)blockIdx.y * H + head) * kvl;
        float* pml = partial + (size_t)kLinMaxSplits * H * kvl + ((size_t)blockIdx.y * H + head) * 2;
#pragma unroll
        for (int k = 0; k < kLinAccRegs; ++k)
            if (k < nacc) pa[lane + 64 * k] = acc[k];
        if (lane == 0) pml[0] = m, pml[1] = l;
    } else {
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
        for (int k = 0; k < kLinAccRegs; ++k)
            if (k < nacc) clat[(size_t)head * kvl + lane + 64 * k] = acc[k] * inv;
    }
}

// crates/backend/kernels/attn.hip:235-277: w_s = exp(m_s - max m), clat = sum w_s acc_s /
// sum w_s l_s, splits in ascending order; everything empty -> zeros.
__global__ __launch_bounds__(128) void mla_attend_linear_combine_kernel(
    const float* __restrict__ partial, int H, int kvl, int n_splits, float* __restrict__ clat) {
    const int head = blockIdx.x;
    const float* ml = partial + (size_t)kLinMaxSplits * H * kvl;
    float m_g = -INFINITY;
    for (int s = 0; s < n_splits; ++s) m_g = fmaxf(m_g, ml[((size_t)s * H + head) * 2]);
    const bool any = m_g > -INFINITY && m_g < INFINITY;
    float l_g = 0.0f;
    for (int s = 0; s < n_splits; ++s) {
        const float* p = ml + ((size_t)s * H + head) * 2;
        l_g += p[1] * (any ? expf(p[0] - m_g) : 0.0f);
    }
    const float inv = l_g > 0.0f ? 1.0f / l_g : 0.0f;
    for (int i = threadIdx.x; i < kvl; i += blockDim.x) {
        float sum = 0.0f;
        for (int s = 0; s < n_splits; ++s) {
            const float w = any ? expf(ml[((size_t)s * H + head) * 2] - m_g) : 0.0f;
            sum += partial[((size_t)s * H + head) * kvl + i] * w;
        }
        clat[(size_t)head * kvl + i] = sum * inv;
    }
}

}  // namespace rk

extern "C" size_t rivoli_mla_attend_scratch_floats(int H, int kvl) {
    if (H <= 0 || kvl <= 0) return 0;
    return (size_t)rk::kLinMaxSplits * (size_t)H * ((size_t)kvl + 2);
}

extern "C" int rivoli_mla_attend(const float* qabs, const float* qrope, const unsigned char* Lc8,
                                 const float* Lscale, const unsigned short* Rc,
                                 const unsigned int* rows, int H, int nr, int kvl, int rope,
                                 int n_blocks, float scale, float* clat, float* partial) {
    using namespace rk;
    if (H <= 0 || nr <= 0 || kvl <= 0 || rope <= 0 || n_blocks <= 0) return 1001;
    const size_t lds = ((size_t)kLinTile * kvl + (size_t)kLinTile * rope) * sizeof(float);
    if (lds > 65536) return 1002;
    if (kvl > kLinAccRegs * kWave || kvl % 128) return 1004;
    const LinPlan sp = lin_plan(H, nr, partial != nullptr);
    float* part = sp.n_splits > 1 ? partial : nullptr;
    (void)hipGetLastError();
    hipLaunchKernelGGL(mla_attend_linear_kernel, dim3((unsigned)((H + kLinHeads - 1) / kLinHeads), (unsigned)sp.n_splits),
                       dim3(kLinHeads * kWave), lds, nullptr, qabs, qrope, Lc8, Lscale, Rc, rows, H, nr, kvl,
                       rope, n_blocks, scale, sp.tps, clat, part);
    int rc = launch_status();
    if (rc != 0 || sp.n_splits <= 1) return rc;
    hipLaunchKernelGGL(mla_attend_linear_combine_kernel, dim3((unsigned)H), dim3(128), 0, nullptr, partial, H,
                       kvl, sp.n_splits, clat);
    return launch_status();
}
