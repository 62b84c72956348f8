// Quantize-and-append: new tokens' rows -> e4m3 codes + f32 scale(s) in the cache.
//
// Two layouts share the arithmetic (scale = amax > 0 ? amax/448 : 1, code = e4m3(v/scale)):
//   * paged, one scale per token (the whole width-wide row is the block), bf16 input rows,
//     destination chosen by a slot mapping;
//   * the reference's linear slabs: f32 input, one scale per 128 latent values, the roped
//     key kept as bf16 (crates/backend/kernels/fwd.hip:51-71).
//
// One wave64 owns one token. A lane holds 8 consecutive elements per step (one 16-byte load
// of bf16), so a 576-wide row is one full step plus an 8-lane tail; the per-token amax is a
// register max followed by a wave butterfly, which is exact and order-free, so it equals
// the reference's LDS tree bit for bit. Codes leave as 8-byte stores, contiguous per wave.
// Launch-only; see include/rivoli_kvcache.h for the contract of every entry point.
#include "codec.hpp"

namespace rk {

constexpr int kAppendWaves = 4;  // tokens per workgroup

// STEPS = ceil(width / 512): how many 8-element chunks a lane may own.
template <int STEPS>
__global__ __launch_bounds__(kAppendWaves* kWave) void kv_append_paged_kernel(
    const uint16_t* __restrict__ rows, const int* __restrict__ slot_mapping,
    uint8_t* __restrict__ pool, int n_tokens, int width, int page_tokens, long long n_slots,
    size_t page_bytes, unsigned int* __restrict__ bad_slots) {
    const int lane = threadIdx.x & (kWave - 1);
    const int token =
        __builtin_amdgcn_readfirstlane((int)(blockIdx.x * kAppendWaves + (threadIdx.x >> 6)));
    if (token >= n_tokens) return;
    const int slot = slot_mapping[token];
    if (slot < 0) return;  // padding
    if ((long long)slot >= n_slots) {
        if (lane == 0 && bad_slots) atomicAdd(bad_slots, 1u);
        return;
    }
    const int n_chunks = width >> 3;
    const u32x4* src = reinterpret_cast<const u32x4*>(rows + (size_t)token * width);

    u32x4 raw[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        int c = lane + s * kWave;
        raw[s] = c < n_chunks ? __builtin_nontemporal_load(src + c) : u32x4{0, 0, 0, 0};
    }
    float v[STEPS][8];
    float amax = 0.0f;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        const uint32_t w[4] = {raw[s].x, raw[s].y, raw[s].z, raw[s].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[s][2 * i] = bf16_lo_to_f32(w[i]);
            v[s][2 * i + 1] = bf16_hi_to_f32(w[i]);
            amax = fmaxf(amax, fmaxf(fabsf(v[s][2 * i]), fabsf(v[s][2 * i + 1])));
        }
    }
    amax = wave_max(amax);
    const float scl = amax > 0.0f ? amax / 448.0f : 1.0f;

    const int page = slot / page_tokens;
    const int off = slot - page * page_tokens;
    uint8_t* pg = pool + (size_t)page * page_bytes;
    u32x2* dst = reinterpret_cast<u32x2*>(pg + (size_t)off * width);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        int c = lane + s * kWave;
        if (c < n_chunks) {
            uint32_t lo = 0, hi = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                lo |= f32_to_e4m3(v[s][i] / scl) << (8 * i);
                hi |= f32_to_e4m3(v[s][4 + i] / scl) << (8 * i);
            }
            dst[c] = u32x2{lo, hi};
        }
    }
    if (lane == 0)
        *reinterpret_cast<float*>(pg + (size_t)page_tokens * width + (size_t)off * 4) = scl;
}

// Linear slabs, reference layout. One wave per token; a lane owns elements lane*2, lane*2+1
// of each 128-block (so a block is exactly one wave-wide butterfly), for up to 8 blocks.
__global__ __launch_bounds__(kAppendWaves* kWave) void append_kv_rows_kernel(
    const float* __restrict__ latent, const float* __restrict__ rope,
    uint8_t* __restrict__ lc8, float* __restrict__ lscale, uint16_t* __restrict__ rc, int pos0,
    int n_tokens, int kvl, int ropn, int n_blocks) {
    const int lane = threadIdx.x & (kWave - 1);
    const int t =
        __builtin_amdgcn_readfirstlane((int)(blockIdx.x * kAppendWaves + (threadIdx.x >> 6)));
    if (t >= n_tokens) return;
    const size_t pos = (size_t)pos0 + t;
    const float* lat = latent + (size_t)t * kvl;
    const int blocks = kvl >> 7;
    for (int b = 0; b < blocks; ++b) {
        // scalar loads and byte stores: the slabs' alignment is whatever the caller has
        const float x0 = lat[b * 128 + lane * 2], x1 = lat[b * 128 + lane * 2 + 1];
        float amax = wave_max(fmaxf(fabsf(x0), fabsf(x1)));
        float scl = amax > 0.0f ? amax / 448.0f : 1.0f;
        if (lane == 0) lscale[pos * n_blocks + b] = scl;
        uint8_t* d = lc8 + pos * kvl + b * 128 + lane * 2;
        d[0] = (uint8_t)f32_to_e4m3(x0 / scl);
        d[1] = (uint8_t)f32_to_e4m3(x1 / scl);
    }
    const float* rp = rope + (size_t)t * ropn;
    for (int i = lane; i < ropn; i += kWave) rc[pos * ropn + i] = f32_to_bf16(rp[i]);
}

__global__ void index_append_kernel(const float* __restrict__ k, uint16_t* __restrict__ kcache,
                                    int pos, int hd) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < hd) kcache[(size_t)pos * hd + i] = f32_to_bf16(k[i]);
}

static int append_kv_rows_launch(const float* latent, const float* rope, unsigned char* lc8,
                                 float* lscale, unsigned short* rc, int pos0, int n_tokens,
                                 int kvl, int ropn, int n_blocks, hipStream_t stream) {
    if (pos0 < 0 || n_tokens <= 0 || kvl <= 0 || ropn <= 0 || n_blocks <= 0) return 1001;
    if (!latent || !rope || !lc8 || !lscale || !rc) return 1001;
    if (kvl > 1024 || kvl < 128 || (kvl % 128) != 0 || ropn > kvl) return 1002;
    (void)hipGetLastError();
    dim3 grid((unsigned)((n_tokens + kAppendWaves - 1) / kAppendWaves));
    hipLaunchKernelGGL(append_kv_rows_kernel, grid, dim3(kAppendWaves * kWave), 0, stream,
                       latent, rope, lc8, lscale, rc, pos0, n_tokens, kvl, ropn, n_blocks);
    return launch_status();
}

}  // namespace rk

extern "C" size_t rivoli_kv_page_bytes(int page_tokens, int width) {
    if (page_tokens <= 0 || width <= 0) return 0;
    return (size_t)page_tokens * (size_t)width + (size_t)page_tokens * sizeof(float);
}

extern "C" int rivoli_kv_append_paged(const unsigned short* rows, const int* slot_mapping,
                                      unsigned char* pool, int n_tokens, int width,
                                      int page_tokens, int n_pages, unsigned int* bad_slots,
                                      void* stream) {
    using namespace rk;
    if (!rows || !slot_mapping || !pool) return 1001;
    if (n_tokens <= 0 || width <= 0 || page_tokens <= 0 || n_pages <= 0) return 1001;
    if (width > 1024) return 1002;
    if ((width % 16) != 0 || (page_tokens % 4) != 0) return 1004;
    const size_t page_bytes = rivoli_kv_page_bytes(page_tokens, width);
    const long long n_slots = (long long)n_pages * page_tokens;
    dim3 grid((unsigned)((n_tokens + kAppendWaves - 1) / kAppendWaves));
    dim3 block(kAppendWaves * kWave);
    (void)hipGetLastError();
    if (width <= 512) {
        hipLaunchKernelGGL(kv_append_paged_kernel<1>, grid, block, 0, (hipStream_t)stream, rows,
                           slot_mapping, pool, n_tokens, width, page_tokens, n_slots, page_bytes,
                           bad_slots);
    } else {
        hipLaunchKernelGGL(kv_append_paged_kernel<2>, grid, block, 0, (hipStream_t)stream, rows,
                           slot_mapping, pool, n_tokens, width, page_tokens, n_slots, page_bytes,
                           bad_slots);
    }
    return launch_status();
}

extern "C" int rivoli_append_kv_rows(const float* latent, const float* rope, unsigned char* lc8,
                                     float* lscale, unsigned short* rc, int pos0, int n_tokens,
                                     int kvl, int ropn, int n_blocks, void* stream) {
    return rk::append_kv_rows_launch(latent, rope, lc8, lscale, rc, pos0, n_tokens, kvl, ropn,
                                     n_blocks, (hipStream_t)stream);
}

extern "C" int rivoli_append_kv(const float* latent, const float* rope, unsigned char* lc8,
                                float* lscale, unsigned short* rc, int pos, int kvl, int ropn,
                                int n_blocks) {
    return rk::append_kv_rows_launch(latent, rope, lc8, lscale, rc, pos, 1, kvl, ropn, n_blocks,
                                     nullptr);
}

extern "C" int rivoli_index_append(const float* k, unsigned short* kcache, int pos, int hd) {
    if (hd <= 0 || pos < 0 || !k || !kcache) return 1001;
    (void)hipGetLastError();
    hipLaunchKernelGGL(rk::index_append_kernel, dim3((unsigned)((hd + 255) / 256)), dim3(256), 0,
                       nullptr, k, kcache, pos, hd);
    return rk::launch_status();
}

extern "C" int rivoli_device_sync(void) {
    hipError_t e = hipDeviceSynchronize();
    return e == hipSuccess ? 0 : -(int)e;
}
