// Quantize-and-append: new tokens' rows -> e4m3 codes + f32 scale(s) in the cache.
//
// Two layouts share the arithmetic (scale = amax > 0 ? amax/448 : 1, code = e4m3(v/scale)):
//   * paged, one scale per token (the whole width-wide row is the block), bf16 input rows,
//     destination chosen by a slot mapping;
//   * the reference's linear slabs: f32 input, one scale per 128 latent values, the roped
//     key kept as bf16 (crates/backend/kernels/fwd.hip:51-71).
//
// Paged: one wave64 owns 8 tokens (see the kernel). Linear: one wave64 owns one token. Either
// way the amax is a max over registers, LDS and wave butterflies — exact and order-free, so
// it equals the reference's LDS tree bit for bit.
// Launch-only; see include/rivoli_kvcache.h for the contract of every entry point.
#include <type_traits>

#include "append_common.hpp"

namespace rk {

constexpr int kAppendWaves = 4;   // linear-slab kernel: tokens per workgroup
constexpr int kRowsPerWave = 8;   // paged kernel: tokens per (one-wave) workgroup
constexpr int kMaxChunksPerRow = 128;  // width <= 1024
// Batches at least this large take the 8-rows-per-wave kernel (throughput); smaller ones the
// one-wave-per-token kernel (latency) — except 576-wide rows, which have a kernel of their own
// for the sizes in between (kWideAppendTokens .. kWideAppendBelow).
// RIVOLI_BULK_APPEND_TOKENS overrides it at build time.
#ifndef RIVOLI_BULK_APPEND_TOKENS
#define RIVOLI_BULK_APPEND_TOKENS 16384
#endif
constexpr int kBulkAppendTokens = RIVOLI_BULK_APPEND_TOKENS;
// From this many tokens (of 576-wide rows) up to the bulk threshold: the 576-thread kernel.
#ifndef RIVOLI_WIDE_APPEND_TOKENS
#define RIVOLI_WIDE_APPEND_TOKENS 512
#endif
constexpr int kWideAppendTokens = RIVOLI_WIDE_APPEND_TOKENS;
constexpr int kWideAppendBelow = 20480;  // from here on the one-wave-per-8-tokens kernel is faster

// Paged append. One wave64 workgroup owns 8 consecutive tokens = one contiguous run of the
// input, cut into 16-byte chunks (8 bf16) dealt round-robin to the lanes: for a 576-wide row
// that is 8 x 72 = 576 chunks, exactly 9 per lane, so no lane idles and every load is a full
// 1 KiB wave access. Per-chunk maxima go through LDS to a segmented reduce (8 lanes per row),
// which is exact and order-free like the reference's LDS tree; one lane per row derives the
// scale, its reciprocal and the row's destination. Codes leave as 8-byte nontemporal stores
// (nothing here is read again; measured 6 % faster than plain stores). With the arithmetic
// hidden (a variant that skips it runs no faster), the kernel moves its 2:1 read:write mix at
// the rate this part gives any such copy.
// CPR = chunks per row at compile time (0 = runtime, up to 128).
template <int CPR>
__global__ __launch_bounds__(kWave) void kv_append_paged_kernel(
    const uint16_t* __restrict__ rows, const int* __restrict__ slot_mapping,
    uint8_t* __restrict__ pool, int n_tokens, int width, int page_tokens, long long n_slots,
    size_t page_bytes, unsigned int* __restrict__ bad_slots) {
    constexpr int MAXJ = CPR ? (kRowsPerWave * CPR + kWave - 1) / kWave
                             : kRowsPerWave * kMaxChunksPerRow / kWave;
    constexpr unsigned long long kSkip = ~0ull;
    __shared__ float s_amax[kRowsPerWave * (CPR ? CPR : kMaxChunksPerRow)];
    __shared__ u32x4 s_row[kRowsPerWave];  // scale, its reciprocal, the exact-path band (bits)
    __shared__ unsigned long long s_dst[kRowsPerWave], s_sdst[kRowsPerWave];

    const int cpr = CPR ? CPR : width >> 3;
    const int lane = threadIdx.x;
    const int t0 = (int)blockIdx.x * kRowsPerWave;
    const int nrows = min(kRowsPerWave, n_tokens - t0);
    const int n_chunks = nrows * cpr;
    const u32x4* src = reinterpret_cast<const u32x4*>(rows + (size_t)t0 * width);

    u32x4 raw[MAXJ];
#pragma unroll
    for (int j = 0; j < MAXJ; ++j) {
        const int c = lane + j * kWave;
        raw[j] = c < n_chunks ? __builtin_nontemporal_load(src + c) : u32x4{0, 0, 0, 0};
    }
    if (lane < kRowsPerWave) {  // where each row goes (or nowhere)
        unsigned long long dst = kSkip, sdst = 0;
        if (lane < nrows) {
            const int slot = slot_mapping[t0 + lane];
            if (slot >= 0) {
                if ((long long)slot < n_slots) {
                    const int page = slot / page_tokens, off = slot - page * page_tokens;
                    dst = (size_t)page * page_bytes + (size_t)off * width;
                    sdst = (size_t)page * page_bytes + (size_t)page_tokens * width + (size_t)off * 4;
                } else if (bad_slots) {
                    atomicAdd(bad_slots, 1u);
                }
            }
        }
        s_dst[lane] = dst;
        s_sdst[lane] = sdst;
    }
    // Row maxima. |bf16| patterns order like the values they encode, so the chunk maxima are
    // packed 16-bit integer maxima (one AND and one packed max per two elements) and every
    // later step compares bit patterns. A NaN's pattern sorts above infinity, while the rule's
    // max ignores NaNs: a row whose maximum comes out a NaN is folded again with float maxima.
    auto row_maxima = [&](auto as_bits) {
        constexpr bool kBits = decltype(as_bits)::value;
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) {
            const int c = lane + j * kWave;
            if (c < n_chunks) {
                const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
                if constexpr (kBits) {
                    u16x2 m = {0, 0};
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2, w[i] & 0x7fff7fffu));
                    s_amax[c] = __uint_as_float((uint32_t)max(m.x, m.y) << 16);
                } else {
                    float m = 0.0f;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        m = fmaxf(m, fmaxf(fabsf(bf16_lo_to_f32(w[i])), fabsf(bf16_hi_to_f32(w[i]))));
                    s_amax[c] = m;
                }
            }
        }
        __syncthreads();
        // lane = (row, part): each of a row's 8 lanes folds a slice of its chunk maxima
        const int r = lane >> 3, part = lane & 7;
        const int per = (cpr + 7) >> 3;
        constexpr int PER_MAX = CPR ? (CPR + 7) / 8 : kMaxChunksPerRow / 8;
        float m = 0.0f;
        if (r < nrows) {
#pragma unroll
            for (int i = 0; i < PER_MAX; ++i) {  // independent LDS reads, not a dependent loop
                const int at = part * per + i;
                if (i < per && at < cpr) {
                    const float v = s_amax[r * cpr + at];
                    m = kBits ? __uint_as_float(max(__float_as_uint(m), __float_as_uint(v))) : fmaxf(m, v);
                }
            }
        }
#pragma unroll
        for (int off = 1; off < 8; off <<= 1) {
            const float o = __shfl_xor(m, off, kWave);
            m = kBits ? __uint_as_float(max(__float_as_uint(m), __float_as_uint(o))) : fmaxf(m, o);
        }
        return m;
    };
    float m = row_maxima(std::true_type{});
    if (__any(__float_as_uint(m) > 0x7f800000u)) {  // some row holds a NaN
        __syncthreads();
        m = row_maxima(std::false_type{});
    }
    {
        const int r = lane >> 3, part = lane & 7;
        if (part == 0 && r < nrows) {
            const float scl = m > 0.0f ? m / 448.0f : 1.0f;
            const u32x4 row = {__float_as_uint(scl), __float_as_uint(1.0f / scl), row_band(scl), 0u};
            s_row[r] = row;
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < MAXJ; ++j) {
        const int c = lane + j * kWave;
        if (c < n_chunks) {
            const int r = c / cpr, col = c - r * cpr;
            const unsigned long long dst = s_dst[r];
            if (dst != kSkip) {
                const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
                const u32x4 row = s_row[r];
                __builtin_nontemporal_store(quantize8(w, __uint_as_float(row.x), __uint_as_float(row.y), row.z),
                                            reinterpret_cast<u32x2*>(pool + dst) + col);
            }
        }
    }
    // the scales last: a global store ahead of a barrier would make the barrier wait for it
    if (lane < nrows && s_dst[lane] != kSkip)
        *reinterpret_cast<float*>(pool + s_sdst[lane]) = __uint_as_float(s_row[lane].x);
}

// Paged append, mid-sized batches of 576-wide rows (a prefill chunk of a few thousand tokens):
// the bulk kernel's work unit — 8 consecutive tokens = 576 16-byte chunks — dealt to 576
// threads, one chunk each, so a launch of a few thousand tokens still fills the chip with
// loads in flight (the one-wave form keeps 9 chunks per lane and, below ~16 K tokens, too few
// waves per compute unit; the wave-per-token form below issues a second, almost empty step for
// the row's last 8 chunks). A chunk's maximum is taken NaN-free on the spot (a chunk holding a
// NaN folds its other values with float maxima), wave 0 folds the 72 chunk maxima of each row
// (8 lanes per row) and derives the row's scale, its reciprocal and the exact-path band.
constexpr int kWideThreads = kRowsPerWave * 72;
// J chunks per thread: a workgroup owns 8 J consecutive tokens.
template <int J>
__global__ __launch_bounds__(kWideThreads) void kv_append_paged_wide_kernel(
    const uint16_t* __restrict__ rows, const int* __restrict__ slot_mapping,
    uint8_t* __restrict__ pool, int n_tokens, int page_tokens, long long n_slots,
    size_t page_bytes, unsigned int* __restrict__ bad_slots) {
    constexpr int CPR = 72, W = CPR * 8, ROWS = kRowsPerWave * J;
    constexpr int PARTS = kWave / ROWS, PER = CPR / PARTS;  // wave 0: lanes per row, chunks per lane
    static_assert(PARTS * ROWS == kWave && PER * PARTS == CPR, "a wave folds the rows' chunk maxima");
    constexpr unsigned long long kSkip = ~0ull;
    __shared__ uint32_t s_amax[kWideThreads * J];
    __shared__ u32x4 s_row[ROWS];
    __shared__ unsigned long long s_dst[ROWS], s_sdst[ROWS];
    const int tid = threadIdx.x;
    const int t0 = (int)blockIdx.x * ROWS;
    const int nrows = min(ROWS, n_tokens - t0);
    const u32x4* src = reinterpret_cast<const u32x4*>(rows + (size_t)t0 * W);
    u32x4 raw[J];
#pragma unroll
    for (int j = 0; j < J; ++j)
        raw[j] = tid + j * kWideThreads < nrows * CPR ? __builtin_nontemporal_load(src + tid + j * kWideThreads)
                                                      : u32x4{0, 0, 0, 0};
    if (tid < ROWS) {  // where each row goes (or nowhere)
        unsigned long long dst = kSkip, sdst = 0;
        if (tid < nrows) {
            const int slot = slot_mapping[t0 + tid];
            if (slot >= 0) {
                if ((long long)slot < n_slots) {
                    const int page = slot / page_tokens, off = slot - page * page_tokens;
                    dst = (size_t)page * page_bytes + (size_t)off * W;
                    sdst = (size_t)page * page_bytes + (size_t)page_tokens * W + (size_t)off * 4;
                } else if (bad_slots) {
                    atomicAdd(bad_slots, 1u);
                }
            }
        }
        s_dst[tid] = dst;
        s_sdst[tid] = sdst;
    }
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
        // |bf16| patterns order like their values: a packed 16-bit integer maximum
        u16x2 m = {0, 0};
#pragma unroll
        for (int i = 0; i < 4; ++i)
            m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2, w[i] & 0x7fff7fffu));
        uint32_t top = (uint32_t)max(m.x, m.y) << 16;
        if (top > 0x7f800000u) {  // the chunk holds a NaN, which the rule's max ignores
            float f = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                f = fmaxf(f, fmaxf(fabsf(bf16_lo_to_f32(w[i])), fabsf(bf16_hi_to_f32(w[i]))));
            top = __float_as_uint(f);
        }
        s_amax[tid + j * kWideThreads] = top;
    }
    __syncthreads();
    if (tid < kWave) {
        const int r = tid / PARTS, part = tid - r * PARTS;
        uint32_t m = 0u;
#pragma unroll
        for (int i = 0; i < PER; ++i) m = max(m, s_amax[r * CPR + part * PER + i]);
#pragma unroll
        for (int off = 1; off < PARTS; off <<= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off, kWave));
        if (part == 0) {
            const float amax = __uint_as_float(m);
            const float scl = amax > 0.0f ? amax / 448.0f : 1.0f;
            s_row[r] = u32x4{__float_as_uint(scl), __float_as_uint(1.0f / scl), row_band(scl), 0u};
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const int c = tid + j * kWideThreads;
        const int r = c / CPR, col = c - r * CPR;
        if (c < nrows * CPR) {
            const unsigned long long dst = s_dst[r];
            if (dst != kSkip) {
                const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
                const u32x4 row = s_row[r];
                __builtin_nontemporal_store(quantize8(w, __uint_as_float(row.x), __uint_as_float(row.y), row.z),
                                            reinterpret_cast<u32x2*>(pool + dst) + col);
                if (col == 0) *reinterpret_cast<float*>(pool + s_sdst[r]) = __uint_as_float(row.x);
            }
        }
    }
}

// Paged append, low-latency form for small batches (decode steps, short prefill chunks): one
// wave64 per token, 4 tokens per workgroup, no LDS and no barrier. A lane holds 8 consecutive
// elements per step (one 16-byte load), so a 576-wide row is one full step plus an 8-lane
// tail; the amax is a register max plus a wave butterfly. Half the lanes idle in the tail
// step, which is why large batches use the 8-rows-per-wave kernel above instead.
// STEPS = ceil(width / 512).
template <int STEPS>
__global__ __launch_bounds__(kAppendWaves* kWave) void kv_append_paged_token_kernel(
    const uint16_t* __restrict__ rows, const int* __restrict__ slot_mapping,
    uint8_t* __restrict__ pool, int n_tokens, int width, int page_tokens, long long n_slots,
    size_t page_bytes, unsigned int* __restrict__ bad_slots) {
    const int token =
        __builtin_amdgcn_readfirstlane((int)(blockIdx.x * kAppendWaves + (threadIdx.x >> 6)));
    if (token >= n_tokens) return;
    append_token_wave<STEPS>(rows + (size_t)token * width, slot_mapping + token, pool, width,
                             page_tokens, n_slots, page_bytes, bad_slots, nullptr);
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
    if ((width % 16) != 0 || (page_tokens % 4) != 0 || !aligned16(rows) || !aligned16(pool)) return 1004;
    const size_t page_bytes = rivoli_kv_page_bytes(page_tokens, width);
    const long long n_slots = (long long)n_pages * page_tokens;
    (void)hipGetLastError();
    // measured on MI355X, 576-wide rows: 512 tokens 4.0 us either way; 8192 tokens 5.6 us (wave per
    // token: 6.7); 16384 tokens 8.6 us (one wave per 8 tokens: 9.6); 24576: 12.3 against 11.7
    if (width == 576 && n_tokens >= kWideAppendTokens && n_tokens < kWideAppendBelow) {
        // chunks per thread by size (8192 tokens: 5.5 / 5.25 / 5.8 us with 1 / 2 / 4; 16384 tokens:
        // 8.4 / 8.0 / 7.7; 4096 tokens: 4.15 / 4.4 with 1 / 2)
#define RK_WIDE(J)                                                                                     \
    hipLaunchKernelGGL(kv_append_paged_wide_kernel<J>,                                                 \
                       dim3((unsigned)((n_tokens + kRowsPerWave * (J) - 1) / (kRowsPerWave * (J)))),   \
                       dim3(kWideThreads), 0, (hipStream_t)stream, rows, slot_mapping, pool, n_tokens, \
                       page_tokens, n_slots, page_bytes, bad_slots)
        if (n_tokens < 6144)
            RK_WIDE(1);
        else if (n_tokens < 12288)
            RK_WIDE(2);
        else
            RK_WIDE(4);
#undef RK_WIDE
        return launch_status();
    }
    if (n_tokens < kBulkAppendTokens) {
        dim3 grid((unsigned)((n_tokens + kAppendWaves - 1) / kAppendWaves));
        dim3 block(kAppendWaves * kWave);
        if (width <= 512)
            hipLaunchKernelGGL(kv_append_paged_token_kernel<1>, grid, block, 0,
                               (hipStream_t)stream, rows, slot_mapping, pool, n_tokens, width,
                               page_tokens, n_slots, page_bytes, bad_slots);
        else
            hipLaunchKernelGGL(kv_append_paged_token_kernel<2>, grid, block, 0,
                               (hipStream_t)stream, rows, slot_mapping, pool, n_tokens, width,
                               page_tokens, n_slots, page_bytes, bad_slots);
        return launch_status();
    }
    dim3 grid((unsigned)((n_tokens + kRowsPerWave - 1) / kRowsPerWave));
    dim3 block(kWave);
    if (width == 576) {
        hipLaunchKernelGGL(kv_append_paged_kernel<72>, grid, block, 0, (hipStream_t)stream, rows,
                           slot_mapping, pool, n_tokens, width, page_tokens, n_slots, page_bytes,
                           bad_slots);
    } else {
        hipLaunchKernelGGL(kv_append_paged_kernel<0>, grid, block, 0, (hipStream_t)stream, rows,
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
