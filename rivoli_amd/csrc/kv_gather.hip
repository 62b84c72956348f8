// Gather + dequantize: fp8 pages -> bf16 rows, dense (block table) and sparse (row list).
//
// The arithmetic is the tile load of the reference's attention kernel
// (crates/backend/kernels/attn.hip:168-177): val = e4m3_to_f32(code) * scale in f32, here
// rounded to nearest even into bf16. Both decodes are exact, the multiply is one IEEE
// operation and the narrowing is one rounding, so the result is bit-identical to the CPU
// rule whatever the schedule.
//
// Dense: one workgroup per 16 rows of a (sequence, page). A page's codes are one contiguous
// run and so is its destination (tokens of a page are consecutive in the output), so the
// kernel is a streaming transform: every lane loads 8 bytes of codes (a wave covers 512
// contiguous bytes) and stores 16 bytes of bf16 (a wave covers 1 KiB contiguous). All of a
// thread's loads are issued before the first use. Loads and stores carry the nontemporal
// hint: nothing here is read twice, and without it the kernel runs ~10% slower.
// Sparse: one workgroup per 32 selected rows of one query; the 32 row bases and scales are
// resolved once into LDS (block-table lookup), then the same 8-in/16-out streaming body runs
// over the 32 x width bytes.
// A decode step's "append one token per sequence, then gather every context" is one launch of
// the same kernels (APPEND): n_seqs extra workgroups quantize the new rows, store their records
// and write those tokens' bf16 rows themselves (dequantized from the codes they just made), and
// the gather units stop one token short of such a sequence's end — no workgroup reads what
// another one writes, so nothing has to be ordered inside the launch.
// Launch-only; see include/rivoli_kvcache.h for the contract of every entry point.
#include "append_common.hpp"

namespace rk {

constexpr int kGatherThreads = 256;
constexpr int kRowsPerGroup = 32;  // sparse gather: rows resolved per workgroup

// What the APPEND forms carry besides the gather's arguments.
struct AppendArgs {
    const uint16_t* new_rows;  // [n_seqs][width] bf16
    const int* slot_mapping;   // [n_seqs]: where sequence s's new token goes (negative: none)
    uint8_t* pool;             // the same pool, writable
    long long n_slots;
    unsigned int* bad_slots;
};
// Whether sequence s's last token is written by its append workgroup (and so skipped by the
// gather units): its slot is a slot of the pool and the sequence has a token to be the last.
__device__ __forceinline__ bool appends_last(const AppendArgs& ap, int s, int len) {
    const int slot = ap.slot_mapping[s];
    return len > 0 && slot >= 0 && (long long)slot < ap.n_slots;
}
// The append workgroup of sequence s: its first wave quantizes the row into the pool and writes
// the token's output row; the other waves have nothing to do.
template <int W>
__device__ __forceinline__ void append_unit(const AppendArgs& ap, const int* __restrict__ seq_lens,
                                            const int* __restrict__ cu_seqlens,
                                            uint16_t* __restrict__ out, int s, int width_rt,
                                            int page_tokens, size_t page_bytes) {
    if (threadIdx.x >= kWave) return;
    const int width = W ? W : width_rt;
    const int len = seq_lens[s];
    uint16_t* out_row = len > 0 ? out + ((size_t)cu_seqlens[s] + len - 1) * width : nullptr;
    if (width <= 512)
        append_token_wave<1>(ap.new_rows + (size_t)s * width, ap.slot_mapping + s, ap.pool, width,
                             page_tokens, ap.n_slots, page_bytes, ap.bad_slots, out_row);
    else
        append_token_wave<2>(ap.new_rows + (size_t)s * width, ap.slot_mapping + s, ap.pool, width,
                             page_tokens, ap.n_slots, page_bytes, ap.bad_slots, out_row);
}

// W / PT are the compile-time row width and page size (0 = take the runtime value), so the
// flagship 576 x 64 shape gets constant divisors and a fully unrolled body. A workgroup owns
// ROWS consecutive rows of one page (PT / ROWS workgroups per page): measured on MI355X,
// work units of 8-16 rows with one or two chunks per thread keep the chip's in-flight writes
// on a compact, nearly sequential frontier of the output and run ~7% faster than one
// workgroup per page.
template <int W, int PT, int THREADS, int ROWS>
__device__ __forceinline__ void gather_unit(const uint8_t* __restrict__ pool,
                                            const int* __restrict__ block_table,
                                            const int* __restrict__ cu_seqlens,
                                            uint16_t* __restrict__ out, int s, int blk, int part,
                                            int len, int max_blocks_per_seq, int width_rt,
                                            int page_tokens_rt, int n_pages, size_t page_bytes,
                                            unsigned int* __restrict__ bad_pages) {
    const int width = W ? W : width_rt;
    const int pt = PT ? PT : page_tokens_rt;
    const int t0 = blk * pt + part * ROWS;
    if (t0 >= len) return;
    const int valid = min(ROWS, len - t0);
    const int page = block_table[(size_t)s * max_blocks_per_seq + blk];
    if ((unsigned)page >= (unsigned)n_pages) {
        if (threadIdx.x == 0 && part == 0 && bad_pages) atomicAdd(bad_pages, 1u);
        return;
    }
    const uint8_t* pg = pool + (size_t)page * page_bytes;
    const u32x2* src = reinterpret_cast<const u32x2*>(pg + (size_t)part * ROWS * width);
    const float* scales = reinterpret_cast<const float*>(pg + (size_t)pt * width) + part * ROWS;
    u32x4* dst = reinterpret_cast<u32x4*>(out + ((size_t)cu_seqlens[s] + t0) * width);
    const int cpr = width >> 3;  // 8-byte chunks per row
    const int n_chunks = valid * cpr;
    // trips is a constant for a compile-time width, so the two loops below unroll fully
    constexpr int kMaxTrips = W ? (ROWS * (W / 8) + THREADS - 1) / THREADS : 4;

    for (int base = threadIdx.x; base < n_chunks; base += THREADS * kMaxTrips) {
        u32x2 raw[kMaxTrips];
        float scl[kMaxTrips];
#pragma unroll
        for (int u = 0; u < kMaxTrips; ++u) {
            int c = base + u * THREADS;
            if (c < n_chunks) {
                raw[u] = __builtin_nontemporal_load(src + c);
                scl[u] = scales[c / cpr];
            }
        }
#pragma unroll
        for (int u = 0; u < kMaxTrips; ++u) {
            int c = base + u * THREADS;
            if (c < n_chunks) __builtin_nontemporal_store(dequant8_bf16(raw[u], scl[u]), dst + c);
        }
    }
}

// The grid spans what the block tables could hold: blockIdx.y = sequence, blockIdx.x = its
// (page, part). Right when every sequence is about as long as the longest; with uneven lengths
// most workgroups only find out that they have nothing to do.
template <int W, int PT, int THREADS, int ROWS, bool APPEND>
__global__ __launch_bounds__(THREADS) void kv_gather_paged_kernel(
    const uint8_t* __restrict__ pool, const int* __restrict__ block_table,
    const int* __restrict__ seq_lens, const int* __restrict__ cu_seqlens,
    uint16_t* __restrict__ out, int max_blocks_per_seq, int width_rt, int page_tokens_rt,
    int n_pages, size_t page_bytes, unsigned int* __restrict__ bad_pages, AppendArgs ap) {
    const int parts = (PT ? PT : page_tokens_rt) / ROWS;
    const int s = blockIdx.y;
    if (APPEND && (int)blockIdx.x == max_blocks_per_seq * parts) {  // one more column: the appends
        append_unit<W>(ap, seq_lens, cu_seqlens, out, s, width_rt, PT ? PT : page_tokens_rt, page_bytes);
        return;
    }
    const int blk = (int)blockIdx.x / parts;
    const int part = (int)blockIdx.x - blk * parts;
    int len = seq_lens[s];
    if (APPEND && appends_last(ap, s, len)) --len;
    gather_unit<W, PT, THREADS, ROWS>(pool, block_table, cu_seqlens, out, s, blk, part, len,
                                      max_blocks_per_seq, width_rt, page_tokens_rt, n_pages,
                                      page_bytes, bad_pages);
}

// The same units on a flat grid sized by the batch's real token count: workgroup u finds the
// sequence its unit belongs to from the device-side lengths; sequence s owns ceil(len_s / ROWS)
// consecutive units. The lengths are scanned 64 per round across the lanes of every wave (one
// coalesced load, a DPP prefix sum, a ballot); walking them with uniform loads and scalar
// compares instead costs ~500 scalar instructions per 16 sequences per wave, which saturates
// the compute unit's one scalar pipe (measured: 0.63 against 0.66 of peak at 32 sequences,
// 0.37 against 0.63 at 128). No LDS, no barrier; at most n_seqs workgroups of the launch (the
// rounding of each sequence's last unit) find nothing to do.
template <int W, int PT, int THREADS, int ROWS, bool APPEND>
__global__ __launch_bounds__(THREADS) void kv_gather_flat_kernel(
    const uint8_t* __restrict__ pool, const int* __restrict__ block_table,
    const int* __restrict__ seq_lens, const int* __restrict__ cu_seqlens,
    uint16_t* __restrict__ out, int n_seqs, int max_blocks_per_seq, int width_rt,
    int page_tokens_rt, int n_pages, size_t page_bytes, unsigned int* __restrict__ bad_pages,
    AppendArgs ap) {
    static_assert(THREADS % kWave == 0, "the scan below runs in every wave and needs all 64 lanes of each");
    const int pt = PT ? PT : page_tokens_rt;
    const int parts = pt / ROWS;
    if (APPEND && (int)blockIdx.x < n_seqs) {  // the first n_seqs workgroups: the appends
        append_unit<W>(ap, seq_lens, cu_seqlens, out, (int)blockIdx.x, width_rt, pt, page_bytes);
        return;
    }
    const uint32_t u = blockIdx.x - (APPEND ? (uint32_t)n_seqs : 0u);
    const int cap = max_blocks_per_seq * pt;  // rows a block-table row can address
    uint32_t first = 0;                       // units of the sequences before s
    int s = -1, my_len = 0;
    {
        const int lane = threadIdx.x & (kWave - 1);
        for (int s0 = 0; s0 < n_seqs; s0 += kWave) {
            // (both loads unconditional, from an index that always exists: a load under a
            // condition is a branch with a wait of its own)
            const int at = min(s0 + lane, n_seqs - 1);
            int len = seq_lens[at];
            if (APPEND) len -= appends_last(ap, at, len) ? 1 : 0;
            len = s0 + lane < n_seqs ? min(max(len, 0), cap) : 0;
            const uint32_t units = (uint32_t)(len + ROWS - 1) / ROWS;
            const uint32_t incl = first + wave_inclusive_sum(units);
            const int passed = __popcll(__ballot(incl <= u));  // sequences ending at or before u
            if (passed < kWave) {
                if (s0 + passed < n_seqs) {
                    if (passed) first = (uint32_t)__builtin_amdgcn_readlane((int)incl, passed - 1);
                    s = s0 + passed;
                    my_len = __builtin_amdgcn_readlane(len, passed);
                }
                break;
            }
            first = wave_total(incl);
        }
    }
    if (s < 0) return;  // past the last sequence's last unit
    const int unit = (int)(u - first);
    const int blk = unit / parts;
    gather_unit<W, PT, THREADS, ROWS>(pool, block_table, cu_seqlens, out, s, blk, unit - blk * parts,
                                      my_len, max_blocks_per_seq, width_rt, page_tokens_rt, n_pages,
                                      page_bytes, bad_pages);
}

template <int W, int PT, int UNROLL>
__global__ __launch_bounds__(kGatherThreads) void kv_gather_rows_kernel(
    const uint8_t* __restrict__ pool, const int* __restrict__ block_table,
    const unsigned int* __restrict__ rows, const int* __restrict__ n_rows,
    uint16_t* __restrict__ out, int k, int nr_cap, int max_blocks_per_seq, int width_rt,
    int page_tokens_rt, int n_pages, size_t page_bytes, unsigned int* __restrict__ bad_rows) {
    const int width = W ? W : width_rt;
    const int pt = PT ? PT : page_tokens_rt;
    __shared__ unsigned long long s_base[kRowsPerGroup];
    __shared__ unsigned long long s_scale_at[kRowsPerGroup];
    __shared__ int s_skipped;

    const int q = blockIdx.y;
    const int r0 = (int)blockIdx.x * kRowsPerGroup;
    const int nr = n_rows ? min(n_rows[q], nr_cap) : nr_cap;
    if (r0 >= nr) return;
    const int cnt = min(kRowsPerGroup, nr - r0);

    if (threadIdx.x == 0) s_skipped = 0;
    __syncthreads();
    if ((int)threadIdx.x < cnt &&
        !resolve_row(rows[(size_t)q * k + r0 + threadIdx.x],
                     block_table + (size_t)q * max_blocks_per_seq, max_blocks_per_seq, width, pt,
                     n_pages, page_bytes, bad_rows, &s_base[threadIdx.x], &s_scale_at[threadIdx.x]))
        s_skipped = 1;
    __syncthreads();
    const bool plain = !s_skipped && cnt * (width >> 3) == kGatherThreads * UNROLL;
    stream_rows<kGatherThreads, UNROLL>(pool, s_base, s_scale_at, cnt, width, plain,
                                        out + ((size_t)q * k + r0) * width);
}

// out[i] = bf16(e4m3_to_f32(codes[i]) * scale): the dequant body alone, for codec census tests.
__global__ void e4m3_dequant_bf16_kernel(const uint8_t* __restrict__ codes, float scale,
                                         uint16_t* __restrict__ out, long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long step = (long long)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        // the packed decoder is the product path; feed it the byte in lane 0 of a dword
        u32x2 r = dequant4_bf16((uint32_t)codes[i], scale);
        out[i] = (uint16_t)(r.x & 0xffffu);
    }
}

}  // namespace rk

// total_tokens < 0: not known, the grid spans what the block tables could hold.
// ap.new_rows != nullptr: the APPEND forms.
static int gather_paged_launch(const unsigned char* pool, const int* block_table,
                               const int* seq_lens, const int* cu_seqlens, unsigned short* out,
                               int n_seqs, int max_blocks_per_seq, long long total_tokens,
                               int width, int page_tokens, int n_pages, unsigned int* bad_pages,
                               rk::AppendArgs ap, void* stream) {
    using namespace rk;
    if (!pool || !block_table || !seq_lens || !cu_seqlens || !out) return 1001;
    if (n_seqs <= 0 || max_blocks_per_seq <= 0 || width <= 0 || page_tokens <= 0 || n_pages <= 0)
        return 1001;
    if (n_seqs > 65535) return 1002;
    if (!gather_shape_ok(width, page_tokens) || !aligned16(pool) || !aligned16(out)) return 1004;
    const bool append = ap.new_rows != nullptr;
    const size_t page_bytes = (size_t)page_tokens * width + (size_t)page_tokens * 4;
    const long long capacity = (long long)n_seqs * max_blocks_per_seq * page_tokens;
    // The flat grid pays for finding each workgroup's sequence and saves the idle workgroups of
    // the grid form. Measured at 32 ragged sequences (1 K - 32 K rows): flat 0.72 of the HBM peak
    // whatever the tables' size, grid 0.70 with tables half full, 0.66 a third full, 0.62 a
    // quarter full; with every sequence at the tables' full length grid 0.75, flat 0.72. So:
    // flat when the batch fills less than 0.7 of what its block tables could hold.
    const bool flat = total_tokens >= 0 && total_tokens * 10 < capacity * 7;
    (void)hipGetLastError();
#define RK_GATHER_AS(WV, PTV, THREADS, FLAT_THREADS, ROWS, APPEND)                                 \
    do {                                                                                           \
        const unsigned parts = (unsigned)(page_tokens / (ROWS));                                   \
        if (flat) {                                                                                \
            const long long units = (total_tokens + (ROWS) - 1) / (ROWS) + n_seqs + ((APPEND) ? n_seqs : 0); \
            if (units > 0x7fffffffLL) return 1002;                                                 \
            hipLaunchKernelGGL((kv_gather_flat_kernel<WV, PTV, FLAT_THREADS, ROWS, APPEND>),       \
                               dim3((unsigned)units), dim3(FLAT_THREADS), 0, (hipStream_t)stream, pool, \
                               block_table, seq_lens, cu_seqlens, out, n_seqs, max_blocks_per_seq, \
                               width, page_tokens, n_pages, page_bytes, bad_pages, ap);            \
        } else {                                                                                   \
            hipLaunchKernelGGL((kv_gather_paged_kernel<WV, PTV, THREADS, ROWS, APPEND>),           \
                               dim3((unsigned)max_blocks_per_seq * parts + ((APPEND) ? 1u : 0u),   \
                                    (unsigned)n_seqs),                                             \
                               dim3(THREADS), 0, (hipStream_t)stream, pool, block_table, seq_lens, \
                               cu_seqlens, out, max_blocks_per_seq, width, page_tokens, n_pages,   \
                               page_bytes, bad_pages, ap);                                         \
        }                                                                                          \
    } while (0)
#define RK_GATHER(WV, PTV, THREADS, FLAT_THREADS, ROWS)                                            \
    do {                                                                                           \
        if (append)                                                                                \
            RK_GATHER_AS(WV, PTV, THREADS, FLAT_THREADS, ROWS, true);                              \
        else                                                                                       \
            RK_GATHER_AS(WV, PTV, THREADS, FLAT_THREADS, ROWS, false);                             \
    } while (0)
    if (width == 576 && page_tokens == 64)
        RK_GATHER(576, 64, 768, 576, 16);  // flat: 576 threads = two 8-byte chunks each
    else if (page_tokens % 16 == 0)
        RK_GATHER(0, 0, kGatherThreads, kGatherThreads, 16);
    else
        RK_GATHER(0, 0, kGatherThreads, kGatherThreads, 4);
#undef RK_GATHER
#undef RK_GATHER_AS
    return launch_status();
}

extern "C" int rivoli_kv_gather_paged(const unsigned char* pool, const int* block_table,
                                      const int* seq_lens, const int* cu_seqlens,
                                      unsigned short* out, int n_seqs, int max_blocks_per_seq,
                                      int width, int page_tokens, int n_pages,
                                      unsigned int* bad_pages, void* stream) {
    return gather_paged_launch(pool, block_table, seq_lens, cu_seqlens, out, n_seqs,
                               max_blocks_per_seq, -1, width, page_tokens, n_pages, bad_pages,
                               rk::AppendArgs{nullptr, nullptr, nullptr, 0, nullptr}, stream);
}

extern "C" int rivoli_kv_gather_paged_packed(const unsigned char* pool, const int* block_table,
                                             const int* seq_lens, const int* cu_seqlens,
                                             unsigned short* out, int n_seqs,
                                             int max_blocks_per_seq, long long total_tokens,
                                             int width, int page_tokens, int n_pages,
                                             unsigned int* bad_pages, void* stream) {
    if (total_tokens < 0) return 1001;
    return gather_paged_launch(pool, block_table, seq_lens, cu_seqlens, out, n_seqs,
                               max_blocks_per_seq, total_tokens, width, page_tokens, n_pages,
                               bad_pages, rk::AppendArgs{nullptr, nullptr, nullptr, 0, nullptr},
                               stream);
}

extern "C" int rivoli_kv_append_gather_paged(const unsigned short* new_rows, const int* slot_mapping,
                                             unsigned char* pool, const int* block_table,
                                             const int* seq_lens, const int* cu_seqlens,
                                             unsigned short* out, int n_seqs,
                                             int max_blocks_per_seq, long long total_tokens,
                                             int width, int page_tokens, int n_pages,
                                             unsigned int* bad_slots, unsigned int* bad_pages,
                                             void* stream) {
    if (!new_rows || !slot_mapping) return 1001;
    if (width > 1024) return 1002;  // the append's widest row
    if (!rk::aligned16(new_rows)) return 1004;
    const rk::AppendArgs ap = {new_rows, slot_mapping, pool, (long long)n_pages * page_tokens, bad_slots};
    return gather_paged_launch(pool, block_table, seq_lens, cu_seqlens, out, n_seqs,
                               max_blocks_per_seq, total_tokens, width, page_tokens, n_pages,
                               bad_pages, ap, stream);
}

// Query q gathers its first min(n_rows[q], nr_cap) listed rows (nr_cap when n_rows is null);
// the lists and the output are k rows apart.
int rk::gather_rows_launch(const unsigned char* pool, const int* block_table,
                           const unsigned int* rows, const int* n_rows, unsigned short* out,
                           int n_queries, int k, int nr_cap, int max_blocks_per_seq, int width,
                           int page_tokens, int n_pages, unsigned int* bad_rows, void* stream) {
    if (!pool || !block_table || !rows || !out) return 1001;
    if (n_queries <= 0 || k <= 0 || nr_cap <= 0 || nr_cap > k || max_blocks_per_seq <= 0 ||
        width <= 0 || page_tokens <= 0 || n_pages <= 0)
        return 1001;
    if (n_queries > 65535) return 1002;
    if (!gather_shape_ok(width, page_tokens) || !aligned16(pool) || !aligned16(out)) return 1004;
    const size_t page_bytes = (size_t)page_tokens * width + (size_t)page_tokens * 4;
    dim3 grid((unsigned)((nr_cap + kRowsPerGroup - 1) / kRowsPerGroup), (unsigned)n_queries);
    (void)hipGetLastError();
    if (width == 576 && page_tokens == 64) {
        hipLaunchKernelGGL((kv_gather_rows_kernel<576, 64, 9>), grid, dim3(kGatherThreads), 0,
                           (hipStream_t)stream, pool, block_table, rows, n_rows, out, k, nr_cap,
                           max_blocks_per_seq, width, page_tokens, n_pages, page_bytes, bad_rows);
    } else {
        hipLaunchKernelGGL((kv_gather_rows_kernel<0, 0, 4>), grid, dim3(kGatherThreads), 0,
                           (hipStream_t)stream, pool, block_table, rows, n_rows, out, k, nr_cap,
                           max_blocks_per_seq, width, page_tokens, n_pages, page_bytes, bad_rows);
    }
    return launch_status();
}

extern "C" int rivoli_kv_gather_rows_paged(const unsigned char* pool, const int* block_table,
                                           const unsigned int* rows, const int* n_rows,
                                           unsigned short* out, int n_queries, int k,
                                           int max_blocks_per_seq, int width, int page_tokens,
                                           int n_pages, unsigned int* bad_rows, void* stream) {
    return rk::gather_rows_launch(pool, block_table, rows, n_rows, out, n_queries, k, k,
                                  max_blocks_per_seq, width, page_tokens, n_pages, bad_rows, stream);
}

extern "C" int rivoli_codec_e4m3_dequant_bf16(const unsigned char* codes, float scale,
                                              unsigned short* out, long long n, void* stream) {
    if (!codes || !out || n <= 0) return 1001;
    long long blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    (void)hipGetLastError();
    hipLaunchKernelGGL(rk::e4m3_dequant_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, codes, scale, out, n);
    return rk::launch_status();
}
