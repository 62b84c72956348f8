// The pooling stage of the second cache format's compressor: `ratio` consecutive positions
// become one compressed cache row (crates/backend/kernels/kvcompress.hip:103-384, launchers
// :386-478; CPU statement crates/oracles/src/v4oracle/compress.rs:42-199). Three launches, the
// reference's signatures:
//   deposit  writes the trailing partial window (prefill) or this step's row (decode) into the
//            per-sequence state, the position-in-block embedding added to the scores;
//   prefill  one output row per complete block: per feature a softmax over the window's
//            entries (2 * ratio of them on overlapping layers: the previous block's rows
//            contribute their first d dims, the block's own rows their last d; block 0's
//            missing half is masked) and the weighted sum; then the bf16 store, RMSNorm with its
//            bf16 store, and the adjacent-pair rotation of the last rd dims at the block's
//            FIRST position, stored as bf16 values in f32;
//   decode   the same out of the state once a window completes, then the window slides.
// The projections that produce kv / score (two GEMMs) and the block quantization that follows
// (act_quant.hip) are separate launches, as in the reference.
//
// Shape here: a workgroup per output row; a lane owns 4 consecutive features (16-byte loads,
// coalesced across the wave). Windows of up to 16 entries are fetched once, all loads in
// flight together, and every pass of the softmax runs from registers (the reference re-reads
// each entry three times and evaluates expf twice per element). Wider windows stream three
// times, one feature per lane with four times the lanes, out of L2. The row then stays in
// LDS through norm and rotation. HBM traffic is the window once plus the row once.
#include "codec.hpp"
#include "rivoli_kvcache.h"

// the rotation's a*c - b*s is two products and a subtraction in the reference's arithmetic
#pragma clang fp contract(off)

namespace rk {

typedef rivoli_comp_geom CompGeom;
typedef rivoli_comp_finish CompFinish;
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kCompEntsMax = 128;   // the reference's bound on a pooling window
constexpr int kCompRegEnts = 16;    // windows up to this many entries live in registers
constexpr int kCompMaxD = 8192;     // one row in LDS

__device__ __forceinline__ float rbf16(float x) {
    return __uint_as_float((uint32_t)f32_to_bf16(x) << 16);
}

// Where entry j of a window lives. The two facts are flags, not null pointers: a pointer
// that was computed must be compared with null again, entry by entry, in scalar code.
struct Entry {
    const float* kv;
    const float* sc;
    const float* ape;
    bool live;  // false: masked, the pointers mean nothing
    bool emb;   // false: the embedding is already in the score
};
__device__ __forceinline__ Entry masked_entry() { return Entry{nullptr, nullptr, nullptr, false, false}; }

// Prefill's overlap_transform as an index map (kvcompress.hip:264-309). kv_own / sc_own point
// at the first row of block b: the one 64-bit product of the address is taken once per
// workgroup and an entry adds a small signed element offset. OVERLAP (two halves per row,
// ratio 4, eight entries: the guard admits no other overlapping geometry) is a compile-time
// fact so that which row and half entry j reads is one too. Decided per entry at run time, the
// scalar arithmetic in front of a row's first load was ~600 instructions and spilled scalar
// registers; it is ~200 now. The launch took the same time either way.
template <bool OVERLAP>
__device__ __forceinline__ Entry prefill_entry(const float* kv_own, const float* sc_own,
                                               const float* ape, const CompGeom& p, int b, int j) {
    if constexpr (OVERLAP) {
        constexpr int kRatio = 4;
        if (j >= kRatio) {  // this block's rows, their second half
            const int rel = (j - kRatio) * p.cd + p.d;
            return Entry{kv_own + rel, sc_own + rel, ape + rel, true, true};
        }
        const int rel = (j - kRatio) * p.cd;  // the block before, first half: block 0 has none
        return Entry{kv_own + rel, sc_own + rel, ape + j * p.cd, b != 0, b != 0};
    } else {
        const int rel = j * p.cd;
        return Entry{kv_own + rel, sc_own + rel, ape + rel, true, true};
    }
}
// Decode reads the state: low slots their overlap half, high slots their normal half
// (kvcompress.hip:340-349).
__device__ __forceinline__ Entry state_entry(const float* kv_state, const float* score_state,
                                             const CompGeom& p, int j) {
    const int half = (p.coff == 2 && j >= p.ratio) ? p.d : 0;
    const size_t src = (size_t)j * p.cd + half;
    return Entry{kv_state + src, score_state + src, nullptr, true, false};
}

// Softmax over the entries of VEC features starting at e, then the weighted sum
// (kvcompress.hip:117-150), from registers. Every load of the window is issued before the
// first is used: a masked entry (and a missing embedding) reads `safe` instead — any address
// that holds a feature row — and is dropped afterwards. A load under a condition, even a
// workgroup-uniform one, compiles to a branch that waits for its own data: one memory round
// trip per entry, one after the other.
template <int VEC, int SLOTS, class GetEntry>
__device__ __forceinline__ void pool_registers(GetEntry&& entry, const float* safe, int ents, int e,
                                               float (&out)[VEC]) {
    static_assert(SLOTS <= kCompRegEnts, "register windows are short");
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    float v[SLOTS][VEC], k[SLOTS][VEC];
    bool live[SLOTS];
    {
        vec_t s_raw[SLOTS], k_raw[SLOTS], a_raw[SLOTS];
        bool emb[SLOTS];
#pragma unroll
        for (int j = 0; j < SLOTS; ++j) {
            const Entry en = j < ents ? entry(j) : masked_entry();
            live[j] = en.live;
            emb[j] = en.live && en.emb;
            s_raw[j] = *reinterpret_cast<const vec_t*>((live[j] ? en.sc : safe) + e);
            k_raw[j] = *reinterpret_cast<const vec_t*>((live[j] ? en.kv : safe) + e);
            a_raw[j] = *reinterpret_cast<const vec_t*>((emb[j] ? en.ape : safe) + e);
        }
#pragma unroll
        for (int j = 0; j < SLOTS; ++j) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                v[j][i] = s_raw[j][i] + (emb[j] ? a_raw[j][i] : 0.0f);
                k[j][i] = k_raw[j][i];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < SLOTS; ++j)
            if (live[j]) mx = fmaxf(mx, v[j][i]);
        if (!isfinite(mx)) {  // every entry masked: a zero row, as the CPU statement has it
            out[i] = 0.0f;
            continue;
        }
        float ex[SLOTS], sum = 0.0f;
#pragma unroll
        for (int j = 0; j < SLOTS; ++j) {
            if (live[j]) {
                ex[j] = expf(v[j][i] - mx);
                sum += ex[j];
            }
        }
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < SLOTS; ++j)
            if (live[j]) acc += k[j][i] * (ex[j] / sum);
        out[i] = acc;
    }
}

// The same for wide windows: three sweeps over memory, one feature.
template <class GetEntry>
__device__ __forceinline__ float pool_streamed(GetEntry&& entry, int ents, int e) {
    float mx = -INFINITY;
    for (int j = 0; j < ents; ++j) {
        const Entry en = entry(j);
        if (!en.live) continue;
        mx = fmaxf(mx, en.sc[e] + (en.emb ? en.ape[e] : 0.0f));
    }
    if (!isfinite(mx)) return 0.0f;
    float sum = 0.0f;
    for (int j = 0; j < ents; ++j) {
        const Entry en = entry(j);
        if (!en.live) continue;
        sum += expf(en.sc[e] + (en.emb ? en.ape[e] : 0.0f) - mx);
    }
    float acc = 0.0f;
    for (int j = 0; j < ents; ++j) {
        const Entry en = entry(j);
        if (!en.live) continue;
        acc += en.kv[e] * (expf(en.sc[e] + (en.emb ? en.ape[e] : 0.0f) - mx) / sum);
    }
    return acc;
}

// Sum over the workgroup; red holds one word per wave. Every thread must call it.
__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int waves = (blockDim.x + kWave - 1) / kWave;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < waves; ++w) t += red[w];
    return t;
}

// Pool one row into LDS, finish it there (kvcompress.hip:176-203) and write it out.
// VEC == 4 requires d % 4 == 0 and 16-byte-aligned rows.
// SLOTS: 8 or 16 = the window is held in that many register slots; 0 = streamed.
template <int VEC, int SLOTS, class GetEntry>
__device__ __forceinline__ void compress_row(GetEntry&& entry, const float* safe, const CompFinish& f, float* out_row,
                                             int pos, int ents, const CompGeom& p, float* row, float* red) {
    const int tid = threadIdx.x, nthr = blockDim.x;
    // what the finishing steps read (this lane's first norm weights and rotation pair) is
    // requested now, with the window, instead of one round trip after each barrier
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    const float* t = f.freqs + (size_t)pos * p.rd;
    vec_t norm0 = 0.0f;
    float cos0 = 0.0f, sin0 = 0.0f;
    if (tid * VEC < p.d) norm0 = *reinterpret_cast<const vec_t*>(f.norm + tid * VEC);
    if (tid < p.rd / 2) {
        cos0 = t[2 * tid];
        sin0 = t[2 * tid + 1];
    }
    float ss = 0.0f;
    for (int e = tid * VEC; e < p.d; e += nthr * VEC) {
        float pooled[VEC];
        static_assert(VEC == 1 || VEC == 4, "one feature or four");
        if constexpr (SLOTS > 0) {
            pool_registers<VEC, SLOTS>(entry, safe, ents, e, pooled);
        } else {
#pragma unroll
            for (int i = 0; i < VEC; ++i) pooled[i] = pool_streamed(entry, ents, e + i);
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const float r = rbf16(pooled[i]);  // the bf16 store before the norm
            row[e + i] = r;
            ss += r * r;
        }
    }
    // 1/sqrt, not a reciprocal-square-root approximation: the factor multiplies the whole row
    const float rs = 1.0f / sqrtf(block_sum(ss, red) / (float)p.d + p.eps);
    for (int e = tid * VEC; e < p.d; e += nthr * VEC) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const float nw = e == tid * VEC ? norm0[i] : f.norm[e + i];
            row[e + i] = rbf16(nw * (row[e + i] * rs));
        }
    }
    __syncthreads();
    float* seg = row + (p.d - p.rd);
    for (int i = tid; i < p.rd / 2; i += nthr) {
        const float c = i == tid ? cos0 : t[2 * i], s = i == tid ? sin0 : t[2 * i + 1];
        const float a = seg[2 * i], b = seg[2 * i + 1];
        seg[2 * i] = rbf16(a * c - b * s);
        seg[2 * i + 1] = rbf16(a * s + b * c);
    }
    __syncthreads();
    // the closing bf16 store is the identity on the dims the rotation did not touch
    for (int e = tid * VEC; e < p.d; e += nthr * VEC) {
        if constexpr (VEC == 4) {
            *reinterpret_cast<f32x4*>(out_row + e) = *reinterpret_cast<const f32x4*>(row + e);
        } else {
            out_row[e] = row[e];
        }
    }
}

// A window held in registers wants a small workgroup; wide windows stream and want many lanes.
template <int VEC, int SLOTS, bool OVERLAP>
__global__ __launch_bounds__(SLOTS ? 256 : 1024) void kv_compress_prefill_kernel(const float* __restrict__ kv,
                                           const float* __restrict__ score,
                                           const float* __restrict__ ape, CompFinish f,
                                           CompGeom p) {
    extern __shared__ float lds[];
    float* row = lds;
    float* red = lds + p.d;
    const int b = blockIdx.x;
    const size_t own = (size_t)b * p.ratio * p.cd;
    const float* const kv_own = kv + own;
    const float* const sc_own = score + own;
    auto entry = [&](int j) { return prefill_entry<OVERLAP>(kv_own, sc_own, ape, p, b, j); };
    compress_row<VEC, SLOTS>(entry, score, f, f.out + (size_t)b * p.d, b * p.ratio,
                             OVERLAP ? 8 : p.ents, p, row, red);
}

// Names the kernel by its window shape alone, as the dispatch below does.
template <bool OVERLAP>
struct PrefillKernel {
    template <int VEC, int SLOTS>
    static constexpr auto fn = &kv_compress_prefill_kernel<VEC, SLOTS, OVERLAP>;
};

// One workgroup: its barriers order the pooling's reads against the window slide.
template <int VEC, int SLOTS>
__global__ __launch_bounds__(SLOTS ? 256 : 1024) void kv_compress_decode_kernel(float* kv_state, float* score_state, CompFinish f,
                                          CompGeom p, int start_pos) {
    extern __shared__ float lds[];
    float* row = lds;
    float* red = lds + p.d;
    auto entry = [&](int j) { return state_entry(kv_state, score_state, p, j); };
    // the block's first absolute position, not its index (kvcompress.hip:360-371)
    compress_row<VEC, SLOTS>(entry, score_state, f, f.out, (start_pos / p.ratio) * p.ratio, p.ents, p, row, red);
    __syncthreads();
    if (p.coff == 2) {
        // this block's normal half becomes the next block's overlap half
        const size_t n = (size_t)p.ratio * p.cd;
        for (size_t i = threadIdx.x; i < n; i += blockDim.x) {
            kv_state[i] = kv_state[n + i];
            score_state[i] = score_state[n + i];
        }
    }
}

// The state update every call makes before it pools (crates/backend/kernels/kvcompress.hip:
// 215-262; model.py:335-336): up to two runs of whole rows move from the call's kv / score
// rows into the state, the scores picking up the position embedding of their slot.
//   carry: on an overlapping layer, the last COMPLETE block of the call -> state rows
//          [0, ratio), embedding rows [0, ratio)            (prefill only: a call of >= ratio rows)
//   tail:  the rows after the last complete block -> state rows [state_off + slot0, ..),
//          embedding rows [slot0, ..)                       (a decode step is one tail row)
// Both runs are contiguous on both sides, so the launch is one flat range of VEC-float pieces,
// carry first, exactly as many threads as pieces, one 16-byte load per source and store per
// destination when VEC == 4.
struct DepositRun {
    size_t src, dst, emb, n;  // element offsets into kv/score, the state, ape; length
};
template <int VEC>
__global__ __launch_bounds__(256) void kv_compress_deposit_kernel(
    const float* __restrict__ kv, const float* __restrict__ score, const float* __restrict__ ape,
    float* __restrict__ kv_state, float* __restrict__ score_state, DepositRun carry, DepositRun tail) {
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    DepositRun r = carry;
    if (i >= carry.n) {
        i -= carry.n;
        r = tail;
        if (i >= tail.n) return;
    }
    const vec_t k = *reinterpret_cast<const vec_t*>(kv + r.src + i);
    const vec_t sc = *reinterpret_cast<const vec_t*>(score + r.src + i);
    const vec_t e = *reinterpret_cast<const vec_t*>(ape + r.emb + i);
    *reinterpret_cast<vec_t*>(kv_state + r.dst + i) = k;
    *reinterpret_cast<vec_t*>(score_state + r.dst + i) = sc + e;
}

// kvcompress.hip:386-405.
static int compress_guard(const CompGeom& p) {
    if (p.ratio <= 1 || p.d <= 0 || p.rd <= 0 || p.coff < 1 || p.coff > 2) return 1001;
    if (p.rd > p.d || (p.rd & 1)) return 1002;
    if (p.cd != p.coff * p.d || p.ents != p.coff * p.ratio) return 1003;
    if (p.ents > kCompEntsMax) return 1004;
    if ((p.coff == 2) != (p.ratio == 4)) return 1010;  // overlap is ratio 4 and nothing else
    return 0;
}

struct RowLaunch {
    bool vec, reg;
    unsigned threads;
    size_t lds;
};
static RowLaunch row_launch(const CompGeom& p, bool aligned) {
    RowLaunch r;
    r.reg = p.ents <= kCompRegEnts;
    // registers hold a short window for four features per lane; a wide one streams, one
    // feature per lane, so that more lanes share the latency
    r.vec = r.reg && aligned && p.d % 4 == 0;
    const int per_lane = r.vec ? 4 : 1, cap = r.reg ? 256 : 1024;
    const int threads = ((p.d + per_lane - 1) / per_lane + kWave - 1) / kWave * kWave;
    r.threads = (unsigned)(threads > cap ? cap : threads);
    r.lds = ((size_t)p.d + 16) * sizeof(float);
    return r;
}

// The instantiations in use: four features per lane with 8 or 16 register slots, one feature
// per lane with 16, one feature per lane streamed.
#define RK_COMPRESS_DISPATCH(KERNEL, GRID, R, ENTS, STREAM, ...)                                  \
    do {                                                                                          \
        if ((R).vec && (ENTS) <= 8)                                                               \
            hipLaunchKernelGGL((KERNEL<4, 8>), GRID, dim3((R).threads), (R).lds, STREAM,          \
                               __VA_ARGS__);                                                      \
        else if ((R).vec)                                                                         \
            hipLaunchKernelGGL((KERNEL<4, 16>), GRID, dim3((R).threads), (R).lds, STREAM,         \
                               __VA_ARGS__);                                                      \
        else if ((R).reg)                                                                         \
            hipLaunchKernelGGL((KERNEL<1, 16>), GRID, dim3((R).threads), (R).lds, STREAM,         \
                               __VA_ARGS__);                                                      \
        else                                                                                      \
            hipLaunchKernelGGL((KERNEL<1, 0>), GRID, dim3((R).threads), (R).lds, STREAM,          \
                               __VA_ARGS__);                                                      \
    } while (0)

}  // namespace rk

extern "C" int rivoli_kv_compress_deposit(const float* kv, const float* score, const float* ape,
                                          float* kv_state, float* score_state,
                                          const rivoli_comp_geom* pp, int s, int slot0,
                                          void* stream) {
    if (!pp) return 1000;
    const rk::CompGeom p = *pp;
    if (int g = rk::compress_guard(p)) return g;
    if (!kv || !score || !ape || !kv_state || !score_state) return 1001;
    if (s <= 0) return 1005;
    if (slot0 < 0 || slot0 + s % p.ratio > p.ratio) return 1008;
    (void)hipGetLastError();
    const int rem = s % p.ratio, cutoff = s - rem;
    const size_t cd = (size_t)p.cd;
    rk::DepositRun carry = {0, 0, 0, 0}, tail = {0, 0, 0, 0};
    if (p.coff == 2 && cutoff >= p.ratio) carry = {(size_t)(cutoff - p.ratio) * cd, 0, 0, (size_t)p.ratio * cd};
    if (rem > 0)
        tail = {(size_t)cutoff * cd, (size_t)((p.coff == 2 ? p.ratio : 0) + slot0) * cd, (size_t)slot0 * cd,
                (size_t)rem * cd};
    if (carry.n + tail.n == 0) return 0;  // whole blocks on a layer without overlap: nothing to keep
    const bool vec = (p.cd % 4) == 0 && rk::aligned16(kv) && rk::aligned16(score) && rk::aligned16(ape) &&
                     rk::aligned16(kv_state) && rk::aligned16(score_state);
    const size_t pieces = (carry.n + tail.n) / (vec ? 4 : 1);
    const dim3 grid((unsigned)((pieces + 255) / 256));
    if (vec)
        hipLaunchKernelGGL(rk::kv_compress_deposit_kernel<4>, grid, dim3(256), 0, (hipStream_t)stream, kv, score,
                           ape, kv_state, score_state, carry, tail);
    else
        hipLaunchKernelGGL(rk::kv_compress_deposit_kernel<1>, grid, dim3(256), 0, (hipStream_t)stream, kv, score,
                           ape, kv_state, score_state, carry, tail);
    return rk::launch_status();
}

extern "C" int rivoli_kv_compress_prefill(const float* kv, const float* score, const float* ape,
                                          const rivoli_comp_finish* ff, const rivoli_comp_geom* pp,
                                          int nblk, void* stream) {
    if (!pp || !ff) return 1000;
    const rk::CompGeom p = *pp;
    if (int g = rk::compress_guard(p)) return g;
    if (!kv || !score || !ape || !ff->norm || !ff->freqs || !ff->out) return 1001;
    if (p.d > rk::kCompMaxD) return 1002;
    // refused, not a silent success: the caller believed a block would be emitted
    if (nblk <= 0) return 1006;
    const bool aligned = rk::aligned16(kv) && rk::aligned16(score) && rk::aligned16(ape) &&
                         rk::aligned16(ff->out);
    const rk::RowLaunch r = rk::row_launch(p, aligned);
    (void)hipGetLastError();
    if (p.coff == 2)
        RK_COMPRESS_DISPATCH(rk::PrefillKernel<true>::fn, dim3((unsigned)nblk), r, p.ents,
                             (hipStream_t)stream, kv, score, ape, *ff, p);
    else
        RK_COMPRESS_DISPATCH(rk::PrefillKernel<false>::fn, dim3((unsigned)nblk), r, p.ents,
                             (hipStream_t)stream, kv, score, ape, *ff, p);
    return rk::launch_status();
}

extern "C" int rivoli_kv_compress_decode(float* kv_state, float* score_state,
                                         const rivoli_comp_finish* ff, const rivoli_comp_geom* pp,
                                         int start_pos, void* stream) {
    if (!pp || !ff) return 1000;
    const rk::CompGeom p = *pp;
    if (int g = rk::compress_guard(p)) return g;
    if (!kv_state || !score_state || !ff->norm || !ff->freqs || !ff->out) return 1001;
    if (p.d > rk::kCompMaxD) return 1002;
    if (start_pos <= 0) return 1007;  // position 0 is the prefill path
    // only a position that COMPLETES a block may pool: a half-filled window still gives
    // finite, plausible numbers
    if ((start_pos + 1) % p.ratio != 0) return 1009;
    const bool aligned = rk::aligned16(kv_state) && rk::aligned16(score_state) &&
                         rk::aligned16(ff->out);
    const rk::RowLaunch r = rk::row_launch(p, aligned);
    (void)hipGetLastError();
    RK_COMPRESS_DISPATCH(rk::kv_compress_decode_kernel, dim3(1), r, p.ents, (hipStream_t)stream,
                         kv_state, score_state, *ff, p, start_pos);
    return rk::launch_status();
}
