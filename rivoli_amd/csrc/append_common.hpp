// One wave64 quantizes and appends one token's row: the body of the small-batch paged append
// (kv_append.hip), shared with the gather kernel that also appends a decode step's new tokens
// (kv_gather.hip). Scale rule and encoder: crates/backend/kernels/fwd.hip:51-71.
#pragma once

#include "gather_common.hpp"

namespace rk {

// A lane holds 8 consecutive elements per step (one 16-byte load), so a 576-wide row is one
// full step plus an 8-lane tail; the amax is a register max plus a wave butterfly; no LDS, no
// barrier. STEPS = ceil(width / 512). `slot_at` points at the token's slot: negative = padding,
// >= n_slots = counted in *bad_slots, never written. With `out_row` (16-byte aligned) the row is
// also written there as bf16 exactly as a gather of the stored record would produce it:
// dequantized from the codes and the scale just made. Returns whether the token was stored.
// Every lane of the wave must call it.
template <int STEPS>
__device__ __forceinline__ bool append_token_wave(const uint16_t* __restrict__ row,
                                                  const int* __restrict__ slot_at,
                                                  uint8_t* __restrict__ pool, int width,
                                                  int page_tokens, long long n_slots,
                                                  size_t page_bytes,
                                                  unsigned int* __restrict__ bad_slots,
                                                  uint16_t* __restrict__ out_row) {
    const int lane = threadIdx.x & (kWave - 1);
    const int n_chunks = width >> 3;
    const u32x4* src = reinterpret_cast<const u32x4*>(row);
    // the row is requested before the slot is looked at: the two fetches overlap instead of
    // queueing one memory round trip behind the other (a padding token costs a wasted read)
    u32x4 raw[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        int c = lane + s * kWave;
        raw[s] = c < n_chunks ? __builtin_nontemporal_load(src + c) : u32x4{0, 0, 0, 0};
    }
    const int slot = *slot_at;
    if (slot < 0) return false;  // padding
    if ((long long)slot >= n_slots) {
        if (lane == 0 && bad_slots) atomicAdd(bad_slots, 1u);
        return false;
    }
    float amax = 0.0f;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        const uint32_t w[4] = {raw[s].x, raw[s].y, raw[s].z, raw[s].w};
#pragma unroll
        for (int i = 0; i < 4; ++i)
            amax = fmaxf(amax, fmaxf(fabsf(bf16_lo_to_f32(w[i])), fabsf(bf16_hi_to_f32(w[i]))));
    }
    amax = wave_max(amax);
    const float scl = amax > 0.0f ? amax / 448.0f : 1.0f;
    const float rinv = 1.0f / scl;
    const uint32_t band = row_band(scl);

    const int page = slot / page_tokens;
    const int off = slot - page * page_tokens;
    uint8_t* pg = pool + (size_t)page * page_bytes;
    u32x2* dst = reinterpret_cast<u32x2*>(pg + (size_t)off * width);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        int c = lane + s * kWave;
        if (c < n_chunks) {
            const uint32_t w[4] = {raw[s].x, raw[s].y, raw[s].z, raw[s].w};
            const u32x2 codes = quantize8(w, scl, rinv, band);
            dst[c] = codes;
            if (out_row) reinterpret_cast<u32x4*>(out_row)[c] = dequant8_bf16(codes, scl);
        }
    }
    if (lane == 0)
        *reinterpret_cast<float*>(pg + (size_t)page_tokens * width + (size_t)off * 4) = scl;
    return true;
}

}  // namespace rk
