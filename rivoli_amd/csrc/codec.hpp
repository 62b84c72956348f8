// Device element codecs and wave64 helpers for the fp8 KV-cache kernels (gfx950 only).
//
// Arithmetic contract (must stay bit-identical to rivoli_core::num, crates/core/src/num.rs):
//   * e4m3 encode: round to nearest even on normals, round HALF AWAY from zero in the
//     subnormal band, saturate |x| >= 448 to 0x7e, |x| < 2^-10 to signed zero, NaN -> 0x7f.
//     gfx950's v_cvt_pk_fp8_f32 is nearest-even everywhere, so it is used only where the two
//     rules coincide; the rest goes through the integer form.
//   * e4m3 decode is exact; gfx950's v_cvt_pk_f32_fp8 decodes OCP e4m3 and is used as is.
//   * bf16 encode is round to nearest even; gfx950's v_cvt_pk_bf16_f32 does exactly that.
//   * scale = amax > 0 ? amax / 448 : 1 and v / scale are IEEE-correct f32 divides (hipcc's
//     default); nothing here may be built with fast-math.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rk {

constexpr int kWave = 64;

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_lo_to_f32(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi_to_f32(uint32_t pair) {
    return __uint_as_float(pair & 0xffff0000u);
}

// Two f32 -> two bf16 packed (lo in the low half), round to nearest even.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    bf16x2 p = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, p);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float x) {
    __bf16 h = (__bf16)x;
    return __builtin_bit_cast(uint16_t, h);
}

// f32 -> OCP e4m3 byte, the KV-cache rule (crates/core/src/num.rs:128-182; device twin in the
// reference at crates/backend/kernels/fwd.hip:20-45), in integer arithmetic: the software
// form, valid for every input.
__device__ __forceinline__ uint32_t f32_to_e4m3_sw(float x) {
    uint32_t xb = __float_as_uint(x);
    uint32_t sign = (xb >> 24) & 0x80u;
    uint32_t ab = xb & 0x7fffffffu;
    float a = __uint_as_float(ab);
    // normal path: keep 3 mantissa bits, nearest even over the 20 dropped ones. Adding
    // 0x7ffff + lsb carries into the exponent field by itself when the mantissa wraps.
    uint32_t r = ab + 0x0007ffffu + ((ab >> 20) & 1u);
    uint32_t normal = (r >> 20) - (120u << 3);  // exponent rebias 127 -> 7
    // subnormal band [2^-10, 2^-6): m = floor(a*512 + 0.5); m == 8 is code 0x08 by itself.
    uint32_t sub = (uint32_t)(a * 512.0f + 0.5f);
    uint32_t mag = a < 0.015625f ? sub : normal;
    mag = a < 0.0009765625f ? 0u : mag;
    mag = a >= 448.0f ? 0x7eu : mag;  // also catches +-inf
    uint32_t code = sign | mag;
    return ab > 0x7f800000u ? 0x7fu : code;
}

// Two / four values through gfx950's v_cvt_pk_fp8_f32 (OCP e4m3, round to nearest even
// everywhere). It agrees with the KV-cache rule exactly where that rule is nearest-even and
// does not saturate: 2^-6 <= |x| < 464 (448..464 rounds down to 448), and at +-0. It differs
// on subnormal-band ties (the rule rounds those half AWAY), so callers route |x| < 2^-6,
// |x| >= 464 and NaN to the software form.
__device__ __forceinline__ uint32_t e4m3x4_hw(float q0, float q1, float q2, float q3) {
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(q0, q1, 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(q2, q3, w, true);
    return (uint32_t)w;
}
__device__ __forceinline__ bool e4m3_hw_exact_domain(float x) {
    const float a = fabsf(x);
    return (a >= 0.015625f && a < 464.0f) || a == 0.0f;  // false for NaN
}

// The rule for one value: hardware conversion inside its exact domain, software outside.
__device__ __forceinline__ uint32_t f32_to_e4m3(float x) {
    if (e4m3_hw_exact_domain(x)) return e4m3x4_hw(x, 0.0f, 0.0f, 0.0f) & 0xffu;
    return f32_to_e4m3_sw(x);
}

// The append quantizer divides by the row scale before encoding: code = rule(RN(x / scl)).
// A correctly rounded divide costs ~11 instructions; the fast path gets the same quotient in
// three: with y = RN(1 / scl) (one divide per row), q0 = RN(x * y), r = fma(-q0, scl, x) (the
// exact residual) and q = fma(r, y, q0), q IS RN(x / scl) (Markstein's correction of a
// reciprocal product). x is a bf16 and scl = RN(amax / 448) with amax a bf16, so the claim
// depends only on two 8-bit mantissas and the exponent gap: it was checked over all of them in
// exact rational arithmetic, and the device is checked the same way against the oracle's divide
// (every amax mantissa against every value below it). It needs the residual to stay a normal
// number, which row_scale_is_fast guarantees. With the exact quotient in hand, gfx950's
// v_cvt_pk_fp8_f32 (nearest even everywhere) is the reference's encoder wherever that one is
// nearest-even too: 2^-6 <= |q| (|q| <= 448 * (1 + 2^-22) always, since |x| <= amax) or q == 0.
// A chunk with a quotient in the subnormal band (the reference rounds those ties AWAY), or a
// NaN, takes the divide and the integer encoder.
__device__ __forceinline__ bool row_scale_is_fast(float scl) { return scl >= 1e-20f && scl <= 1e20f; }

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

// The band test is made on the inputs, where it is a packed 16-bit compare: q < 2^-6 needs
// |x| < scl * 2^-6, and |bf16| patterns order like their values, so every such x has a pattern
// <= T = bits(scl * 2^-6) >> 16. A chunk is sent to the exact path when some non-zero |x| has a
// pattern <= T + 1 (one pattern of slack; the exact path is right for any input). A row whose
// scale is not fast gets the band 0x10000, which every pattern is below.
__device__ __forceinline__ uint32_t row_band(float scl) {
    return row_scale_is_fast(scl) ? (__float_as_uint(scl * 0.015625f) >> 16) + 1u : 0x10000u;
}

// Eight consecutive bf16 (four dwords) -> eight e4m3 codes (two dwords) under one row scale.
// Per two elements the test costs an AND, a packed subtract, a packed min and a packed max:
//   some 0 < |x| pattern <= band - 1   <=> min over (|pattern| - 1, wrapping zero to 0xffff) < band
//   some NaN                           <=> max over |pattern| > 0x7f80
__device__ __forceinline__ u32x2 quantize8(const uint32_t (&w)[4], float scl, float rinv,
                                           uint32_t band) {
    u16x2 low = {0xffff, 0xffff}, top = {0, 0};
    const u16x2 one = {1, 1};
    float x[8], q[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u16x2 mag = __builtin_bit_cast(u16x2, w[i] & 0x7fff7fffu);
        low = __builtin_elementwise_min(low, mag - one);
        top = __builtin_elementwise_max(top, mag);
        x[2 * i] = bf16_lo_to_f32(w[i]);
        x[2 * i + 1] = bf16_hi_to_f32(w[i]);
    }
    const bool exact = (uint32_t)min(low.x, low.y) < band || max(top.x, top.y) > 0x7f80;
    if (!exact) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float q0 = x[i] * rinv;
            // q0 - (q0 * scl - x) * rinv: the residual with this sign keeps a -0.0 input -0.0
            q[i] = __builtin_fmaf(-__builtin_fmaf(q0, scl, -x[i]), rinv, q0);
        }
        u32x2 r = {e4m3x4_hw(q[0], q[1], q[2], q[3]), e4m3x4_hw(q[4], q[5], q[6], q[7])};
        return r;
    }
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        lo |= f32_to_e4m3_sw(x[i] / scl) << (8 * i);
        hi |= f32_to_e4m3_sw(x[4 + i] / scl) << (8 * i);
    }
    u32x2 r = {lo, hi};
    return r;
}

// Four packed e4m3 codes -> four f32, exact.
__device__ __forceinline__ void e4m3x4_to_f32(uint32_t w, float (&v)[4]) {
    f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
    f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
    v[0] = lo.x;
    v[1] = lo.y;
    v[2] = hi.x;
    v[3] = hi.y;
}

// Four packed e4m3 codes times one scale -> four bf16 in two dwords.
__device__ __forceinline__ u32x2 dequant4_bf16(uint32_t w, float scale) {
    float v[4];
    e4m3x4_to_f32(w, v);
    u32x2 r = {pack_bf16x2(v[0] * scale, v[1] * scale), pack_bf16x2(v[2] * scale, v[3] * scale)};
    return r;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}
__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
// A workgroup barrier that orders LDS traffic only. __syncthreads() also waits for every global
// load and store the wave has in flight (a full memory round trip when a store was just issued);
// where only LDS contents are handed between waves, that wait is pure latency.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Inclusive prefix sum over the 64 lanes on the DPP path: four shifts inside each row of 16
// lanes, then the two row broadcasts (lane 15 of a row into the next row, lane 31 into the
// upper half). A step is one ALU instruction; the generic cross-lane shuffle goes through the
// LDS crossbar and costs an LDS round trip per step.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_or_zero(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ uint32_t wave_inclusive_sum(uint32_t v) {
    v += dpp_or_zero<0x111, 0xf>(v);  // row_shr:1
    v += dpp_or_zero<0x112, 0xf>(v);  // row_shr:2
    v += dpp_or_zero<0x114, 0xf>(v);  // row_shr:4
    v += dpp_or_zero<0x118, 0xf>(v);  // row_shr:8
    v += dpp_or_zero<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
    v += dpp_or_zero<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}
// The sum over the wave, as a scalar.
__device__ __forceinline__ uint32_t wave_total(uint32_t inclusive) {
    return (uint32_t)__builtin_amdgcn_readlane((int)inclusive, kWave - 1);
}
__device__ __forceinline__ unsigned long long wave_xor(unsigned long long v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v ^= __shfl_xor(v, off, kWave);
    return v;
}

// The vector loads and stores of these kernels are 16 bytes wide: a launcher refuses (1004) a
// buffer that is not 16-byte aligned rather than let the kernel fault on it.
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Launcher epilogue shared by every entry point: 0 or -(hipError_t).
inline int launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : -(int)e;
}

}  // namespace rk
