// Block activation quantization of the second cache format: the fused quantize-then-
// dequantize that leaves "what fp8 arithmetic produces" in an f32 row
// (crates/backend/kernels/mla.hip:319-338, launcher :527-548; arithmetic in
// crates/backend/kernels/actquant.hpp:69-101 and formats.hpp:245-264; CPU statement
// crates/oracles/src/v4oracle/numerics.rs:245-285). The cache entry runs it over dims
// [0, n) at block 64 and leaves the rotated tail [n, row_stride) alone.
//
// Per block: amax = max(1e-4, |x_i|); s = 2^ceil(log2(amax * (1/448))) by exponent surgery;
// out_i = decode(encode_rne(clamp(x_i / s, +-448))) * s. Bit-exact by construction:
//   * s is a power of two, so x / s is x times the exact reciprocal 2^-e (one IEEE multiply
//     gives the same correctly rounded result as the divide; the divide itself is kept for the
//     out-of-contract amax = inf, whose s = inf has no such reciprocal);
//   * the reference's encoder is round-to-nearest-even everywhere, subnormals included, with
//     NaN -> 0x7f: exactly gfx950's v_cvt_pk_fp8_f32 once the value is clamped to +-448, and
//     the decode is v_cvt_pk_f32_fp8, exact;
//   * the clamp is written with comparisons so a NaN stays a NaN (actquant.hpp:90-99).
//
// Shape: the reference gives each block to one thread that walks it twice. Here a lane owns
// four consecutive values (one 16-byte load and store, coalesced across the wave), block / 4
// neighbouring lanes reduce the amax by cross-lane maxima, and every thread has several
// independent blocks in flight. 8 bytes of traffic per element: HBM-bound.
#include "codec.hpp"

namespace rk {

constexpr float kFp8Max = 448.0f;
constexpr float kFp8MaxInv = 1.0f / 448.0f;
constexpr float kAmaxFloor = 1e-4f;
constexpr int kAqThreads = 256;
constexpr int kAqInFlight = 4;  // 16-byte pieces per thread

typedef float f32x4 __attribute__((ext_vector_type(4)));

// actquant.hpp:69-81: the exponent field of amax * max_inv, plus one when the mantissa is
// not zero, rebuilt as a bare power of two.
__device__ __forceinline__ int round_scale_exponent(float amax) {
    const uint32_t b = __float_as_uint(amax * kFp8MaxInv);
    return (int)((b >> 23) & 0xffu) - 127 + ((b & 0x7fffffu) ? 1 : 0);
}

struct BlockScale {
    float s;     // 2^e
    float rinv;  // 2^-e when usable
    bool mul;    // x * rinv is exact; otherwise divide by s
};
__device__ __forceinline__ BlockScale block_scale(float amax) {
    const int e = round_scale_exponent(amax);
    BlockScale r;
    r.s = __uint_as_float((uint32_t)(e + 127) << 23);
    r.mul = e >= -126 && e <= 126;
    r.rinv = __uint_as_float((uint32_t)(127 - e) << 23);
    return r;
}

__device__ __forceinline__ float clamp_keep_nan(float q) {
    return q < -kFp8Max ? -kFp8Max : (q > kFp8Max ? kFp8Max : q);
}

__device__ __forceinline__ f32x4 roundtrip4(f32x4 x, BlockScale sc) {
    float q[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = clamp_keep_nan(sc.mul ? x[i] * sc.rinv : x[i] / sc.s);
    float v[4];
    e4m3x4_to_f32(e4m3x4_hw(q[0], q[1], q[2], q[3]), v);
    f32x4 r = {v[0] * sc.s, v[1] * sc.s, v[2] * sc.s, v[3] * sc.s};
    return r;
}

// LANES = block / 4 lanes share one block; LANES is a power of two <= 64 so a block never
// straddles a wave. Piece p of the launch is 16 bytes: block p / LANES, lane p % LANES.
template <int LANES>
__global__ __launch_bounds__(kAqThreads) void act_quant_kernel(const float* src, float* dst,
                                                               uint32_t n_pieces, uint32_t nb,
                                                               uint32_t row_stride) {
    const uint32_t stride = gridDim.x * kAqThreads;
    // 64-bit walk so that p0 + j * stride cannot wrap; everything live is below n_pieces
    for (unsigned long long p0 = blockIdx.x * kAqThreads + threadIdx.x; p0 < n_pieces;
         p0 += (unsigned long long)stride * kAqInFlight) {
        f32x4 x[kAqInFlight];
        size_t off[kAqInFlight];
        bool live[kAqInFlight];
#pragma unroll
        for (int j = 0; j < kAqInFlight; ++j) {
            const unsigned long long p = p0 + (unsigned long long)j * stride;
            live[j] = p < n_pieces;
            const uint32_t p32 = live[j] ? (uint32_t)p : 0u;
            const uint32_t blk = p32 / LANES, lane = p32 % LANES;
            off[j] = (size_t)(blk / nb) * row_stride + (size_t)(blk % nb) * (LANES * 4) + lane * 4;
            x[j] = live[j] ? *reinterpret_cast<const f32x4*>(src + off[j]) : f32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int j = 0; j < kAqInFlight; ++j) {
            // n_pieces is a multiple of LANES and the launch strides by a multiple of 64, so
            // the LANES lanes of one block are live, or not, together
            float amax = fmaxf(fmaxf(fabsf(x[j][0]), fabsf(x[j][1])),
                               fmaxf(fabsf(x[j][2]), fabsf(x[j][3])));
            amax = fmaxf(amax, kAmaxFloor);
#pragma unroll
            for (int o = LANES / 2; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, kWave));
            const f32x4 y = roundtrip4(x[j], block_scale(amax));
            if (live[j]) *reinterpret_cast<f32x4*>(dst + off[j]) = y;
        }
    }
}

// Any block size and alignment: one thread per block, as the reference does it.
__global__ __launch_bounds__(kAqThreads) void act_quant_serial_kernel(const float* src, float* dst,
                                                                      long long n_blocks, int nb,
                                                                      int row_stride, int block) {
    const long long id = (long long)blockIdx.x * kAqThreads + threadIdx.x;
    if (id >= n_blocks) return;
    const size_t off = (size_t)(id / nb) * row_stride + (size_t)(id % nb) * block;
    float amax = kAmaxFloor;
    for (int i = 0; i < block; ++i) amax = fmaxf(amax, fabsf(src[off + i]));
    const BlockScale sc = block_scale(amax);
    for (int i = 0; i < block; ++i) {
        const float x = src[off + i];
        const float q = clamp_keep_nan(sc.mul ? x * sc.rinv : x / sc.s);
        float v[4];
        e4m3x4_to_f32(e4m3x4_hw(q, 0.0f, 0.0f, 0.0f), v);
        dst[off + i] = v[0] * sc.s;
    }
}

template <int LANES>
static void launch_act_quant(const float* src, float* dst, long long n_blocks, int nb,
                             int row_stride, hipStream_t stream) {
    const long long n_pieces = n_blocks * LANES;  // the caller keeps this below 2^32
    const long long per_group = (long long)kAqThreads * kAqInFlight;
    long long groups = (n_pieces + per_group - 1) / per_group;
    if (groups > 256 * 16) groups = 256 * 16;
    hipLaunchKernelGGL(act_quant_kernel<LANES>, dim3((unsigned)groups), dim3(kAqThreads), 0, stream,
                       src, dst, (uint32_t)n_pieces, (uint32_t)nb, (uint32_t)row_stride);
}

}  // namespace rk

extern "C" int rivoli_act_quant_f8_prefix(const float* src, float* dst, int rows, int row_stride,
                                          int n, int block, void* stream) {
    if (!src || !dst) return 1001;
    if (rows <= 0 || n <= 0 || block <= 0 || row_stride < n) return 1001;
    // a quantize-from-source that covers part of the row would leave the rest of dst stale
    if (src != dst && n != row_stride) return 1002;
    if (n % block) return 1004;
    const int nb = n / block;
    const long long n_blocks = (long long)rows * nb;
    if ((long long)rows * n > 0xffffffffLL) return 1002;  // pieces and blocks are counted in 32 bits
    hipStream_t st = (hipStream_t)stream;
    (void)hipGetLastError();
    const bool vec = block % 4 == 0 && row_stride % 4 == 0 && rk::aligned16(src) && rk::aligned16(dst);
    switch (vec ? block : 0) {
        case 16: rk::launch_act_quant<4>(src, dst, n_blocks, nb, row_stride, st); break;
        case 32: rk::launch_act_quant<8>(src, dst, n_blocks, nb, row_stride, st); break;
        case 64: rk::launch_act_quant<16>(src, dst, n_blocks, nb, row_stride, st); break;
        case 128: rk::launch_act_quant<32>(src, dst, n_blocks, nb, row_stride, st); break;
        case 256: rk::launch_act_quant<64>(src, dst, n_blocks, nb, row_stride, st); break;
        default: {
            const long long groups = (n_blocks + rk::kAqThreads - 1) / rk::kAqThreads;
            hipLaunchKernelGGL(rk::act_quant_serial_kernel, dim3((unsigned)groups),
                               dim3(rk::kAqThreads), 0, st, src, dst, n_blocks, nb, row_stride,
                               block);
        }
    }
    return rk::launch_status();
}
