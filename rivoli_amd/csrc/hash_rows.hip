// XOR fold of a buffer's exact bits, and the element codecs as standalone launchers.
//
// hash_rows is the device twin of rivoli_core::hash::xor_fold_strided
// (crates/core/src/hash.rs:68-112; reference kernel crates/backend/kernels/fwd.hip:358-427):
//   *out ^= XOR_i splitmix64_finalize(((i_base + i) << 32) ^ bits(x[i])),  i = 0, stride, ...
// XOR is commutative and associative, so the fold does not depend on the schedule: lanes fold
// their own samples, a wave butterfly and a 4-entry LDS step reduce the workgroup, and one
// atomic per workgroup lands in *out. It is how results far larger than a host copy are held
// bit-exact against the CPU rule.
// Launch-only; see include/rivoli_kvcache.h for the contract of every entry point.
#include "codec.hpp"

namespace rk {

constexpr int kHashThreads = 256;

__device__ __forceinline__ unsigned long long splitmix_finalize(unsigned long long z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__global__ __launch_bounds__(kHashThreads) void hash_rows_kernel(
    const uint32_t* __restrict__ x, long long n, long long stride, unsigned long long i_base,
    unsigned long long* __restrict__ out) {
    __shared__ unsigned long long red[kHashThreads / kWave];
    const long long samples = (n + stride - 1) / stride;
    unsigned long long acc = 0;
    for (long long si = (long long)blockIdx.x * kHashThreads + threadIdx.x; si < samples;
         si += (long long)kHashThreads * gridDim.x) {
        const long long i = si * stride;
        acc ^= splitmix_finalize(((i_base + (unsigned long long)i) << 32) ^
                                 (unsigned long long)x[i]);
    }
    acc = wave_xor(acc);
    if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long h = red[0];
#pragma unroll
        for (int w = 1; w < kHashThreads / kWave; ++w) h ^= red[w];
        atomicXor(out, h);
    }
}

__global__ void e4m3_encode_kernel(const float* __restrict__ x, uint8_t* __restrict__ out,
                                   long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long step = (long long)gridDim.x * blockDim.x;
    for (; i < n; i += step) out[i] = (uint8_t)f32_to_e4m3(x[i]);
}

__global__ void bf16_encode_kernel(const float* __restrict__ x, uint16_t* __restrict__ out,
                                   long long n) {
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long step = (long long)gridDim.x * blockDim.x;
    for (; i < n; i += step) out[i] = f32_to_bf16(x[i]);
}

static inline unsigned capped_blocks(long long n, int threads, long long cap) {
    long long b = (n + threads - 1) / threads;
    return (unsigned)(b > cap ? cap : b);
}

}  // namespace rk

extern "C" int rivoli_hash_rows(const float* x, int n, int stride, unsigned long long i_base,
                                unsigned long long* out, void* stream) {
    using namespace rk;
    if (n <= 0 || stride <= 0 || !x || !out) return 1001;
    const long long samples = ((long long)n + stride - 1) / stride;
    (void)hipGetLastError();
    // Grid-stride over samples with a capped grid: one atomic per workgroup, so the cap
    // bounds the atomics whatever n is; 2048 workgroups is 8 per CU on 256 CUs.
    hipLaunchKernelGGL(hash_rows_kernel, dim3(capped_blocks(samples, kHashThreads, 2048)),
                       dim3(kHashThreads), 0, (hipStream_t)stream,
                       reinterpret_cast<const uint32_t*>(x), (long long)n, (long long)stride,
                       i_base, out);
    return launch_status();
}

extern "C" int rivoli_codec_e4m3_encode(const float* x, unsigned char* out, long long n,
                                        void* stream) {
    if (!x || !out || n <= 0) return 1001;
    (void)hipGetLastError();
    hipLaunchKernelGGL(rk::e4m3_encode_kernel, dim3(rk::capped_blocks(n, 256, 4096)), dim3(256), 0,
                       (hipStream_t)stream, x, out, n);
    return rk::launch_status();
}

extern "C" int rivoli_codec_bf16_encode(const float* x, unsigned short* out, long long n,
                                        void* stream) {
    if (!x || !out || n <= 0) return 1001;
    (void)hipGetLastError();
    hipLaunchKernelGGL(rk::bf16_encode_kernel, dim3(rk::capped_blocks(n, 256, 4096)), dim3(256), 0,
                       (hipStream_t)stream, x, out, n);
    return rk::launch_status();
}
