// The sliding-window ring of the second cache format: rows [0, win) of a layer's
// [ring | compressed] cache, slot t % win holding position t
// (crates/engine/src/v4/attn.rs:332-378 write_ring, which issues one or two device copies per
// call). One launch here: a decode step copies its single row into slot start_pos % win; a
// prompt of s <= win rows seeds slots [0, s); a longer prompt seeds every slot from its last
// win rows. Launch-only.
#include "codec.hpp"

namespace rk {

// One workgroup per copied row. `first` is the position of the first copied row and `src_row0`
// its row in kv.
template <class T>
__global__ __launch_bounds__(256) void kv_ring_write_kernel(const T* __restrict__ kv,
                                                            T* __restrict__ cache, int win,
                                                            int row_elems, int first,
                                                            int src_row0) {
    const int r = blockIdx.x;
    const T* src = kv + (size_t)(src_row0 + r) * row_elems;
    T* dst = cache + (size_t)((first + r) % win) * row_elems;
    for (int i = threadIdx.x; i < row_elems; i += 256) dst[i] = src[i];
}

}  // namespace rk

extern "C" int rivoli_kv_ring_write(const float* kv, float* cache, int win, int hd, int seqlen,
                                    int start_pos, void* stream) {
    if (!kv || !cache || win <= 0 || hd <= 0 || seqlen <= 0 || start_pos < 0) return 1001;
    if (start_pos != 0 && seqlen != 1) return 1005;
    // positions [first, first + n) are copied; kv row of position p is p at prefill, 0 at decode
    const int n = start_pos != 0 ? 1 : (seqlen < win ? seqlen : win);
    const int first = start_pos != 0 ? start_pos : seqlen - n;
    const int src_row0 = start_pos != 0 ? 0 : first;
    (void)hipGetLastError();
    const bool wide = hd % 4 == 0 && ((uintptr_t)kv | (uintptr_t)cache) % 16 == 0;
    if (wide)
        hipLaunchKernelGGL(rk::kv_ring_write_kernel<rk::u32x4>, dim3((unsigned)n), dim3(256), 0,
                           (hipStream_t)stream, reinterpret_cast<const rk::u32x4*>(kv),
                           reinterpret_cast<rk::u32x4*>(cache), win, hd / 4, first, src_row0);
    else
        hipLaunchKernelGGL(rk::kv_ring_write_kernel<float>, dim3((unsigned)n), dim3(256), 0,
                           (hipStream_t)stream, kv, cache, win, hd, first, src_row0);
    return rk::launch_status();
}
