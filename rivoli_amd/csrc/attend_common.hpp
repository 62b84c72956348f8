// Pieces the attention kernels share: operand vector types, typed LDS pointers, the
// reductions over the four 16-lane rows of a wave, and the order in which a 32-token tile's
// tokens sit in the value contraction.
#pragma once
#include "codec.hpp"

namespace rk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <class T>
using lds_ptr = __attribute__((address_space(3))) T*;

constexpr float kLazyRescale = 8.0f;       // log2 units
constexpr float kLog2e = 1.4426950408889634f;

// max / sum of a value over the four 16-lane rows of the wave, in every lane. gfx950's row
// swaps stay in the vector ALU; the generic cross-lane shuffle goes through the LDS crossbar.
__device__ __forceinline__ float rows_max(float x) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));  // rows {0,1} and {2,3} paired
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float rows_sum(float x) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// In the score tile (rows = tokens, 16 per MFMA) a lane of row group g holds rows 4g..4g+3
// of both 16-token halves, and those 8 values are element j = 4*half + i of the value MFMA's
// A operand for contraction index 8g + j. Staging wave w (of 8) owns contraction indices
// 4w..4w+3 — tile positions 16*(w&1) + 4*(w>>1) + i, four consecutive tokens.
__device__ __forceinline__ int tile_pos_of(int wave, int i) { return 16 * (wave & 1) + 4 * (wave >> 1) + i; }

}  // namespace rk
