// v_mfma_f32_16x16x32 on 16-byte operand pieces: lane l brings A[m = l % 16][k = 8 (l / 16) .. +7] and
// B[k = 8 (l / 16) .. +7][n = l % 16]; result register i of lane l is C[m = 4 (l / 16) + i][n = l % 16].
#pragma once
#include "common.hpp"

namespace mrs {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

template <typename T> struct Mma32;
template <> struct Mma32<bf16_t> {
    __device__ static __forceinline__ v4f mma(uint4 a, uint4 b, v4f c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
    }
};
template <> struct Mma32<f16_t> {
    __device__ static __forceinline__ v4f mma(uint4 a, uint4 b, v4f c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
    }
};

}  // namespace mrs
