// Scalar formulas of the Mamba-3 layer step shared by the engine's kernels (src/mamba3_siso/cpu/inference.rs:68-258).
#pragma once
#include "common.hpp"

namespace mrs {

// a mod 2 pi in [0, 2 pi) (src/mamba3_siso/cpu/inference.rs:179-180 divides; an f64 division is a ~30-instruction
// dependent sequence and this sits in a serial chain over time, so the quotient comes from the reciprocal and the
// rare off-by-one of its floor is folded back).
__device__ __forceinline__ double wrap_2pi(double a) {
    const double two_pi = 6.283185307179586, inv_two_pi = 0.15915494309189535;
    double r = fma(-two_pi, floor(a * inv_two_pi), a);
    r = r < 0.0 ? r + two_pi : r;
    return r >= two_pi ? r - two_pi : r;
}


constexpr float kPi = 3.14159265358979323846f;

__device__ __forceinline__ float heavy_tail(float x) { return x >= 0.0f ? 1.0f + x : 1.0f / (1.0f - x); }
__device__ __forceinline__ float sigmoidf_fast(float x) { return fast_rcp(1.0f + fast_exp2(-x * kLog2e)); }

}  // namespace mrs
