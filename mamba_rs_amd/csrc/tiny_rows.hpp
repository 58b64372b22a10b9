// Building blocks of the single-launch backbone steps for small f32 models (tiny_step.hip, tiny_m3_step.hip): a workgroup
// walks one batch row through the whole network, its products are matrix-vector sweeps over weights that sit in L2.
#pragma once
#include "common.hpp"

namespace mrs {
namespace {

constexpr int kTinyThreads = 512;    // 8 waves: one float4 of SSM state per lane and pass at d_inner 256, d_state 16
constexpr int kTinyPre = 2;          // passes of the scan step whose state is requested at the top of the layer
constexpr int kTinySlices = 16;      // most k slices per product (their partial sums are added serially)
constexpr int kTinyPart = 2048;      // floats of k-slice partial sums: (N / 4 column quads) x (k slices) <= 512 threads x 4

// Every array carved out of the workgroup's LDS starts on a 16-byte boundary: some of them (the partial sums, K and Q of the
// Mamba-3 step) are read and written as float4, and an array in front of them whose length is not a multiple of four
// floats (an input row wider than d_model, an odd d_inner) would otherwise shift them off it.
__host__ __device__ constexpr int rup4(int n) { return (n + 3) & ~3; }

// out[n] = bias[n] + sum_k x[k] W[k][n] for n < N; W row-major [K][N] in global memory, x and out in LDS, N % 4 == 0 and
// N <= 2048.  A thread owns four consecutive columns over one slice of K (16-byte weight loads, consecutive lanes on
// consecutive quads, sixteen rows requested before the first multiply-add); the slices' partial sums meet in LDS and are
// added in slice order.
__device__ __forceinline__ void gemv_rows(const float *__restrict__ W, int K, int N, const float *x, float *out, float *part,
                                          const float *__restrict__ bias) {
    const int tid = threadIdx.x;
    const int nq = N >> 2;
    const int ks_n = min(kTinyThreads / nq, kTinySlices);   // k slices (>= 1)
    const int kper = (K + ks_n - 1) / ks_n;
    const int q = tid % nq, ks = tid / nq;
    if (ks < ks_n) {
        const int k0 = ks * kper, k1 = min(K, k0 + kper);
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        const float *wp = W + 4 * q;
        for (int kb = k0; kb < k1; kb += 16) {
            float4 w[16];
#pragma unroll
            for (int j = 0; j < 16; j++) w[j] = *reinterpret_cast<const float4 *>(wp + (int64_t)min(kb + j, k1 - 1) * N);   // rows past the slice re-read its last one
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const float xv = kb + j < k1 ? x[kb + j] : 0.0f;
                acc.x = fmaf(xv, w[j].x, acc.x); acc.y = fmaf(xv, w[j].y, acc.y); acc.z = fmaf(xv, w[j].z, acc.z); acc.w = fmaf(xv, w[j].w, acc.w);
            }
        }
        *reinterpret_cast<float4 *>(&part[ks * N + 4 * q]) = acc;
    }
    __syncthreads();
    for (int n = tid; n < N; n += kTinyThreads) {
        float s = bias ? bias[n] : 0.0f;
        for (int j = 0; j < ks_n; j++) s += part[j * N + n];
        out[n] = s;
    }
    __syncthreads();
}

// sum of v over the workgroup (every thread gets it); red: one float of LDS per wave
__device__ __forceinline__ float block_sum(float v, float *red) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < kTinyThreads / 64; i++) s += red[i];
    __syncthreads();
    return s;
}

__device__ __forceinline__ float rms_inv(float ss, int dm, float eps) {
    float rms = sqrtf(ss / (float)dm + eps);
    if (!isfinite(rms) || rms < 1e-20f) rms = 1.0f;   // the reference's finite guard (kernels/norms.cu:58-61)
    return 1.0f / rms;
}

// Rounds of sixteen weight rows a lane goes through in a [K][N] sweep (each is a dependent trip to L2); the routes built
// on these sweeps take a model only while every sweep stays within kTinyMaxRounds -- beyond that the kernel chains with
// their full-width GEMMs are faster (d_model 256 x d_inner 512: 16 rounds for in_proj, 264 us against 102 us per step).
constexpr int kTinyMaxRounds = 3;
inline int sweep_rounds(int K, int N) {
    if (N % 4 != 0 || N < 4 || N / 4 > kTinyThreads || K < 1) return 1 << 20;
    const int ks_n = kTinyThreads / (N / 4) < kTinySlices ? kTinyThreads / (N / 4) : kTinySlices;
    const int kper = (K + ks_n - 1) / ks_n;
    return (kper + 15) / 16;
}

}  // namespace
}  // namespace mrs
