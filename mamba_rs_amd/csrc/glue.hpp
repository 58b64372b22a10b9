// Glue kernels shared by the backbone engines: residual add + RMSNorm, casts, bias rows.
#pragma once
#include "common.hpp"

namespace mrs {

// One workgroup per row: residual (f32) += add (storage dtype, may be null); out = rmsnorm(residual) * w.
// Reference: residual_add_f32_* + rmsnorm_forward_f32in_* (kernels/elementwise.cu:366-376,
// kernels/norms.cu:21-171), with its finite guard: rms = 1 if not finite or < 1e-20 (norms.cu:58-61).
// out2 (may be null): the same result once more in the storage type (the LM head's operand).
template <typename T, typename TO>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float *__restrict__ residual, const T *__restrict__ add,
                                                          TO *__restrict__ out, T *__restrict__ out2, const float *__restrict__ w,
                                                          float eps, int64_t rows, int dm, int64_t out_stride) {
    constexpr int kMaxPer = 16;  // elements per thread kept in registers (d_model <= 4096); longer rows re-read
    __shared__ float part[4];
    const int64_t row = blockIdx.x;
    float *r = residual + row * dm;
    float v[kMaxPer];   // indexed by unrolled loop counters only (a run-time index would put it in scratch memory)
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < kMaxPer; k++) {
        const int i = threadIdx.x + 256 * k;
        float x = 0.0f;
        if (i < dm) {
            x = r[i];
            if (add) { x += Store<T>::ld(add + row * dm + i); r[i] = x; }
        }
        v[k] = x;
        ss = fmaf(x, x, ss);
    }
    for (int i = threadIdx.x + 256 * kMaxPer; i < dm; i += 256) {
        float x = r[i];
        if (add) { x += Store<T>::ld(add + row * dm + i); r[i] = x; }
        ss = fmaf(x, x, ss);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, kWave);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = part[0] + part[1] + part[2] + part[3];
    float rms = sqrtf(ss / (float)dm + eps);
    if (!isfinite(rms) || rms < 1e-20f) rms = 1.0f;
    const float inv = 1.0f / rms;
#pragma unroll
    for (int k = 0; k < kMaxPer; k++) {
        const int i = threadIdx.x + 256 * k;
        if (i < dm) {
            const float o = v[k] * inv * w[i];
            Store<TO>::st(out + row * out_stride + i, o);
            if (out2) Store<T>::st(out2 + row * out_stride + i, o);
        }
    }
    for (int i = threadIdx.x + 256 * kMaxPer; i < dm; i += 256) {
        const float o = r[i] * inv * w[i];
        Store<TO>::st(out + row * out_stride + i, o);
        if (out2) Store<T>::st(out2 + row * out_stride + i, o);
    }
}

// Prefill-sized rows: one wave per row, 4 elements per lane and trip (16-byte residual accesses), the row
// kept in registers between the sum of squares and the scaling.  Same arithmetic as add_rmsnorm_kernel.  TRIPS (the
// number of 16-byte pieces a lane holds, d_model <= 256 TRIPS) is a template parameter: the register array must be
// indexed by compile-time constants, or it lands in scratch memory and every element makes a round trip through it.
template <typename T, typename TO, int TRIPS>
__global__ __launch_bounds__(256) void add_rmsnorm_rows_kernel(float *__restrict__ residual, const T *__restrict__ add,
                                                               TO *__restrict__ out, const float *__restrict__ w,
                                                               float eps, int64_t rows, int dm) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const int nv = dm >> 2;
    float4 *r4 = reinterpret_cast<float4 *>(residual + row * dm);
    struct alignas(4 * sizeof(T)) V4 { T v[4]; };
    struct alignas(4 * sizeof(TO)) O4 { TO v[4]; };
    const V4 *a4 = reinterpret_cast<const V4 *>(add ? add + row * dm : nullptr);
    const float4 *w4 = reinterpret_cast<const float4 *>(w);
    float4 v[TRIPS], ww[TRIPS];
    V4 a[TRIPS];
    // every load of the row before the first use
#pragma unroll
    for (int k = 0; k < TRIPS; k++) {
        const int c = lane + 64 * k;
        if (c < nv) {
            v[k] = r4[c];
            if (add) a[k] = a4[c];
            ww[k] = w4[c];
        }
    }
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < TRIPS; k++) {
        const int c = lane + 64 * k;
        if (c < nv) {
            if (add) {
                v[k].x += Store<T>::ld(&a[k].v[0]); v[k].y += Store<T>::ld(&a[k].v[1]);
                v[k].z += Store<T>::ld(&a[k].v[2]); v[k].w += Store<T>::ld(&a[k].v[3]);
                r4[c] = v[k];
            }
            ss = fmaf(v[k].x, v[k].x, ss); ss = fmaf(v[k].y, v[k].y, ss); ss = fmaf(v[k].z, v[k].z, ss); ss = fmaf(v[k].w, v[k].w, ss);
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, kWave);
    float rms = sqrtf(ss / (float)dm + eps);
    if (!isfinite(rms) || rms < 1e-20f) rms = 1.0f;
    const float inv = 1.0f / rms;
    O4 *o4 = reinterpret_cast<O4 *>(out + row * dm);
#pragma unroll
    for (int k = 0; k < TRIPS; k++) {
        const int c = lane + 64 * k;
        if (c < nv) {
            O4 o;
            Store<TO>::st(&o.v[0], v[k].x * inv * ww[k].x); Store<TO>::st(&o.v[1], v[k].y * inv * ww[k].y);
            Store<TO>::st(&o.v[2], v[k].z * inv * ww[k].z); Store<TO>::st(&o.v[3], v[k].w * inv * ww[k].w);
            o4[c] = o;
        }
    }
}

// Decode-sized row counts past the own chain's limit (64 to 255 rows): one workgroup per row with the same 16-byte
// accesses, every load of the row issued before the first use (a row of 2560 is 2.5 pieces per lane: one round trip to
// memory, a reduction through LDS, one store).  Same arithmetic as add_rmsnorm_kernel.
template <typename T, typename TO, int TRIPS>
__global__ __launch_bounds__(256) void add_rmsnorm_block_kernel(float *__restrict__ residual, const T *__restrict__ add,
                                                                TO *__restrict__ out, const float *__restrict__ w, float eps, int dm) {
    __shared__ float part[4];
    const int64_t row = blockIdx.x;
    const int nv = dm >> 2;
    float4 *r4 = reinterpret_cast<float4 *>(residual + row * dm);
    struct alignas(4 * sizeof(T)) V4 { T v[4]; };
    struct alignas(4 * sizeof(TO)) O4 { TO v[4]; };
    const V4 *a4 = reinterpret_cast<const V4 *>(add ? add + row * dm : nullptr);
    const float4 *w4 = reinterpret_cast<const float4 *>(w);
    float4 v[TRIPS], ww[TRIPS];
    V4 a[TRIPS];
#pragma unroll
    for (int k = 0; k < TRIPS; k++) {
        const int c = threadIdx.x + 256 * k;
        if (c < nv) {
            v[k] = r4[c];
            if (add) a[k] = a4[c];
            ww[k] = w4[c];
        }
    }
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < TRIPS; k++) {
        const int c = threadIdx.x + 256 * k;
        if (c < nv) {
            if (add) {
                v[k].x += Store<T>::ld(&a[k].v[0]); v[k].y += Store<T>::ld(&a[k].v[1]);
                v[k].z += Store<T>::ld(&a[k].v[2]); v[k].w += Store<T>::ld(&a[k].v[3]);
                r4[c] = v[k];
            }
            ss = fmaf(v[k].x, v[k].x, ss); ss = fmaf(v[k].y, v[k].y, ss); ss = fmaf(v[k].z, v[k].z, ss); ss = fmaf(v[k].w, v[k].w, ss);
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, kWave);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = part[0] + part[1] + part[2] + part[3];
    float rms = sqrtf(ss / (float)dm + eps);
    if (!isfinite(rms) || rms < 1e-20f) rms = 1.0f;
    const float inv = 1.0f / rms;
    O4 *o4 = reinterpret_cast<O4 *>(out + row * dm);
#pragma unroll
    for (int k = 0; k < TRIPS; k++) {
        const int c = threadIdx.x + 256 * k;
        if (c < nv) {
            O4 o;
            Store<TO>::st(&o.v[0], v[k].x * inv * ww[k].x); Store<TO>::st(&o.v[1], v[k].y * inv * ww[k].y);
            Store<TO>::st(&o.v[2], v[k].z * inv * ww[k].z); Store<TO>::st(&o.v[3], v[k].w * inv * ww[k].w);
            o4[c] = o;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void cast_from_f32_kernel(T *__restrict__ out, const float *__restrict__ in, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) Store<T>::st(out + i, in[i]);
}

static __global__ __launch_bounds__(256) void bias_rows_kernel(float *__restrict__ out, const float *__restrict__ bias, int64_t n, int dm) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = bias[i % dm];
}

// residual (f32, rows x dm) += add (storage type, may be null); out = rmsnorm(residual) * w as f32 (out_f32) or in the
// storage type; out2 (may be null): the result once more in the storage type.  Prefill-sized row counts take the
// wave-per-row kernel.
template <typename T>
inline void launch_add_rmsnorm_typed(hipStream_t st, float *residual, const void *add, void *out, bool out_f32, void *out2, const float *w,
                                     float eps, int64_t rows, int dm, int64_t out_stride) {
    const dim3 grid((unsigned)rows), block(256);
    if (rows >= 64 && rows < 256 && dm % 4 == 0 && dm <= 4096 && out_stride == dm && !out2 && !out_f32) {
#define MRS_BLK(TR) hipLaunchKernelGGL((add_rmsnorm_block_kernel<T, T, TR>), grid, block, 0, st, residual, (const T *)add, (T *)out, w, eps, dm)
        const int trips = (dm / 4 + 255) / 256;
        if (trips <= 1) MRS_BLK(1);
        else if (trips <= 2) MRS_BLK(2);
        else MRS_BLK(4);
#undef MRS_BLK
        return;
    }
    if (rows >= 256 && dm % 4 == 0 && dm <= 4096 && out_stride == dm && !out2 && !out_f32) {
        const dim3 g4((unsigned)((rows + 3) / 4));
#define MRS_ROWS(TR) hipLaunchKernelGGL((add_rmsnorm_rows_kernel<T, T, TR>), g4, block, 0, st, residual, (const T *)add, (T *)out, w, eps, rows, dm)
        const int trips = (dm / 4 + 63) / 64;
        if (trips <= 2) MRS_ROWS(2);
        else if (trips <= 4) MRS_ROWS(4);
        else if (trips <= 8) MRS_ROWS(8);
        else MRS_ROWS(16);
#undef MRS_ROWS
        return;
    }
    if (out_f32)
        hipLaunchKernelGGL((add_rmsnorm_kernel<T, float>), grid, block, 0, st, residual, (const T *)add, (float *)out, (T *)out2, w, eps, rows, dm,
                           out_stride);
    else
        hipLaunchKernelGGL((add_rmsnorm_kernel<T, T>), grid, block, 0, st, residual, (const T *)add, (T *)out, (T *)out2, w, eps, rows, dm,
                           out_stride);
}

inline int launch_add_rmsnorm_any(hipStream_t st, int dtype, float *residual, const void *add, void *out, bool out_f32, void *out2,
                                  const float *w, float eps, int64_t rows, int dm, int64_t out_stride) {
    MRS_DISPATCH_DTYPE(dtype, T_, launch_add_rmsnorm_typed<T_>(st, residual, add, out, out_f32, out2, w, eps, rows, dm, out_stride));
    return check_launch("add_rmsnorm_kernel");
}

}  // namespace mrs
