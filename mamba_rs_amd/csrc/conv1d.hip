// Causal depthwise conv1d with bias and (optionally) SiLU, channel-last layout.
//
// Replaces conv1d_step_forward[_silu]_* (kernels/conv1d.cu:14-115) and
// conv1d_burnin_forward_nosave_* (kernels/conv1d.cu:209-315).  The window state
// is the reference's GPU layout: [batch, d_inner, d_conv] f32, oldest first,
// holding the last d_conv inputs after the call.
//
// The sequence kernel is a pure streaming op (read x once, write u once), so it
// is split over time as well as channels: a position only needs its d_conv-1
// predecessors, which a chunk re-reads from x (or from the carried state for the
// first positions of the sequence).  Each lane owns 4 consecutive channels and a
// short run of steps.
#include "common.hpp"
#include <type_traits>

namespace mrs {

constexpr int kMaxConv = 8;  // reference limit, src/config.rs:154-159

template <typename T, bool SILU, bool DC4 = false>
__global__ __launch_bounds__(256) void conv1d_step_kernel(
    T *__restrict__ out, float *__restrict__ state, const T *__restrict__ new_x, int64_t x_stride,
    const float *__restrict__ weight, const float *__restrict__ bias, int64_t total, int di, int dc) {
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= total) return;
    const int d = (int)(r % di);
    const int64_t xi = (r / di) * x_stride + d;  // new_x rows may be wider than d_inner (x half of in_proj's output)
    float *st = state + r * dc;
    const float *w = weight + (int64_t)d * dc;
    float s = bias[d];
    if constexpr (DC4) {
        // d_conv 4 with 16-byte aligned state and taps: the window and the taps as one 16-byte access each (three 4-byte loads at a 16-byte lane stride
        // ask for every cache line of the wave's window three times)
        const float4 sv = *reinterpret_cast<const float4 *>(st), wv = *reinterpret_cast<const float4 *>(w);
        const float xn = Store<T>::ld(new_x + xi);
        s = fmaf(sv.y, wv.x, s); s = fmaf(sv.z, wv.y, s); s = fmaf(sv.w, wv.z, s); s = fmaf(xn, wv.w, s);
        *reinterpret_cast<float4 *>(st) = make_float4(sv.y, sv.z, sv.w, xn);
        Store<T>::st(out + r, SILU ? silu(s) : s);
        return;
    }
    float win[kMaxConv];
#pragma unroll
    for (int k = 0; k < kMaxConv; k++)
        if (k < dc) win[k] = (k + 1 < dc) ? st[k + 1] : Store<T>::ld(new_x + xi);
#pragma unroll
    for (int k = 0; k < kMaxConv; k++)
        if (k < dc) { s = fmaf(win[k], w[k], s); st[k] = win[k]; }
    Store<T>::st(out + r, SILU ? silu(s) : s);
}

// The sequence kernel: a lane owns VEC consecutive channels and TPL consecutive steps, requests all of its rows (the
// d_conv-1 rows before its first step included) before it computes anything, and runs straight through them -- no loop,
// no per-step bounds test: rows at and beyond T lie outside the buffer resources, so their loads return zero and their
// stores are dropped.  Small tiles and few registers per lane (rows stay packed until they are used) keep many short
// waves resident, which is what a streaming kernel needs.  Measured at batch 8 x 2048 x 1536, bf16: 8 channels x 16-32
// steps per lane with a double-buffered loop (192 registers, per-step bounds tests) 26.1 us; 4 channels x 8 steps,
// straight-line, 20.0 us; 4 x 16 21.2 us, 8 x 8 24.9 us, 4 x 4 22.3 us; 64- to 192-lane workgroups alike, 256 slower.
template <typename T, int VEC> struct RowVec;
template <typename T> struct RowVec<T, 4> {   // 16-bit: 8 bytes, f32: 16 bytes
    typedef typename std::conditional<sizeof(T) == 2, uint2, uint4>::type raw;
};

template <typename T, int VEC> __device__ __forceinline__ typename RowVec<T, VEC>::raw row_ld(__amdgpu_buffer_rsrc_t r, unsigned off) {
    typedef typename RowVec<T, VEC>::raw raw;
    if constexpr (sizeof(raw) == 8) return __builtin_bit_cast(raw, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
    else return __builtin_bit_cast(raw, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
}
template <typename T, int VEC> __device__ __forceinline__ void row_st(typename RowVec<T, VEC>::raw v, __amdgpu_buffer_rsrc_t r, unsigned off) {
    typedef typename RowVec<T, VEC>::raw raw;
    if constexpr (sizeof(raw) == 8) { typedef unsigned v2u __attribute__((ext_vector_type(2))); __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u, v), r, off, 0, 0); }
    else { typedef unsigned v4u __attribute__((ext_vector_type(4))); __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), r, off, 0, 0); }
}
template <typename T, int VEC> __device__ __forceinline__ void row_widen(const typename RowVec<T, VEC>::raw &v, float (&o)[VEC]) {
    const T *e = reinterpret_cast<const T *>(&v);
#pragma unroll
    for (int c = 0; c < VEC; c++) o[c] = Store<T>::ld(e + c);
}

template <typename T, int DC, int VEC, int TPL>
__global__ __launch_bounds__(64) void conv1d_seq_silu_stream_kernel(
    T *__restrict__ u_out, float *__restrict__ state, const T *__restrict__ x, int64_t x_stride,
    const float *__restrict__ weight, const float *__restrict__ bias, int batch, int Tlen, int di, int nchunk) {
    typedef typename RowVec<T, VEC>::raw raw;
    // (batch row, time chunk) come from the block index alone: they are the same for every lane, so the buffer resources
    // below sit in scalar registers (a per-lane resource makes the compiler loop over its distinct values at every access)
    const int nvec = di / VEC;
    const int nblk = (nvec + (int)blockDim.x - 1) / (int)blockDim.x;
    // Workgroups go to the chip's 8 L2 domains round-robin by index; each domain is given a contiguous eighth of the work
    // instead, so the chunk that re-reads the d_conv-1 rows before its first step finds them in the L2 that the chunk
    // before it filled (with neighbouring chunks in different domains those rows came from memory twice: 69.6 MB
    // fetched for 50.3 MB of x).
    const unsigned n8 = gridDim.x / 8;
    const unsigned bid = blockIdx.x < 8 * n8 ? (blockIdx.x & 7) * n8 + (blockIdx.x >> 3) : blockIdx.x;
    const int cvb = (int)(bid % (unsigned)nblk);
    const int rest = (int)(bid / (unsigned)nblk);
    const int chunk = rest % nchunk;
    const int b = rest / nchunk;
    const int cv = cvb * (int)blockDim.x + (int)threadIdx.x;
    if (cv >= nvec) return;
    const int d0 = cv * VEC;
    const int t0 = chunk * TPL;
    constexpr unsigned es = (unsigned)sizeof(T);
    // one batch row of x and of u; a row at or beyond T starts past the end of the resource
    const __amdgpu_buffer_rsrc_t xb = __builtin_amdgcn_make_buffer_rsrc(const_cast<T *>(x + (int64_t)b * Tlen * x_stride), 0,
                                                                       (int)(((int64_t)(Tlen - 1) * x_stride + di) * es), 0x00020000);
    const __amdgpu_buffer_rsrc_t ub = __builtin_amdgcn_make_buffer_rsrc(u_out + (int64_t)b * Tlen * di, 0, (int)((int64_t)Tlen * di * es), 0x00020000);
    const unsigned xrow = (unsigned)x_stride * es, urow = (unsigned)di * es;

    raw rows[TPL + DC - 1];   // rows[j]: step t0 - (DC-1) + j
    if (chunk > 0) {
#pragma unroll
        for (int j = 0; j < DC - 1; j++) rows[j] = row_ld<T, VEC>(xb, (unsigned)(t0 - (DC - 1) + j) * xrow + (unsigned)d0 * es);
    }
#pragma unroll
    for (int j = 0; j < TPL; j++) rows[DC - 1 + j] = row_ld<T, VEC>(xb, (unsigned)(t0 + j) * xrow + (unsigned)d0 * es);

    float w[DC][VEC], bs[VEC], win[DC][VEC];
#pragma unroll
    for (int c = 0; c < VEC; c++) {
        bs[c] = bias[d0 + c];
#pragma unroll
        for (int k = 0; k < DC; k++) w[k][c] = weight[(int64_t)(d0 + c) * DC + k];
    }
    // window before the first step: win[k] = input at time t0 - DC + k (k = 0 is dropped by the first shift)
    if (chunk > 0) {
#pragma unroll
        for (int k = 1; k < DC; k++) row_widen<T, VEC>(rows[k - 1], win[k]);
    } else {
        // carried state: slot s holds the input at time s - DC; the chunk-0 lane of a channel vector is the only reader of
        // that channel's old state, so it is also the one that writes the new one (from x alone when T >= DC)
#pragma unroll
        for (int k = 1; k < DC; k++)
#pragma unroll
            for (int c = 0; c < VEC; c++) win[k][c] = state[((int64_t)b * di + d0 + c) * DC + k];
        float nw[VEC][DC];
#pragma unroll
        for (int k = 0; k < DC; k++) {
            const int tt = Tlen - DC + k;  // time of slot k after the call
            if (tt >= 0) {
                float v[VEC];
                row_widen<T, VEC>(row_ld<T, VEC>(xb, (unsigned)tt * xrow + (unsigned)d0 * es), v);
#pragma unroll
                for (int c = 0; c < VEC; c++) nw[c][k] = v[c];
            } else {
#pragma unroll
                for (int c = 0; c < VEC; c++) {   // old slot tt + DC = Tlen + k, in 1..DC-1
                    float v = 0.0f;
#pragma unroll
                    for (int kk = 1; kk < DC; kk++)
                        if (kk == Tlen + k) v = win[kk][c];
                    nw[c][k] = v;
                }
            }
        }
        float *sp = state + ((int64_t)b * di + d0) * DC;
#pragma unroll
        for (int c = 0; c < VEC; c++)
#pragma unroll
            for (int k = 0; k < DC; k++) sp[c * DC + k] = nw[c][k];
    }
#pragma unroll
    for (int j = 0; j < TPL; j++) {
        float xin[VEC];
        row_widen<T, VEC>(rows[DC - 1 + j], xin);
        raw ov;
        T *oe = reinterpret_cast<T *>(&ov);
#pragma unroll
        for (int c = 0; c < VEC; c++) {
#pragma unroll
            for (int k = 0; k + 1 < DC; k++) win[k][c] = win[k + 1][c];
            win[DC - 1][c] = xin[c];
            float sacc = bs[c];
#pragma unroll
            for (int k = 0; k < DC; k++) sacc = fmaf(win[k][c], w[k][c], sacc);
            Store<T>::st(oe + c, silu(sacc));
        }
        row_st<T, VEC>(ov, ub, (unsigned)(t0 + j) * urow + (unsigned)d0 * es);
    }
}

// Fallback for shapes the vector kernel does not take (d_inner % VEC != 0 or
// unaligned rows): one lane per (b,d), serial in time, register window.
template <typename T>
__global__ __launch_bounds__(256) void conv1d_seq_silu_generic_kernel(
    T *__restrict__ u_out, float *__restrict__ state, const T *__restrict__ x, int64_t x_stride,
    const float *__restrict__ weight, const float *__restrict__ bias, int64_t total, int Tlen, int di,
    int dc) {
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= total) return;
    const int b = (int)(r / di);
    const int d = (int)(r - (int64_t)b * di);
    float *st = state + r * dc;
    float win[kMaxConv], w[kMaxConv];
#pragma unroll
    for (int k = 0; k < kMaxConv; k++) {
        win[k] = (k < dc) ? st[k] : 0.0f;
        w[k] = (k < dc) ? weight[(int64_t)d * dc + k] : 0.0f;
    }
    const float bd = bias[d];
    for (int t = 0; t < Tlen; t++) {
        const float xn = Store<T>::ld(x + ((int64_t)b * Tlen + t) * x_stride + d);
        float s = bd;
#pragma unroll
        for (int k = 0; k < kMaxConv; k++) {
            if (k < dc) {
                win[k] = (k + 1 < dc) ? win[k + 1] : xn;
                s = fmaf(win[k], w[k], s);
            }
        }
        Store<T>::st(u_out + ((int64_t)b * Tlen + t) * di + d, silu(s));
    }
#pragma unroll
    for (int k = 0; k < kMaxConv; k++)
        if (k < dc) st[k] = win[k];
}

template <typename T>
static int launch_conv_seq(hipStream_t st, void *u_out, float *state, const void *x, int64_t x_stride,
                           const float *weight, const float *bias, int batch, int Tlen, int di, int dc) {
    const int64_t total = (int64_t)batch * di;
    // the streaming kernel moves 4 channels per lane (8 bytes of 16-bit storage, 16 of f32) and addresses one batch row of
    // x and of u with 32-bit byte offsets
    const size_t lane_bytes = 4 * sizeof(T);
    const bool vec_ok = (dc >= 2 && dc <= 4) && di % 4 == 0 && x_stride % 4 == 0 && aligned(x, lane_bytes) && aligned(u_out, lane_bytes) &&
                        (int64_t)Tlen * x_stride * (int64_t)sizeof(T) < 0x7fffffffLL;
    if (!vec_ok) {
        const int64_t blocks = (total + 255) / 256;
        hipLaunchKernelGGL((conv1d_seq_silu_generic_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st,
                           (T *)u_out, state, (const T *)x, x_stride, weight, bias, total, Tlen, di, dc);
        return check_launch("conv1d_seq_silu_generic_kernel");
    }
    constexpr int kVec = 4, kTpl = 8, kBlock = 64;
    const int nch = (Tlen + kTpl - 1) / kTpl;
    const int nblk = (di / kVec + kBlock - 1) / kBlock;
    const int64_t blocks = (int64_t)batch * nch * nblk;
    if (blocks > 0x7fffffffLL) return fail(MRS_E_SHAPE, "conv1d seq: grid too large");
#define MRS_DC(K)                                                                                          \
    case K:                                                                                                \
        hipLaunchKernelGGL((conv1d_seq_silu_stream_kernel<T, K, kVec, kTpl>), dim3((unsigned)blocks), dim3(kBlock), 0, st, \
                           (T *)u_out, state, (const T *)x, x_stride, weight, bias, batch, Tlen, di, nch); \
        break
    switch (dc) { MRS_DC(2); MRS_DC(3); MRS_DC(4); }
#undef MRS_DC
    return check_launch("conv1d_seq_silu_stream_kernel");
}

static int conv_check(const char *fn, int dtype, const void *out, const void *state, const void *x,
                      const void *w, const void *b, int batch, int di, int dc) {
    if (dtype != MRS_F32 && dtype != MRS_F16 && dtype != MRS_BF16)
        return fail(MRS_E_DTYPE, "%s: dtype %d is not f32/f16/bf16", fn, dtype);
    if (!out || !state || !x || !w || !b) return fail(MRS_E_NULL, "%s: null pointer", fn);
    if (batch < 1 || di < 1) return fail(MRS_E_SHAPE, "%s: batch=%d d_inner=%d must be >= 1", fn, batch, di);
    if (dc < 1 || dc > kMaxConv) return fail(MRS_E_SHAPE, "%s: d_conv=%d outside 1..=%d", fn, dc, kMaxConv);
    return MRS_OK;
}

int launch_conv1d_step(hipStream_t st, int dtype, void *out, float *state, const void *new_x, int64_t x_stride,
                       const float *weight, const float *bias, int batch, int d_inner, int d_conv, int apply_silu) {
    const int64_t total = (int64_t)batch * d_inner;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffLL) return fail(MRS_E_SHAPE, "conv1d step: grid too large");
    const dim3 grid((unsigned)blocks), block(256);
    const bool dc4 = d_conv == 4 && aligned(state, 16) && aligned(weight, 16);
    MRS_DISPATCH_DTYPE(dtype, T_, {
        if (apply_silu && dc4) hipLaunchKernelGGL((conv1d_step_kernel<T_, true, true>), grid, block, 0, st, (T_ *)out, state, (const T_ *)new_x, x_stride, weight, bias, total, d_inner, d_conv);
        else if (apply_silu) hipLaunchKernelGGL((conv1d_step_kernel<T_, true>), grid, block, 0, st, (T_ *)out, state, (const T_ *)new_x, x_stride, weight, bias, total, d_inner, d_conv);
        else hipLaunchKernelGGL((conv1d_step_kernel<T_, false>), grid, block, 0, st, (T_ *)out, state, (const T_ *)new_x, x_stride, weight, bias, total, d_inner, d_conv);
    });
    return check_launch("conv1d_step_kernel");
}

}  // namespace mrs

using namespace mrs;

extern "C" int mrs_conv1d_step(void *stream, int dtype, void *out, float *state, const void *new_x,
                               const float *weight, const float *bias, int batch, int d_inner,
                               int d_conv, int apply_silu) {
    int rc = conv_check("mrs_conv1d_step", dtype, out, state, new_x, weight, bias, batch, d_inner, d_conv);
    if (rc) return rc;
    return launch_conv1d_step(as_stream(stream), dtype, out, state, new_x, d_inner, weight, bias, batch, d_inner, d_conv, apply_silu);
}

extern "C" int mrs_conv1d_seq_silu(void *stream, int dtype, void *u_out, float *state, const void *x_branch,
                                   int64_t x_stride, const float *weight, const float *bias, int batch,
                                   int T, int d_inner, int d_conv) {
    int rc = conv_check("mrs_conv1d_seq_silu", dtype, u_out, state, x_branch, weight, bias, batch, d_inner, d_conv);
    if (rc) return rc;
    if (T < 1) return fail(MRS_E_SHAPE, "mrs_conv1d_seq_silu: T=%d must be >= 1", T);
    if (x_stride < d_inner) return fail(MRS_E_SHAPE, "mrs_conv1d_seq_silu: x_stride=%lld < d_inner=%d", (long long)x_stride, d_inner);
    if ((int64_t)batch * T * x_stride > 0x7fffffffLL * 4) return fail(MRS_E_SHAPE, "mrs_conv1d_seq_silu: tensor too large");
    hipStream_t st = as_stream(stream);
    MRS_DISPATCH_DTYPE(dtype, T_, return launch_conv_seq<T_>(st, u_out, state, x_branch, x_stride, weight, bias, batch, T, d_inner, d_conv));
    return MRS_OK;
}
