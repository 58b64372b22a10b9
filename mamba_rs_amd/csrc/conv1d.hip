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
// first positions of the sequence).  Each lane owns VEC consecutive channels and
// moves them with one 16-byte access per row.
#include "common.hpp"

namespace mrs {

constexpr int kMaxConv = 8;  // reference limit, src/config.rs:154-159

template <typename T, bool SILU>
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
    float win[kMaxConv];
#pragma unroll
    for (int k = 0; k < kMaxConv; k++)
        if (k < dc) win[k] = (k + 1 < dc) ? st[k + 1] : Store<T>::ld(new_x + xi);
#pragma unroll
    for (int k = 0; k < kMaxConv; k++)
        if (k < dc) { s = fmaf(win[k], w[k], s); st[k] = win[k]; }
    Store<T>::st(out + r, SILU ? silu(s) : s);
}

constexpr int kConvGroup = 8;  // timesteps whose rows a lane requests together

template <typename T> struct alignas(16) Vec16 {
    static constexpr int N = 16 / sizeof(T);
    T v[N];
};

// One lane: VEC = 16/sizeof(T) channels, TPL consecutive timesteps.
// Grid: x = channel-vector groups * time chunks folded, see launch.
template <typename T, int DC>
__global__ __launch_bounds__(256) void conv1d_seq_silu_kernel(
    T *__restrict__ u_out, float *__restrict__ state, const T *__restrict__ x, int64_t x_stride,
    const float *__restrict__ weight, const float *__restrict__ bias, int batch, int Tlen, int di,
    int tpl, int nchunk) {
    constexpr int VEC = Vec16<T>::N;
    const int nvec = di / VEC;  // host guarantees di % VEC == 0
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int cv = (int)(gid % nvec);
    const int64_t rest = gid / nvec;
    const int chunk = (int)(rest % nchunk);
    const int b = (int)(rest / nchunk);
    if (b >= batch) return;
    const int d0 = cv * VEC;
    const int t0 = chunk * tpl;
    const int t1 = min(Tlen, t0 + tpl);

    float w[DC][VEC], bs[VEC], win[DC][VEC];
#pragma unroll
    for (int c = 0; c < VEC; c++) {
        bs[c] = bias[d0 + c];
#pragma unroll
        for (int k = 0; k < DC; k++) w[k][c] = weight[(int64_t)(d0 + c) * DC + k];
    }
    // window before position t0: win[k] = input at time t0 - DC + k (k = 0 is dropped by the first shift)
#pragma unroll
    for (int k = 1; k < DC; k++) {
        const int tt = t0 - DC + k;
        if (tt >= 0) {
            const Vec16<T> xv = *reinterpret_cast<const Vec16<T> *>(x + ((int64_t)b * Tlen + tt) * x_stride + d0);
#pragma unroll
            for (int c = 0; c < VEC; c++) win[k][c] = Store<T>::ld(&xv.v[c]);
        } else {
            // carried state slot: state holds inputs at times -DC..-1, slot s <-> time s - DC
            const int s = tt + DC;
#pragma unroll
            for (int c = 0; c < VEC; c++) win[k][c] = state[((int64_t)b * di + d0 + c) * DC + s];
        }
    }
    // New window state = the last DC inputs of (old window ++ x[0..T)).  The chunk-0 lane of a channel vector is
    // the only reader of that channel's old state (chunks are longer than the window), so it is the one that
    // writes the new one, after its own read above and from x alone (old slots only when T < DC).
    if (chunk == 0) {
        float nw[VEC][DC];
#pragma unroll
        for (int k = 0; k < DC; k++) {
            const int tt = Tlen - DC + k;  // time of slot k after the call
            if (tt >= 0) {
                const Vec16<T> xv = *reinterpret_cast<const Vec16<T> *>(x + ((int64_t)b * Tlen + tt) * x_stride + d0);
#pragma unroll
                for (int c = 0; c < VEC; c++) nw[c][k] = Store<T>::ld(&xv.v[c]);
            } else {
                // old slot tt + DC = Tlen + k, in 1..DC-1: it is win[Tlen + k] of the window loaded above
#pragma unroll
                for (int c = 0; c < VEC; c++) {
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
    // Groups of kConvGroup steps: the rows of the next group are requested before the current one is
    // computed, so a lane always has kConvGroup 16-byte loads in flight.
    Vec16<T> cur[kConvGroup], nxt[kConvGroup];
    auto load_group = [&](Vec16<T> (&g)[kConvGroup], int tg) {
#pragma unroll
        for (int j = 0; j < kConvGroup; j++) {
            const int t = min(tg + j, t1 - 1);
            g[j] = *reinterpret_cast<const Vec16<T> *>(x + ((int64_t)b * Tlen + t) * x_stride + d0);
        }
    };
    if (t0 < t1) load_group(cur, t0);
    for (int tg = t0; tg < t1; tg += kConvGroup) {
        if (tg + kConvGroup < t1) load_group(nxt, tg + kConvGroup);
#pragma unroll
        for (int j = 0; j < kConvGroup; j++) {
            const int t = tg + j;
            if (t < t1) {
                Vec16<T> ov;
#pragma unroll
                for (int c = 0; c < VEC; c++) {
#pragma unroll
                    for (int k = 0; k + 1 < DC; k++) win[k][c] = win[k + 1][c];
                    win[DC - 1][c] = Store<T>::ld(&cur[j].v[c]);
                    float s = bs[c];
#pragma unroll
                    for (int k = 0; k < DC; k++) s = fmaf(win[k][c], w[k][c], s);
                    Store<T>::st(&ov.v[c], silu(s));
                }
                *reinterpret_cast<Vec16<T> *>(u_out + ((int64_t)b * Tlen + t) * di + d0) = ov;
            }
        }
#pragma unroll
        for (int j = 0; j < kConvGroup; j++) cur[j] = nxt[j];
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
    constexpr int VEC = Vec16<T>::N;
    const int64_t total = (int64_t)batch * di;
    const bool vec_ok = (dc >= 2 && dc <= 4) && di % VEC == 0 && x_stride % VEC == 0 && aligned(x, 16) && aligned(u_out, 16);
    if (!vec_ok) {
        const int64_t blocks = (total + 255) / 256;
        hipLaunchKernelGGL((conv1d_seq_silu_generic_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st,
                           (T *)u_out, state, (const T *)x, x_stride, weight, bias, total, Tlen, di, dc);
        return check_launch("conv1d_seq_silu_generic_kernel");
    }
    const int nvec = di / VEC;
    // timesteps per lane: enough lanes to fill the chip, long enough to amortise the window reload
    int tpl = 32;
    while (tpl > 16 && (int64_t)batch * nvec * ((Tlen + tpl - 1) / tpl) < 2 * 256 * 256) tpl >>= 1;
    const int nchunk = (Tlen + tpl - 1) / tpl;
    const int64_t threads = (int64_t)batch * nchunk * nvec;
    const int64_t blocks = (threads + 255) / 256;
    if (blocks > 0x7fffffffLL) return fail(MRS_E_SHAPE, "conv1d seq: grid too large");
    const dim3 grid((unsigned)blocks), block(256);
#define MRS_DC(K)                                                                                       \
    case K:                                                                                             \
        hipLaunchKernelGGL((conv1d_seq_silu_kernel<T, K>), grid, block, 0, st, (T *)u_out, state,       \
                           (const T *)x, x_stride, weight, bias, batch, Tlen, di, tpl, nchunk);         \
        break
    switch (dc) { MRS_DC(2); MRS_DC(3); MRS_DC(4); }
#undef MRS_DC
    return check_launch("conv1d_seq_silu_kernel");
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
    MRS_DISPATCH_DTYPE(dtype, T_, {
        if (apply_silu) hipLaunchKernelGGL((conv1d_step_kernel<T_, true>), grid, block, 0, st, (T_ *)out, state, (const T_ *)new_x, x_stride, weight, bias, total, d_inner, d_conv);
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
