// Mamba-3 SISO trapezoidal recurrence, sequential in time (decode step and short sequences).
//
//   H[p,n] <- alpha H[p,n] + beta v_prev[p] k_prev[n] + gamma x[p] k[n]
//   y[p]    = sum_n H[p,n] q[n] + D[h] x[p];   then k_prev <- k, v_prev <- x
//
// Replaces m3_step_fwd_* (kernels/mamba3_ssd.cu:56-215) and m3_burnin_fwd_nosave_*
// (kernels/mamba3_ssd.cu:453-546).  One workgroup per (batch row, head).  The state
// H [headdim, d_state] f32 is what moves -- 2*4*hd*ds bytes per head per step against a
// few hundred bytes of activations -- so a group of LG = d_state/4 lanes owns one row p
// and each lane keeps one float4 of it: every state access is a coalesced 16-byte piece,
// the row dot product with q is finished with lane shuffles, and over a sequence the
// state, the previous k and the previous x never leave registers.
#include "common.hpp"

namespace mrs {

template <typename T> struct Vec4Ld;
template <> struct Vec4Ld<float> {
    __device__ static __forceinline__ float4 ld(const float *p) { return *reinterpret_cast<const float4 *>(p); }
};
template <> struct Vec4Ld<bf16_t> {
    __device__ static __forceinline__ float4 ld(const bf16_t *p) {
        const uint2 w = *reinterpret_cast<const uint2 *>(p);
        return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u),
                           __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xffff0000u));
    }
};
template <> struct Vec4Ld<f16_t> {
    __device__ static __forceinline__ float4 ld(const f16_t *p) {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        const h4 v = *reinterpret_cast<const h4 *>(p);
        return make_float4((float)v.x, (float)v.y, (float)v.z, (float)v.w);
    }
};

// blockDim.x = hd * LG (<= 1024), LG = ds / 4 a power of two <= 64.
template <typename T, int LG>
__global__ __launch_bounds__(1024) void m3_seq_kernel(
    float *__restrict__ ssm, float *__restrict__ kst, float *__restrict__ vst, T *__restrict__ y,
    const T *__restrict__ x, const T *__restrict__ k, const T *__restrict__ q,
    const float *__restrict__ alpha, const float *__restrict__ beta, const float *__restrict__ gamma,
    const float *__restrict__ Dp, int Tlen, int nh, int hd) {
    constexpr int ds = 4 * LG;
    const int b = blockIdx.x / nh, h = blockIdx.x - b * nh;
    const int p = threadIdx.x / LG, g = threadIdx.x % LG;
    const int di = nh * hd;
    const int64_t bh = (int64_t)b * nh + h;
    float *Hrow = ssm + (bh * hd + p) * ds + 4 * g;
    float4 H = *reinterpret_cast<const float4 *>(Hrow);
    float4 kp = *reinterpret_cast<const float4 *>(kst + bh * ds + 4 * g);
    float vp = vst[bh * hd + p];
    const float Dh = Dp[h];
    float4 kc = kp;
    float xv = vp;
    for (int t = 0; t < Tlen; t++) {
        const int64_t bt = (int64_t)b * Tlen + t;
        const float al = alpha[bt * nh + h], be = beta[bt * nh + h], ga = gamma[bt * nh + h];
        kc = Vec4Ld<T>::ld(k + (bt * nh + h) * ds + 4 * g);
        const float4 qc = Vec4Ld<T>::ld(q + (bt * nh + h) * ds + 4 * g);
        xv = Store<T>::ld(x + bt * di + h * hd + p);
        const float bv = be * vp, gx = ga * xv;
        H.x = fmaf(al, H.x, fmaf(bv, kp.x, gx * kc.x));
        H.y = fmaf(al, H.y, fmaf(bv, kp.y, gx * kc.y));
        H.z = fmaf(al, H.z, fmaf(bv, kp.z, gx * kc.z));
        H.w = fmaf(al, H.w, fmaf(bv, kp.w, gx * kc.w));
        float acc = H.x * qc.x;
        acc = fmaf(H.y, qc.y, acc);
        acc = fmaf(H.z, qc.z, acc);
        acc = fmaf(H.w, qc.w, acc);
#pragma unroll
        for (int m = 1; m < LG; m <<= 1) acc += __shfl_xor(acc, m, kWave);
        if (g == 0) Store<T>::st(y + bt * di + h * hd + p, fmaf(Dh, xv, acc));
        kp = kc;
        vp = xv;
    }
    *reinterpret_cast<float4 *>(Hrow) = H;
    // every lane of the workgroup has read the old k_state before anyone replaces it
    __syncthreads();
    if (p == 0) *reinterpret_cast<float4 *>(kst + bh * ds + 4 * g) = kc;
    if (g == 0) vst[bh * hd + p] = xv;
}

// Any headdim / d_state: one lane per row p, states streamed through global memory.
template <typename T>
__global__ __launch_bounds__(256) void m3_seq_generic_kernel(
    float *__restrict__ ssm, float *__restrict__ kst, float *__restrict__ vst, T *__restrict__ y,
    const T *__restrict__ x, const T *__restrict__ k, const T *__restrict__ q,
    const float *__restrict__ alpha, const float *__restrict__ beta, const float *__restrict__ gamma,
    const float *__restrict__ Dp, int Tlen, int nh, int hd, int ds) {
    const int b = blockIdx.x / nh, h = blockIdx.x - b * nh;
    const int di = nh * hd;
    const int64_t bh = (int64_t)b * nh + h;
    extern __shared__ float kprev[];  // [ds]
    for (int n = threadIdx.x; n < ds; n += blockDim.x) kprev[n] = kst[bh * ds + n];
    __syncthreads();
    for (int t = 0; t < Tlen; t++) {
        const int64_t bt = (int64_t)b * Tlen + t;
        const float al = alpha[bt * nh + h], be = beta[bt * nh + h], ga = gamma[bt * nh + h];
        const T *kc = k + (bt * nh + h) * ds;
        const T *qc = q + (bt * nh + h) * ds;
        for (int p = threadIdx.x; p < hd; p += blockDim.x) {
            const float xv = Store<T>::ld(x + bt * di + h * hd + p);
            const float bv = be * vst[bh * hd + p], gx = ga * xv;
            float *H = ssm + (bh * hd + p) * ds;
            float acc = Dp[h] * xv;
            for (int n = 0; n < ds; n++) {
                const float hn = fmaf(al, H[n], fmaf(bv, kprev[n], gx * Store<T>::ld(kc + n)));
                H[n] = hn;
                acc = fmaf(hn, Store<T>::ld(qc + n), acc);
            }
            Store<T>::st(y + bt * di + h * hd + p, acc);
            vst[bh * hd + p] = xv;
        }
        __syncthreads();
        for (int n = threadIdx.x; n < ds; n += blockDim.x) kprev[n] = Store<T>::ld(kc + n);
        __syncthreads();
    }
    for (int n = threadIdx.x; n < ds; n += blockDim.x) kst[bh * ds + n] = kprev[n];
}

template <typename T>
static int launch_m3_seq(hipStream_t st, float *ssm, float *kst, float *vst, void *y, const void *x,
                         const void *k, const void *q, const float *alpha, const float *beta,
                         const float *gamma, const float *D, int batch, int Tlen, int nh, int hd, int ds) {
    const dim3 grid((unsigned)(batch * nh));
#define MRS_ARGS ssm, kst, vst, (T *)y, (const T *)x, (const T *)k, (const T *)q, alpha, beta, gamma, D, Tlen, nh, hd
    const int lg = ds / 4;
    const bool vec_ok = ds % 4 == 0 && (lg & (lg - 1)) == 0 && lg >= 1 && lg <= 64 && hd * lg <= 1024 &&
                        aligned(ssm, 16) && aligned(kst, 16) && aligned(k, 8) && aligned(q, 8);
    if (vec_ok) {
        const dim3 block((unsigned)(hd * lg));
#define MRS_LG(L) case L: hipLaunchKernelGGL((m3_seq_kernel<T, L>), grid, block, 0, st, MRS_ARGS); break
        switch (lg) { MRS_LG(1); MRS_LG(2); MRS_LG(4); MRS_LG(8); MRS_LG(16); MRS_LG(32); MRS_LG(64); }
#undef MRS_LG
    } else {
        int threads = hd < 256 ? ((hd + 63) / 64) * 64 : 256;
        hipLaunchKernelGGL((m3_seq_generic_kernel<T>), grid, dim3((unsigned)threads), (size_t)ds * sizeof(float), st,
                           MRS_ARGS, ds);
    }
#undef MRS_ARGS
    return check_launch("m3_seq_kernel");
}

static int m3_check(const char *fn, int dtype, const void *ssm, const void *kst, const void *vst,
                    const void *y, const void *x, const void *k, const void *q, const void *al,
                    const void *be, const void *ga, const void *D, int batch, int T, int nh, int hd, int ds) {
    if (dtype != MRS_F32 && dtype != MRS_F16 && dtype != MRS_BF16)
        return fail(MRS_E_DTYPE, "%s: dtype %d is not f32/f16/bf16", fn, dtype);
    if (!ssm || !kst || !vst || !y || !x || !k || !q || !al || !be || !ga || !D)
        return fail(MRS_E_NULL, "%s: null pointer", fn);
    if (batch < 1 || T < 1 || nh < 1 || hd < 1) return fail(MRS_E_SHAPE, "%s: batch=%d T=%d nheads=%d headdim=%d must be >= 1", fn, batch, T, nh, hd);
    if (ds < 1 || ds > 256) return fail(MRS_E_SHAPE, "%s: d_state=%d outside 1..=256", fn, ds);
    if (hd > 1024) return fail(MRS_E_SHAPE, "%s: headdim=%d > 1024", fn, hd);
    if ((int64_t)batch * T * nh * hd * ds > 0x7fffffffLL * 8) return fail(MRS_E_SHAPE, "%s: problem too large", fn);
    return MRS_OK;
}

}  // namespace mrs

using namespace mrs;

extern "C" int mrs_m3_seq_fwd(void *stream, int dtype, float *ssm_state, float *k_state, float *v_state,
                              void *y, const void *x, const void *k, const void *q, const float *alpha,
                              const float *beta, const float *gamma, const float *D, int batch, int T,
                              int nheads, int headdim, int d_state) {
    int rc = m3_check("mrs_m3_seq_fwd", dtype, ssm_state, k_state, v_state, y, x, k, q, alpha, beta, gamma, D, batch, T, nheads, headdim, d_state);
    if (rc) return rc;
    hipStream_t st = as_stream(stream);
    MRS_DISPATCH_DTYPE(dtype, T_, return launch_m3_seq<T_>(st, ssm_state, k_state, v_state, y, x, k, q, alpha, beta, gamma, D,
                                                           batch, T, nheads, headdim, d_state));
    return MRS_OK;
}

extern "C" int mrs_m3_step(void *stream, int dtype, float *ssm_state, float *k_state, float *v_state, void *y,
                           const void *x, const void *k_cur, const void *q_cur, const float *alpha,
                           const float *beta, const float *gamma, const float *D, int batch, int nheads,
                           int headdim, int d_state) {
    return mrs_m3_seq_fwd(stream, dtype, ssm_state, k_state, v_state, y, x, k_cur, q_cur, alpha, beta, gamma, D, batch, 1,
                          nheads, headdim, d_state);
}
