// Mamba-1 selective scan, one timestep (decode).
//
// Replaces ssm_step_forward_*, ssm_step_forward_gather_* and
// ssm_step_forward_gather_gate_* (kernels/mamba_ssm.cu:26-227).  The work is a
// read-modify-write of h [batch, d_inner, d_state] f32 -- 2*4*ds bytes per
// (b,d) against 3-4 activation elements -- so the kernel is laid out for the
// state stream: a group of LG = ds/4 lanes owns one (b,d) row and each lane
// moves one float4 of it, which makes every h access a fully coalesced 1 KiB
// wave transaction; the partial dot products are combined with lane shuffles.
#include "common.hpp"

namespace mrs {

// B and C of batch row b are read at xdbl + b*stride + {b_off, c_off}; the plain
// step passes stride = ds and separate base pointers.

// gate_mode: 0 none, 1 y *= gate, 2 y *= silu(gate); gate rows have gate_stride elements.
// dt_bias != nullptr: delta holds the raw dt_proj output and softplus(delta + dt_bias[d]) is applied here
// (dt_proj bias add + softplus_forward of the decode chain, src/mamba_ssm/gpu/inference.rs:1129-1158).
// Four consecutive elements as f32: one 8-byte (16-bit storage) or 16-byte (f32) load when the
// address is aligned for it (vec), four scalar loads otherwise.
template <typename T, bool VEC> __device__ __forceinline__ void ld4(const T *p, float (&o)[4]) {
    if constexpr (VEC) {
        struct alignas(4 * sizeof(T)) V { T v[4]; };
        const V t = *reinterpret_cast<const V *>(p);
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = Store<T>::ld(&t.v[i]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = Store<T>::ld(p + i);
    }
}

constexpr int kFoldMaxXd = 256;

// DT: where delta comes from -- 0: `delta` holds it; 1: dt_proj folded in, dt_w [dt_rank][d_inner]; 2: dt_proj folded
// in, dt_w transposed ([d_inner][dt_rank]) with dt_rank / LG a multiple of 4, so lane g takes the contiguous terms
// [g dt_rank/LG, (g+1) dt_rank/LG) of both operands as 4-element vectors.  VECBC: B/C rows may be read as aligned
// 4-element vectors.  Both are template parameters so that the body is straight-line code: with them as run-time flags
// the compiler fenced every group of loads with its own wait and the kernel was a chain of eight memory round trips
// (8.4 us at batch 64 against 4.2 us for the same state traffic without the folded dt_proj).
//
// FOLD: the x_proj row (dt input, B, C) has not been formed yet -- the in_proj launch before left its 16-column
// shares in fold.xpart [tile][row][xd] -- so each workgroup first sums the shares of its batch row, in tile order,
// rounds them to the storage type as the stored projection would be, and keeps the row in LDS.  A workgroup's 256 / LG
// channels lie in one batch row (d_inner is a multiple of that).
template <typename T, int LG, int DT, bool VECBC, bool FOLD = false, int PRE = 4>
__global__ __launch_bounds__(256) void ssm_step_kernel(
    float *__restrict__ h, T *__restrict__ y, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bbase, const T *__restrict__ Cbase, int64_t bc_stride,
    const T *__restrict__ gate, int64_t gate_stride, int gate_mode, const float *__restrict__ dt_bias,
    const T *__restrict__ dt_in, const T *__restrict__ dt_w, int dr,
    const float *__restrict__ a_neg, const float *__restrict__ Dp, int64_t total, int di, int ds, StepFold fold) {
    __shared__ alignas(16) T xs_l[FOLD ? kFoldMaxXd : 4];
    __shared__ alignas(16) float comb[FOLD ? 1024 : 4];
    // total = batch*d_inner rows; ds == 4*LG here.
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t rowi = gid / LG;
    const int g = (int)(gid % LG);
    const bool live = rowi < total;
    const int64_t r = live ? rowi : total - 1;
    const int b = (int)(r / di);
    const int d = (int)(r - (int64_t)b * di);
    // ---- every load that does not wait for another one, up front; the shares of the x_proj row first, since the
    // first thing computed is their sum ----
    float4 share[FOLD ? 8 : 1];
    int fold_G = 1, fold_tg = 0, fold_jq = 0;
    if constexpr (FOLD) {
        // thread (group tg, quad jq): 4 consecutive entries of the row over tiles tg, tg + G, ...: one round of 16-byte loads
        const int xq = fold.xd >> 2;
        fold_G = 256 / xq; fold_tg = (int)threadIdx.x / xq; fold_jq = (int)threadIdx.x - fold_tg * xq;
        const float *src = fold.xpart + (int64_t)b * fold.xd + 4 * fold_jq;
        const int64_t tstride = (int64_t)fold.rows * fold.xd;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int t = fold_tg + i * fold_G;
            share[i] = (fold_tg < fold_G && t < fold.n_tiles) ? *reinterpret_cast<const float4 *>(src + t * tstride) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    float4 hv = *reinterpret_cast<const float4 *>(h + r * ds + 4 * g);
    const float4 av = *reinterpret_cast<const float4 *>(a_neg + (int64_t)d * ds + 4 * g);
    const float uu = Store<T>::ld(u + r);
    const float Dd = Dp[d];
    // the optional operands are loaded on every path, from an address that is valid either way, and looked at only where
    // they apply: a value that is a load on one path and a preset on the other is copied into place once the load is
    // back, and the wait for that copy stood between these requests and the ones below (a round trip of its own)
    // (the stand-in address is one that nothing else here loads from: a load the compiler finds twice becomes a branch
    // around the other one again)
    const float bias = *(dt_bias ? dt_bias + d : Dp + (d + 1 < di ? d + 1 : 0));
    const float gz = Store<T>::ld(gate_mode != 0 ? gate + (int64_t)b * gate_stride + d : u + (r + 1 < total ? r + 1 : 0));
    float dl = 0.0f;
    if constexpr (DT == 0) dl = Store<T>::ld(delta + r);
    float Bv[4], Cv[4];
    if constexpr (!FOLD) {
        ld4<T, VECBC>(Bbase + (int64_t)b * bc_stride + 4 * g, Bv);
        ld4<T, VECBC>(Cbase + (int64_t)b * bc_stride + 4 * g, Cv);
    }
    const int kpl = DT == 2 ? dr / LG : 0;
    // DT 2: this lane's share of the weight row is requested here, with everything else that waits for nothing -- the
    // first 16 terms, or the first 48 (16-bit storage, d_state 16: a dt_rank of 160 over four lanes is 40 -- fetched inside
    // the loop below they were two more round trips behind the sum of the x_proj shares)
    // PRE = 12 costs 14 registers (a sixth wave per SIMD, which the 130m shape at 64 rows needs to run in one round), so
    // only a dt_rank that needs it takes that variant
    constexpr int kPre = PRE;   // groups of four terms
    struct alignas(4 * sizeof(T)) W4 { T v[4]; };
    W4 wq[kPre];
    if constexpr (DT == 2) {
        const T *wp = dt_w + (int64_t)d * dr + g * kpl;
#pragma unroll
        for (int cb = 0; cb < kPre / 4; cb++) {
            if (cb == 0 || 16 * cb < kpl) {   // the same for every lane; a narrow dt_rank asks for its one round only
#pragma unroll
                for (int j = 4 * cb; j < 4 * cb + 4; j++) wq[j] = *reinterpret_cast<const W4 *>(wp + (4 * j < kpl ? 4 * j : 0));
            }
        }
    }
    if constexpr (FOLD) {
        const int xd = fold.xd;
        if (fold_tg < fold_G) {
            float4 a = share[0];
#pragma unroll
            for (int i = 1; i < 8; i++) { a.x += share[i].x; a.y += share[i].y; a.z += share[i].z; a.w += share[i].w; }
            // more than 8 tiles per group (wide models): the rest in a second round
            const float *src = fold.xpart + (int64_t)b * xd + 4 * fold_jq;
            const int64_t tstride = (int64_t)fold.rows * xd;
            for (int t = fold_tg + 8 * fold_G; t < fold.n_tiles; t += fold_G) {
                const float4 v = *reinterpret_cast<const float4 *>(src + t * tstride);
                a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
            }
            *reinterpret_cast<float4 *>(&comb[fold_tg * xd + 4 * fold_jq]) = a;
        }
        lds_barrier();
        if ((int)threadIdx.x < xd) {
            float sum = 0.0f;
            for (int gg = 0; gg < fold_G; gg++) sum += comb[gg * xd + threadIdx.x];   // fixed order
            Store<T>::st(&xs_l[threadIdx.x], sum);
        }
        lds_barrier();
        ld4<T, true>(xs_l + fold.b_off + 4 * g, Bv);
        ld4<T, true>(xs_l + fold.c_off + 4 * g, Cv);
    }
    if constexpr (DT != 0) {
        // dt_proj folded in: delta_raw[b,d] = sum_r dt_in[b,r] * dt_w[r,d], the dt_rank terms split over the
        // LG lanes of the row (dt_proj GEMM of the decode chain, src/mamba_ssm/gpu/inference.rs:1129-1146)
        const T *xr = FOLD ? xs_l : dt_in + (int64_t)b * bc_stride;
        float part = 0.0f;
        if constexpr (DT == 2) {
            const T *xp = xr + g * kpl, *wp = dt_w + (int64_t)d * dr + g * kpl;
            // the prefetched groups, sixteen terms a round (the same order of additions as the loop behind them)
#pragma unroll
            for (int cb = 0; cb < kPre / 4; cb++) {
                const int c0 = 16 * cb;
                if (c0 < kpl) {
                    float xv[4][4];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const int kk = c0 + 4 * j;
                        const bool in = kk < kpl;
                        ld4<T, true>(xp + (in ? kk : 0), xv[j]);      // masked-off chunks read an in-range address
#pragma unroll
                        for (int i = 0; i < 4; i++) xv[j][i] = in ? xv[j][i] : 0.0f;
                    }
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int i = 0; i < 4; i++) part = fmaf(xv[j][i], Store<T>::ld(&wq[4 * cb + j].v[i]), part);
                }
            }
            for (int c0 = 4 * kPre; c0 < kpl; c0 += 16) {
                float xv[4][4], wv[4][4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int kk = c0 + 4 * j;
                    const bool in = kk < kpl;
                    ld4<T, true>(xp + (in ? kk : 0), xv[j]);
                    ld4<T, true>(wp + (in ? kk : 0), wv[j]);
#pragma unroll
                    for (int i = 0; i < 4; i++) xv[j][i] = in ? xv[j][i] : 0.0f;
                }
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int i = 0; i < 4; i++) part = fmaf(xv[j][i], wv[j][i], part);
            }
        } else {
            const T *wc = dt_w + d;
            // batches of 12 terms per lane with every load of a batch issued before the first multiply-add:
            // the loop is a latency chain otherwise (dt_rank 48 over 4 lanes = one batch)
            constexpr int kBatch = 12;
            for (int k0 = g; k0 < dr; k0 += kBatch * LG) {
                float xv[kBatch], wv[kBatch];
#pragma unroll
                for (int j = 0; j < kBatch; j++) {
                    const int k = k0 + j * LG;
                    const int kc = k < dr ? k : g;   // in-range address for the masked-off terms
                    xv[j] = Store<T>::ld(xr + kc);
                    wv[j] = Store<T>::ld(wc + (int64_t)kc * di);
                    xv[j] = k < dr ? xv[j] : 0.0f;
                }
#pragma unroll
                for (int j = 0; j < kBatch; j++) part = fmaf(xv[j], wv[j], part);
            }
        }
#pragma unroll
        for (int m = 1; m < LG; m <<= 1) part += __shfl_xor(part, m, kWave);
        dl = part;
    }
    if (dt_bias) dl = softplus20(dl + bias);
    const float du = dl * uu;
    const float x = dl * kLog2e;
    hv.x = fmaf(fast_exp2(x * av.x), hv.x, du * Bv[0]);
    hv.y = fmaf(fast_exp2(x * av.y), hv.y, du * Bv[1]);
    hv.z = fmaf(fast_exp2(x * av.z), hv.z, du * Bv[2]);
    hv.w = fmaf(fast_exp2(x * av.w), hv.w, du * Bv[3]);
    float acc = hv.x * Cv[0];
    acc = fmaf(hv.y, Cv[1], acc);
    acc = fmaf(hv.z, Cv[2], acc);
    acc = fmaf(hv.w, Cv[3], acc);
#pragma unroll
    for (int m = 1; m < LG; m <<= 1) acc += __shfl_xor(acc, m, kWave);
    if (live) {
        *reinterpret_cast<float4 *>(h + r * ds + 4 * g) = hv;
        if (g == 0) {
            acc = fmaf(Dd, uu, acc);
            if (gate_mode == 1) acc *= gz;
            if (gate_mode == 2) acc *= silu(gz);
            Store<T>::st(y + (fold.y_mt ? tiled_a_index(b, d, fold.y_mt) : r), acc);
        }
    }
}

// Any d_state (1..=256), one lane per (b,d), states streamed in order.
template <typename T>
__global__ __launch_bounds__(256) void ssm_step_generic_kernel(
    float *__restrict__ h, T *__restrict__ y, const T *__restrict__ delta, const T *__restrict__ u,
    const T *__restrict__ Bbase, const T *__restrict__ Cbase, int64_t bc_stride,
    const T *__restrict__ gate, int64_t gate_stride, int gate_mode, const float *__restrict__ dt_bias,
    const T *__restrict__ dt_in, const T *__restrict__ dt_w, int dr,
    const float *__restrict__ a_neg, const float *__restrict__ Dp, int64_t total, int di, int ds) {
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= total) return;
    const int b = (int)(r / di);
    const int d = (int)(r - (int64_t)b * di);
    float dl;
    if (dt_w) {
        dl = 0.0f;
        for (int k = 0; k < dr; k++) dl = fmaf(Store<T>::ld(dt_in + (int64_t)b * bc_stride + k), Store<T>::ld(dt_w + (int64_t)k * di + d), dl);
    } else {
        dl = Store<T>::ld(delta + r);
    }
    if (dt_bias) dl = softplus20(dl + dt_bias[d]);
    const float uu = Store<T>::ld(u + r);
    const float du = dl * uu;
    const float x = dl * kLog2e;
    float acc = Dp[d] * uu;
    float *hr = h + r * ds;
    const float *ar = a_neg + (int64_t)d * ds;
    const T *Br = Bbase + (int64_t)b * bc_stride;
    const T *Cr = Cbase + (int64_t)b * bc_stride;
    for (int n = 0; n < ds; n++) {
        const float hn = fmaf(fast_exp2(x * ar[n]), hr[n], du * Store<T>::ld(Br + n));
        hr[n] = hn;
        acc = fmaf(hn, Store<T>::ld(Cr + n), acc);
    }
    if (gate_mode == 1) acc *= Store<T>::ld(gate + (int64_t)b * gate_stride + d);
    if (gate_mode == 2) acc *= silu(Store<T>::ld(gate + (int64_t)b * gate_stride + d));
    Store<T>::st(y + r, acc);
}

template <typename T>
static int launch_step(hipStream_t st, float *h, void *y, const void *delta, const void *u,
                       const void *Bb, const void *Cb, int64_t bc_stride, const void *gate,
                       int64_t gate_stride, int gate_mode, const float *dt_bias, const void *dt_in,
                       const void *dt_w, int dr, int dt_transposed, const float *a_neg, const float *D, int batch, int di, int ds,
                       const StepFold *fold = nullptr, int y_mt = 0) {
    const int64_t total = (int64_t)batch * di;
    if (!gate) gate_mode = 0;
#define MRS_ARGS h, (T *)y, (const T *)delta, (const T *)u, (const T *)Bb, (const T *)Cb, bc_stride, \
                 (const T *)gate, gate_stride, gate_mode, dt_bias, (const T *)dt_in, (const T *)dt_w, dr, a_neg, D, total, di, ds
    const bool vec_ok = aligned(h, 16) && aligned(a_neg, 16);
    int lg = 0;
    if (vec_ok && (ds == 4 || ds == 8 || ds == 16 || ds == 32 || ds == 64 || ds == 128 || ds == 256)) lg = ds / 4;
    const size_t v4 = 4 * sizeof(T);
    const bool vec_bc = bc_stride % 4 == 0 && aligned(Bb, v4) && aligned(Cb, v4);
    int dt_mode = dt_w ? 1 : 0;
    if (dt_w && dt_transposed) {
        if (!(lg && dr % (4 * lg) == 0 && bc_stride % 4 == 0 && aligned(dt_in, v4) && aligned(dt_w, v4)))
            return fail(MRS_E_SHAPE, "ssm step: transposed dt_w needs d_state a power of two in 4..256, dt_rank %% d_state == 0 and 4-element aligned rows");
        dt_mode = 2;
    }
    if (lg) {
        const int64_t threads = total * lg;
        const int64_t blocks = (threads + 255) / 256;
        if (blocks > 0x7fffffffLL) return fail(MRS_E_SHAPE, "ssm step: grid too large");
        const dim3 grid((unsigned)blocks), block(256);
        if (fold) {
            // the row sits in LDS: offsets must suit the vector reads, every workgroup must lie inside one batch row
            if (!(fold->xpart && fold->xd >= 4 && fold->xd % 4 == 0 && fold->xd <= kFoldMaxXd && fold->rows == batch && di % (256 / lg) == 0 &&
                  dt_mode == 2 && fold->b_off % 4 == 0 && fold->c_off % 4 == 0 && fold->b_off + ds <= fold->xd && fold->c_off + ds <= fold->xd &&
                  dr <= fold->xd))
                return fail(MRS_E_SHAPE, "ssm step: folded x_proj needs xd <= %d, d_inner %% %d == 0, 4-aligned B/C offsets, transposed dt_w",
                            kFoldMaxXd, 256 / lg);
            StepFold folded = *fold;
            folded.y_mt = y_mt;
#define MRS_LGF(L) case L: hipLaunchKernelGGL((ssm_step_kernel<T, L, 2, true, true>), grid, block, 0, st, MRS_ARGS, folded); break
            if constexpr (sizeof(T) == 2) {
                if (lg == 4 && dr / lg > 16) {   // a wide dt_rank: the whole weight share requested up front
                    hipLaunchKernelGGL((ssm_step_kernel<T, 4, 2, true, true, 12>), grid, block, 0, st, MRS_ARGS, folded);
                    return check_launch("ssm_step_kernel");
                }
            }
            switch (lg) { MRS_LGF(1); MRS_LGF(2); MRS_LGF(4); MRS_LGF(8); MRS_LGF(16); MRS_LGF(32); MRS_LGF(64); }
#undef MRS_LGF
            return check_launch("ssm_step_kernel");
        }
        StepFold nofold = {};
        nofold.y_mt = y_mt;
        // (delta source, vector B/C): the transposed dt_w route implies vector rows (checked above)
        const int variant = dt_mode == 2 ? 4 : dt_mode * 2 + (vec_bc ? 1 : 0);
#define MRS_LGV(L, DT_, V_) hipLaunchKernelGGL((ssm_step_kernel<T, L, DT_, V_>), grid, block, 0, st, MRS_ARGS, nofold)
#define MRS_LG(L)                                   \
    case L:                                         \
        switch (variant) {                          \
            case 0: MRS_LGV(L, 0, false); break;    \
            case 1: MRS_LGV(L, 0, true); break;     \
            case 2: MRS_LGV(L, 1, false); break;    \
            case 3: MRS_LGV(L, 1, true); break;     \
            default: MRS_LGV(L, 2, true); break;    \
        }                                           \
        break
        switch (lg) { MRS_LG(1); MRS_LG(2); MRS_LG(4); MRS_LG(8); MRS_LG(16); MRS_LG(32); MRS_LG(64); }
#undef MRS_LG
#undef MRS_LGV
    } else {
        if (fold || y_mt) return fail(MRS_E_SHAPE, "ssm step: folded x_proj and tiled y need d_state a power of two in 4..256");
        const int64_t blocks = (total + 255) / 256;
        if (blocks > 0x7fffffffLL) return fail(MRS_E_SHAPE, "ssm step: grid too large");
        hipLaunchKernelGGL((ssm_step_generic_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st, MRS_ARGS);
    }
#undef MRS_ARGS
    return check_launch("ssm_step_kernel");
}

int launch_ssm_step_fused(hipStream_t st, int dtype, float *h, void *y, const void *delta, const float *dt_bias,
                          const void *dt_in, const void *dt_w, int dr, int dt_transposed,
                          const void *u, const void *Bb, const void *Cb, int64_t bc_stride, const void *gate,
                          int64_t gate_stride, int gate_mode, const float *a_neg, const float *D, int batch,
                          int di, int ds, const StepFold *fold, int y_mt) {
    MRS_DISPATCH_DTYPE(dtype, T_, return launch_step<T_>(st, h, y, delta, u, Bb, Cb, bc_stride, gate, gate_stride, gate_mode,
                                                         dt_bias, dt_in, dt_w, dr, dt_transposed, a_neg, D, batch, di, ds, fold, y_mt));
    return MRS_OK;
}

static int step_check(const char *fn, int dtype, const void *h, const void *y, const void *delta,
                      const void *u, const void *B, const void *C, const void *a_neg, const void *D,
                      int batch, int di, int ds) {
    if (dtype != MRS_F32 && dtype != MRS_F16 && dtype != MRS_BF16)
        return fail(MRS_E_DTYPE, "%s: dtype %d is not f32/f16/bf16", fn, dtype);
    if (!h || !y || !delta || !u || !B || !C || !a_neg || !D) return fail(MRS_E_NULL, "%s: null pointer", fn);
    if (batch < 1 || di < 1) return fail(MRS_E_SHAPE, "%s: batch=%d d_inner=%d must be >= 1", fn, batch, di);
    if (ds < 1 || ds > 256) return fail(MRS_E_SHAPE, "%s: d_state=%d outside 1..=256", fn, ds);
    if ((int64_t)batch * di * ds > 0x7fffffffLL) return fail(MRS_E_SHAPE, "%s: batch*d_inner*d_state exceeds i32", fn);
    return MRS_OK;
}

}  // namespace mrs

using namespace mrs;

extern "C" int mrs_ssm_step(void *stream, int dtype, float *h, void *y, const void *delta, const void *u,
                            const void *B, const void *C, const float *a_neg, const float *D,
                            int batch, int d_inner, int d_state) {
    int rc = step_check("mrs_ssm_step", dtype, h, y, delta, u, B, C, a_neg, D, batch, d_inner, d_state);
    if (rc) return rc;
    hipStream_t st = as_stream(stream);
    MRS_DISPATCH_DTYPE(dtype, T_, return launch_step<T_>(st, h, y, delta, u, B, C, d_state, nullptr, 0, 0, nullptr, nullptr, nullptr, 0, 0, a_neg, D, batch, d_inner, d_state));
    return MRS_OK;
}

extern "C" int mrs_ssm_step_gather_gate(void *stream, int dtype, float *h, void *y, const void *delta,
                                        const void *u, const void *xdbl, const void *gate_silu,
                                        const float *a_neg, const float *D, int batch, int d_inner,
                                        int d_state, int xdbl_stride, int b_offset, int c_offset) {
    int rc = step_check("mrs_ssm_step_gather_gate", dtype, h, y, delta, u, xdbl, xdbl, a_neg, D, batch, d_inner, d_state);
    if (rc) return rc;
    if (b_offset < 0 || c_offset < 0 || b_offset + d_state > xdbl_stride || c_offset + d_state > xdbl_stride)
        return fail(MRS_E_SHAPE, "mrs_ssm_step_gather_gate: offsets %d/%d + d_state %d exceed xdbl_stride %d",
                    b_offset, c_offset, d_state, xdbl_stride);
    const size_t es = (dtype == MRS_F32) ? 4 : 2;
    const char *xb = static_cast<const char *>(xdbl);
    hipStream_t st = as_stream(stream);
    MRS_DISPATCH_DTYPE(dtype, T_, return launch_step<T_>(st, h, y, delta, u, xb + es * b_offset, xb + es * c_offset,
                                                         xdbl_stride, gate_silu, d_inner, 1, nullptr, nullptr, nullptr, 0, 0, a_neg, D, batch, d_inner, d_state));
    return MRS_OK;
}
